"""Full-size tensors against the CPU checker, through the C ABI.

The network tests at full size compare a policy with BASELINE: the same kernels on both sides. Here single launches
at the sizes of the benchmark configurations - VGG16's conv1_2 (64 -> 64 channels at 224 x 224: tensors of 1.6 GB at
batch 128, 3.3 GB at batch 256 and at batch 512 in bfloat16, beyond 2^31 bytes, where the reference's `int` byte counts
overflow: network.cu:1010-1040, layer.h:240), conv4_2 (512 -> 512 at 28 x 28), the first fully connected layer
(25088 -> 4096) and the ReLU / pooling launches on the largest tensor - are compared with the checker itself:

* forward and backward data are independent per sample: the device computes the whole batch, and samples 0, N/2 and
  N-1 are compared with the checker run on those samples alone;
* backward filter sums over the whole batch: blocks dW[k0:k0+4, c0:c0+4] are compared with the checker run over the
  whole batch on the four-channel slices of x and dy (its sums in double);
* ReLU is compared element by element over the whole tensor, pooling on the three samples.

Tolerances: 1e-4 relative (max |a-b| / max |b|) for float results and for parameter gradients; bfloat16 results within
one bfloat16 unit in the last place of the checker's double-precision value (util.assert_close_bf16); ReLU and pooling
bit-exact.
"""
from concurrent.futures import ThreadPoolExecutor

import numpy as np
import pytest

import oracle
import vdnn_implementation_amd.backend as be
from gpu_util import announce
from util import assert_close, assert_close_bf16, from_bf16_bits
from vdnn_implementation_amd.backend import check, lib

pytestmark = pytest.mark.gpu
TOL = 1e-4
THREADS = 16

# (batch, bfloat16 activations): the headline's batch, the batch whose tensors pass 2^31 bytes in float, config 5's
CONFIGS = [(128, False), (256, False), (512, True)]
IDS = ["b128-f32", "b256-f32", "b512-bf16"]


@pytest.fixture(scope="module")
def ctx():
    c = be.Context(pool_bytes=17 << 30)
    yield c
    check(lib.vdnn_ctx_set_activation_dtype(c.handle, 0))
    c.close()


@pytest.fixture(autouse=True)
def accurate_oracle():
    oracle.set_accumulate_double(True)
    oracle.set_threads(THREADS)
    yield
    oracle.set_accumulate_double(False)


class Tensor:
    """An activation tensor drawn on the host (standard normal; truncated to bfloat16 values when `bf16`), as the array
    that is uploaded: float32, or the 16-bit patterns."""

    def __init__(self, shape, seed, bf16, scale=1.0):
        self.shape, self.bf16 = tuple(int(v) for v in shape), bf16
        count = int(np.prod(self.shape))
        self.host = np.empty(count, np.uint16 if bf16 else np.float32)
        chunk = 1 << 24
        starts = list(range(0, count, chunk))

        def fill(i):
            lo, hi = starts[i], min(starts[i] + chunk, count)
            v = np.random.default_rng([seed, i]).standard_normal(hi - lo, dtype=np.float32)
            if scale != 1.0:
                v *= np.float32(scale)
            if bf16:
                self.host[lo:hi] = (v.view(np.uint32) >> 16).astype(np.uint16)   # truncation: a bfloat16 value
            else:
                self.host[lo:hi] = v

        with ThreadPoolExecutor(THREADS) as ex:
            list(ex.map(fill, range(len(starts))))
        self.host = self.host.reshape(self.shape)

    def values(self, index):
        """float32 values of host[index]"""
        part = np.ascontiguousarray(self.host[index])
        return from_bf16_bits(part) if self.bf16 else part


class Dev:
    def __init__(self, ctx):
        self.ctx, self.bufs = ctx, []

    def up(self, a):
        b = self.ctx.to_device(a, a.dtype)
        self.bufs.append(b)
        return b

    def empty(self, nbytes):
        b = self.ctx.alloc(max(int(nbytes), 4))
        self.bufs.append(b)
        return b

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.ctx.synchronize()
        for b in self.bufs:
            b.free()


def fetch(ctx, buf, first, shape, bf16):
    """Elements [first, first + prod(shape)) of a device tensor, as float32 values."""
    out = np.empty(shape, np.uint16 if bf16 else np.float32)
    off = int(first) * out.itemsize
    assert off + out.nbytes <= buf.nbytes
    check(lib.vdnn_memcpy_d2h(ctx.handle, out.ctypes.data, buf.ptr + off, out.nbytes))
    return from_bf16_bits(out) if bf16 else out


def compare_act(got, want, bf16, what):
    if bf16:
        assert_close_bf16(got, want, what)
    else:
        assert_close(got, want, TOL, what)


def workspace(d, g, algo, which):
    n = int(lib.vdnn_conv_workspace_bytes(g, algo, which))
    return (d.empty(n).ptr, n) if n else (None, 0)


CONVS = {"conv1_2": (64, 224, 64), "conv4_2": (512, 28, 512)}


@pytest.mark.parametrize("batch,bf16", CONFIGS, ids=IDS)
@pytest.mark.parametrize("layer", list(CONVS))
def test_convolution_passes_at_full_size(ctx, layer, batch, bf16):
    c, hw, k = CONVS[layer]
    geom = (batch, c, hw, hw, k, 3, 3, 1, 1, 1, 1)
    g = be.shape(*geom)
    check(lib.vdnn_ctx_set_activation_dtype(ctx.handle, 1 if bf16 else 0))
    rng = np.random.default_rng(batch + c)
    w = (rng.standard_normal((k, c, 3, 3)) * np.sqrt(2.0 / (c * 9))).astype(np.float32)
    b = rng.standard_normal(k).astype(np.float32)
    wr = oracle.round_bf16(w) if bf16 else w    # with bfloat16 activations forward / backward data multiply the rounded filter
    x = Tensor((batch, c, hw, hw), 11, bf16)
    dy = Tensor((batch, k, hw, hw), 12, bf16)
    samples = (0, batch // 2, batch - 1)
    one = oracle.shape(1, c, hw, hw, k, 3, 3, 1, 1, 1, 1)
    plane_in, plane_out = c * hw * hw, k * hw * hw
    print("[full size] %s batch %d %s: x %.2f GB, dy %.2f GB" % (layer, batch, "bf16" if bf16 else "f32", x.host.nbytes / 1e9, dy.host.nbytes / 1e9), flush=True)
    with Dev(ctx) as d:
        dx_, ddy, dw, db = d.up(x.host), d.up(dy.host), d.up(w), d.up(b)
        out = d.empty(max(x.host.nbytes, dy.host.nbytes))
        for algo in (0, 1):
            announce("full size", layer, geom, "bf16" if bf16 else "f32", "algo", algo, "fwd")
            p, n = workspace(d, g, algo, 0)
            check(lib.vdnn_conv_fwd(ctx.handle, None, g, algo, dx_.ptr, dw.ptr, db.ptr, out.ptr, p, n))
            for s in samples:
                want = oracle.conv_fwd(one, x.values(slice(s, s + 1)), wr, b)
                compare_act(fetch(ctx, out, s * plane_out, (1, k, hw, hw), bf16), want, bf16, "%s fwd sample %d algo %d" % (layer, s, algo))
            announce("full size", layer, geom, "bf16" if bf16 else "f32", "algo", algo, "bwd_data")
            p, n = workspace(d, g, algo, 1)
            check(lib.vdnn_conv_bwd_data(ctx.handle, None, g, algo, ddy.ptr, dw.ptr, out.ptr, p, n))
            for s in samples:
                want = oracle.conv_bwd_data(one, dy.values(slice(s, s + 1)), wr)
                compare_act(fetch(ctx, out, s * plane_in, (1, c, hw, hw), bf16), want, bf16, "%s bwd data sample %d algo %d" % (layer, s, algo))
        # both algorithm modes (with float activations the perf-optimal one is another kernel, with another split of the batch)
        got = {}
        for algo in (0, 1):
            announce("full size", layer, geom, "bf16" if bf16 else "f32", "algo", algo, "bwd_filter")
            gw = d.up(np.zeros_like(w))
            p, n = workspace(d, g, algo, 2)
            check(lib.vdnn_conv_bwd_filter(ctx.handle, None, g, algo, dx_.ptr, ddy.ptr, gw.ptr, p, n))
            got[algo] = gw.download(w.shape)
        four = oracle.shape(batch, 4, hw, hw, 4, 3, 3, 1, 1, 1, 1)
        for k0, c0 in ((0, 0), (k // 2 - 2, c // 2 + 4), (k - 4, c - 4)):
            xs = x.values((slice(None), slice(c0, c0 + 4)))
            dys = dy.values((slice(None), slice(k0, k0 + 4)))
            want = oracle.conv_bwd_filter_sgd(four, xs, dys, np.zeros((4, 4, 3, 3), np.float32), 1.0)
            for algo in (0, 1):
                assert_close(got[algo][k0:k0 + 4, c0:c0 + 4], want, TOL, "%s bwd filter block (%d, %d) algo %d" % (layer, k0, c0, algo))
        # the bias gradient reads the same dy: every channel against a float64 sum over the batch
        announce("full size", layer, geom, "bf16" if bf16 else "f32", "bwd_bias")
        gb = d.up(np.zeros_like(b))
        check(lib.vdnn_conv_bwd_bias(ctx.handle, None, g, ddy.ptr, gb.ptr))
        sums = np.zeros(k, np.float64)
        for s0 in range(0, batch, 16):
            sums += dy.values(slice(s0, s0 + 16)).sum(axis=(0, 2, 3), dtype=np.float64)
        assert_close(gb.download((k,)), sums, TOL, "%s bwd bias" % layer)
    check(lib.vdnn_ctx_set_activation_dtype(ctx.handle, 0))


@pytest.mark.parametrize("batch,bf16", CONFIGS, ids=IDS)
def test_first_fully_connected_layer_at_full_size(ctx, batch, bf16):
    cin, cout = 25088, 4096
    check(lib.vdnn_ctx_set_activation_dtype(ctx.handle, 1 if bf16 else 0))
    rng = np.random.default_rng(batch)
    w = (rng.standard_normal((cout, cin), dtype=np.float32) * np.float32(np.sqrt(2.0 / cin)))
    b = rng.standard_normal(cout).astype(np.float32)
    wr = oracle.round_bf16(w) if bf16 else w
    x, dy = Tensor((batch, cin), 21, bf16), Tensor((batch, cout), 22, bf16)
    rows = [0, batch // 2, batch - 1]
    announce("full size fc1", batch, cin, cout, "bf16" if bf16 else "f32")
    with Dev(ctx) as d:
        dx_, ddy, dw, db = d.up(x.host), d.up(dy.host), d.up(w), d.up(b)
        y, gx, gw = d.empty(batch * cout * 4), d.empty(batch * cin * 4), d.up(np.zeros((cout, cin), np.float32))
        check(lib.vdnn_fc_fwd(ctx.handle, None, batch, cin, cout, dx_.ptr, dw.ptr, db.ptr, y.ptr))
        check(lib.vdnn_fc_bwd_data(ctx.handle, None, batch, cin, cout, ddy.ptr, dw.ptr, gx.ptr))
        check(lib.vdnn_fc_bwd_weight(ctx.handle, None, batch, cin, cout, dx_.ptr, ddy.ptr, gw.ptr))
        want_y = oracle.fc_fwd(x.values(rows), wr, b)
        want_gx = oracle.fc_bwd_data(dy.values(rows), wr)
        for i, r in enumerate(rows):
            compare_act(fetch(ctx, y, r * cout, (cout,), bf16), want_y[i], bf16, "fc1 fwd row %d" % r)
            compare_act(fetch(ctx, gx, r * cin, (cin,), bf16), want_gx[i], bf16, "fc1 bwd data row %d" % r)
        got = gw.download((cout, cin))
        xs = x.values(slice(None))
        for k0 in (0, cout // 2 - 2, cout - 4):
            want = oracle.fc_bwd_weight_sgd(xs, dy.values((slice(None), slice(k0, k0 + 4))), np.zeros((4, cin), np.float32), 1.0)
            assert_close(got[k0:k0 + 4], want, TOL, "fc1 dW rows %d..%d" % (k0, k0 + 3))
    check(lib.vdnn_ctx_set_activation_dtype(ctx.handle, 0))


@pytest.mark.parametrize("batch,bf16", CONFIGS, ids=IDS)
def test_relu_and_pooling_on_the_largest_tensor(ctx, batch, bf16):
    """conv1_2's output (N x 64 x 224 x 224): ReLU forward / backward over the whole tensor, the 2 x 2 pooling layer
    behind it on three samples; all bit-exact."""
    c, hw = 64, 224
    check(lib.vdnn_ctx_set_activation_dtype(ctx.handle, 1 if bf16 else 0))
    x = Tensor((batch, c, hw, hw), 31, bf16)
    count = x.host.size
    es = x.host.itemsize
    samples = (0, batch // 2, batch - 1)
    g, og = be.shape(batch, c, hw, hw, 0, 2, 2, 0, 0, 2, 2), oracle.shape(1, c, hw, hw, 0, 2, 2, 0, 0, 2, 2)
    plane, plane_out = c * hw * hw, c * (hw // 2) * (hw // 2)
    announce("full size relu / pool", batch, "bf16" if bf16 else "f32", "%.2f GB" % (x.host.nbytes / 1e9))
    with Dev(ctx) as d:
        dx_ = d.up(x.host)
        y = d.empty(count * es)
        check(lib.vdnn_relu_fwd(ctx.handle, None, count, dx_.ptr, y.ptr))
        got = y.download(x.shape, x.host.dtype)
        # max(x, 0) on the stored patterns: a negative value (sign bit set) becomes +0
        sign = np.uint16(0x8000) if bf16 else np.uint32(0x80000000)
        bits = x.host if bf16 else x.host.view(np.uint32)
        got_bits = got if bf16 else got.view(np.uint32)
        step = 1 << 26
        flat_bits, flat_got = bits.reshape(-1), got_bits.reshape(-1)
        for lo in range(0, count, step):
            part = flat_bits[lo:lo + step]
            assert np.array_equal(flat_got[lo:lo + step], np.where(part & sign, 0, part).astype(part.dtype)), "relu fwd at %d" % lo
        # backward: dy is the tensor itself shifted by one sample, so every element has a different partner
        gxd = d.empty(count * es)
        dy_first = plane  # dy[i] = x[(i + plane) % count]: build it on the device side from two copies
        ddy = d.empty(count * es)
        check(lib.vdnn_memcpy_d2d_async(ctx.handle, ddy.ptr, dx_.ptr + dy_first * es, (count - dy_first) * es, None))
        check(lib.vdnn_memcpy_d2d_async(ctx.handle, ddy.ptr + (count - dy_first) * es, dx_.ptr, dy_first * es, None))
        check(lib.vdnn_relu_bwd(ctx.handle, None, count, dx_.ptr, y.ptr, ddy.ptr, gxd.ptr))
        for s in samples:
            xs = x.values(slice(s, s + 1))
            dys = x.values(slice((s + 1) % batch, (s + 1) % batch + 1))
            want = oracle.relu_bwd(xs, np.maximum(xs, 0), dys)
            assert np.array_equal(fetch(ctx, gxd, s * plane, (1, c, hw, hw), bf16).view(np.uint32), want.view(np.uint32)), "relu bwd sample %d" % s
        # pooling: forward of x, backward with dy = the first quarter of the shifted tensor
        py, pgx = d.empty(batch * plane_out * es), gxd
        check(lib.vdnn_maxpool_fwd(ctx.handle, None, g, dx_.ptr, py.ptr))
        check(lib.vdnn_maxpool_bwd(ctx.handle, None, g, dx_.ptr, py.ptr, ddy.ptr, pgx.ptr))
        for s in samples:
            xs = x.values(slice(s, s + 1))
            want_y = oracle.maxpool_fwd(og, xs)
            assert np.array_equal(fetch(ctx, py, s * plane_out, want_y.shape, bf16).view(np.uint32), want_y.view(np.uint32)), "pool fwd sample %d" % s
            dys = fetch(ctx, ddy, s * plane_out, want_y.shape, bf16)
            want_gx = oracle.maxpool_bwd(og, xs, want_y, dys)
            assert np.array_equal(fetch(ctx, pgx, s * plane, xs.shape, bf16).view(np.uint32), want_gx.view(np.uint32)), "pool bwd sample %d" % s
    check(lib.vdnn_ctx_set_activation_dtype(ctx.handle, 0))
