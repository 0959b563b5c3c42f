"""GPU parity with bfloat16 activation storage, through the C ABI.

Activation tensors are bfloat16 in memory, parameters float, accumulation float; a result is rounded once when
stored. Forward and backward data multiply the filter rounded to bfloat16 (nearest even), so that every product
has two bfloat16 factors and can run on the bfloat16 matrix cores; the update acts on the float master copy. The checker computes the same layer on the same (bfloat16-valued)
inputs in double and the GPU result must lie within one bfloat16 unit in the last place of it
(util.assert_close_bf16). ReLU, max-pool and subtraction have exactly representable results: bit-exact.
"""
import numpy as np
import pytest

import oracle
import vdnn_implementation_amd.backend as be
from gpu_util import announce
from test_gpu_kernels import drawn_geometries
from util import assert_close, assert_close_bf16, from_bf16_bits, to_bf16_bits
from vdnn_implementation_amd.backend import check, lib

pytestmark = pytest.mark.gpu
BF16 = 1


@pytest.fixture(scope="module")
def ctx():
    c = be.Context(pool_bytes=4 << 30)
    check(lib.vdnn_ctx_set_activation_dtype(c.handle, BF16))
    assert lib.vdnn_ctx_activation_dtype(c.handle) == BF16
    yield c
    c.close()


@pytest.fixture(autouse=True)
def accurate_oracle():
    oracle.set_accumulate_double(True)
    yield
    oracle.set_accumulate_double(False)


class Dev:
    def __init__(self, ctx):
        self.ctx, self.bufs = ctx, []

    def act(self, a):
        """uploads a bfloat16-valued float32 array as bfloat16"""
        b = self.ctx.to_device(to_bf16_bits(a), np.uint16)
        self.bufs.append(b)
        return b

    def f32(self, a):
        b = self.ctx.to_device(a, np.float32)
        self.bufs.append(b)
        return b

    def empty_act(self, shape):
        b = self.ctx.alloc(max(int(np.prod(shape)) * 2, 4))
        self.bufs.append(b)
        return b

    def raw(self, nbytes):
        b = self.ctx.alloc(max(nbytes, 4))
        self.bufs.append(b)
        return b

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        for b in self.bufs:
            b.free()


def get_act(buf, shape):
    return from_bf16_bits(buf.download(shape, np.uint16))


def rnd(rng, shape, scale=1.0):
    return oracle.round_bf16((rng.standard_normal(shape) * scale).astype(np.float32))


def ws(d, g, algo, which):
    n = int(lib.vdnn_conv_workspace_bytes(g, algo, which))
    return (d.raw(n).ptr, n) if n else (None, 0)


def test_rounding_on_the_device_is_the_checkers(ctx):
    """Every store of a bfloat16 activation rounds a float on the device with the hardware's conversion; the checker
    rounds in integer arithmetic (nearest, ties to even, NaN stays NaN). bias_add on a tensor of zeros stores
    round(0 + b): ties, neighbours of ties, denormals, the largest finite value, infinities and random bit patterns
    must come back with the checker's bits."""
    rng = np.random.default_rng(5)
    edge = np.array([0x3F808000, 0x3F818000, 0x3F807FFF, 0x3F808001, 0x3F817FFF, 0x3F818001, 0x7F7FFFFF, 0x7F7F8000, 0x7F7F7FFF,
                     0x00000001, 0x00008000, 0x00008001, 0x00018000, 0x00017FFF, 0x007FFFFF, 0x00800000, 0x7F800000, 0x00000000,
                     0x7FC00000, 0x7FC12345, 0x7FFFFFFF], np.uint32)
    bits = np.concatenate([edge, edge | np.uint32(0x80000000), rng.integers(0, 2 ** 32, 60000, dtype=np.uint64).astype(np.uint32)])
    b = bits.view(np.float32)
    c = b.size
    announce("rounding to bf16 on the device, %d values" % c)
    with Dev(ctx) as d:
        y = d.act(np.zeros((1, c, 1, 1), np.float32))
        db = d.f32(b)
        check(lib.vdnn_bias_add(ctx.handle, None, 1, c, 1, db.ptr, y.ptr))
        got = y.download((c,), np.uint16)
    with np.errstate(invalid="ignore", over="ignore"):
        want = (oracle.round_bf16(np.float32(0) + b).view(np.uint32) >> 16).astype(np.uint16)
    nan = np.isnan(b)
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all(np.isnan(from_bf16_bits(got[nan])))
    # quiet NaNs keep their sign and the upper bits of their payload
    quiet = nan & ((bits & 0x00400000) != 0)
    assert np.array_equal(got[quiet], (bits[quiet] >> 16).astype(np.uint16))


CONV = [
    (3, 64, 28, 28, 64, 3, 3, 1, 1, 1, 1),     # blocked tap-major loaders, 64-row tile
    (2, 128, 14, 14, 256, 3, 3, 1, 1, 1, 1),   # two row tiles
    (2, 3, 32, 32, 64, 3, 3, 1, 1, 1, 1),      # three input channels: dense forward, vector-ALU backward passes
    (2, 70, 9, 13, 130, 3, 3, 1, 1, 1, 1),     # nothing divides the tiles; odd plane size (scalar dy loads)
    (2, 3, 67, 67, 96, 11, 11, 0, 0, 4, 4),    # AlexNet conv1: large window, stride 4
    (2, 48, 27, 27, 96, 5, 5, 2, 2, 1, 1),     # AlexNet conv2
    (5, 64, 6, 6, 200, 6, 6, 0, 0, 1, 1),      # OverFeat 6x6 -> 1x1
    (1, 16, 20, 24, 32, 3, 5, 1, 2, 2, 1),     # asymmetric, strided backward data
    # the bfloat16 matrix-core engine (reduced channels a multiple of 32):
    (6, 96, 27, 27, 160, 5, 5, 2, 2, 1, 1),    # 25 taps, three channel blocks, ragged row and column tiles
    (4, 32, 12, 20, 64, 3, 3, 1, 1, 2, 2),     # strided: the engine in forward and backward filter only
    (3, 64, 16, 22, 96, 3, 3, 0, 0, 1, 1),     # no padding, plane not a multiple of the slice
    (9, 256, 14, 14, 64, 3, 3, 1, 1, 1, 1),    # 14x14: three row wraps per slice in backward filter; forward splits its reduction
    (2, 64, 40, 36, 64, 1, 1, 0, 0, 1, 1),     # 1x1 window
    # the windowed 3x3 kernel (stride 1, padding 1, even rows): tiles of 256 pixels
    (2, 32, 5, 260, 64, 3, 3, 1, 1, 1, 1),     # rows longer than a tile: a tile starts and ends in the middle of a row
    (40, 64, 5, 2, 160, 3, 3, 1, 1, 1, 1),     # two-pixel rows: a tile spans 25 samples, every pixel touches both borders
    (3, 96, 56, 56, 128, 3, 3, 1, 1, 1, 1),    # three channel blocks, 128-row tiles, 36.75 tiles of pixels
    (44, 96, 56, 56, 64, 3, 3, 1, 1, 1, 1),    # 539 tiles on 512 places: the last 27 are split along the reduction (tail mode)
    # backward filter with one filter row and 64 input channels per workgroup (rows of whole 8-pixel groups, C % 64 == 0)
    (2, 64, 4, 32, 64, 3, 3, 1, 1, 1, 1),      # 64-row tile, one reduction split (results stored directly), rows one slice long
    (7, 128, 6, 32, 192, 3, 3, 1, 1, 1, 1),    # two channel blocks, a ragged second row tile, five splits that straddle samples, the last shorter
    (3, 64, 56, 56, 130, 3, 3, 1, 1, 1, 1),    # VGG-sized rows: a slice wraps an image row in the middle; two rows in the last tile
    (2, 192, 8, 40, 128, 3, 3, 1, 1, 1, 1),    # rows of five groups: slices start at every group of a row
    (2, 128, 12, 20, 192, 3, 3, 1, 1, 1, 1),   # rows of two and a half groups: every other row begins in the middle of a group
    (5, 64, 2, 16, 64, 3, 3, 1, 1, 1, 1),      # a slice covers a whole two-row sample: every row touches the upper or the lower border
    (3, 64, 6, 28, 96, 3, 3, 1, 1, 1, 1),      # 28-pixel rows, plane not a multiple of the slice: slices straddle samples
    (2, 96, 12, 20, 128, 3, 3, 1, 1, 1, 1),    # 96 channels: backward filter on the tile engine, four taps per tile, four pixels per load
    (2, 3, 11, 140, 32, 3, 3, 1, 1, 1, 1),     # three input channels: the streaming first-layer kernels, two backward-data column blocks
    (7, 3, 40, 36, 16, 3, 3, 1, 1, 1, 1),      # first layer: pixels that do not fill the last unit of 64, half a block of output channels
    (5, 2, 7, 9, 40, 3, 3, 1, 1, 1, 1),        # two input channels, rows shorter than a block of pixels, a ragged second block of output channels
]


@pytest.mark.parametrize("geom", CONV, ids=lambda g: "x".join(map(str, g)))
@pytest.mark.parametrize("algo", [0, 1])
def test_conv_bf16(ctx, geom, algo):
    rng = np.random.default_rng(hash(geom) % (2 ** 31) + 7)
    g, og = be.shape(*geom), oracle.shape(*geom)
    x = rnd(rng, (g.n, g.c, g.h, g.w))
    w = (rng.standard_normal((g.k, g.c, g.r, g.s)) * np.sqrt(2.0 / (g.c * g.r * g.s))).astype(np.float32)
    b = rng.standard_normal(g.k).astype(np.float32)
    wr = oracle.round_bf16(w)  # forward and backward data multiply the filter rounded to bfloat16
    want_y = oracle.conv_fwd(og, x, wr, b)
    dy = rnd(rng, want_y.shape)
    with Dev(ctx) as d:
        dx_, ddy, dw, db = d.act(x), d.act(dy), d.f32(w), d.f32(b)
        y, gx = d.empty_act(want_y.shape), d.empty_act(x.shape)
        announce("conv bf16", geom, "algo", algo, "fwd")
        p, n = ws(d, g, algo, 0)
        check(lib.vdnn_conv_fwd(ctx.handle, None, g, algo, dx_.ptr, dw.ptr, db.ptr, y.ptr, p, n))
        assert_close_bf16(get_act(y, want_y.shape), want_y, "fwd")
        announce("conv bf16", geom, "algo", algo, "bwd_data")
        p, n = ws(d, g, algo, 1)
        check(lib.vdnn_conv_bwd_data(ctx.handle, None, g, algo, ddy.ptr, dw.ptr, gx.ptr, p, n))
        assert_close_bf16(get_act(gx, x.shape), oracle.conv_bwd_data(og, dy, wr), "bwd data")
        # parameter gradients stay float: the float tolerance applies
        announce("conv bf16", geom, "algo", algo, "bwd_filter")
        gw = d.f32(np.zeros_like(w))
        p, n = ws(d, g, algo, 2)
        check(lib.vdnn_conv_bwd_filter(ctx.handle, None, g, algo, dx_.ptr, ddy.ptr, gw.ptr, p, n))
        assert_close(gw.download(w.shape), oracle.conv_bwd_filter_sgd(og, x, dy, np.zeros_like(w), 1.0), 1e-4, "bwd filter")
        announce("conv bf16", geom, "algo", algo, "bwd_bias")
        gb = d.f32(np.zeros_like(b))
        check(lib.vdnn_conv_bwd_bias(ctx.handle, None, g, ddy.ptr, gb.ptr))
        assert_close(gb.download(b.shape), oracle.conv_bwd_bias_sgd(og, dy, np.zeros_like(b), 1.0), 1e-4, "bwd bias")


@pytest.mark.parametrize("geom,inside", [
    ((7, 3, 40, 36, 16, 3, 3, 1, 1, 1, 1), True),      # first-layer kernel: the product's spare column multiplies dy by one
    ((2, 64, 4, 32, 64, 3, 3, 1, 1, 1, 1), True),      # filter-row kernel, one split
    ((7, 128, 6, 32, 192, 3, 3, 1, 1, 1, 1), True),    # two channel blocks, a ragged second row tile, several splits
    ((3, 64, 6, 28, 96, 3, 3, 1, 1, 1, 1), True),      # the variant with groups across image rows
    ((9, 256, 14, 14, 64, 3, 3, 1, 1, 1, 1), False),   # 14 x 14: the tile engine; the bias kernels run behind it
], ids=lambda v: "x".join(map(str, v)) if isinstance(v, tuple) else str(v))
def test_conv_bwd_filter_with_the_bias_gradient_bf16(ctx, geom, inside):
    """vdnn_conv_bwd_filter_bias_sgd / _bias with bfloat16 activations (layer.cu:631-660 in one call): the filter with
    the bits of the separate call, the bias gradient within the float tolerance, twice the same bits."""
    rng = np.random.default_rng(hash(geom) % (2 ** 31) + 13)
    g, og = be.shape(*geom), oracle.shape(*geom)
    assert bool(lib.vdnn_conv_bwd_filter_sums_bias(g, 0, BF16)) == inside
    x = rnd(rng, (g.n, g.c, g.h, g.w))
    w = (rng.standard_normal((g.k, g.c, g.r, g.s)) * np.sqrt(2.0 / (g.c * g.r * g.s))).astype(np.float32)
    b = rng.standard_normal(g.k).astype(np.float32)
    dy = oracle.round_bf16((rng.standard_normal((g.n, g.k, g.h, g.w)) + 0.25).astype(np.float32))
    alpha = np.float32(-0.37)
    announce("bwd filter + bias bf16", geom)
    with Dev(ctx) as d:
        dx_, ddy, dw, db = d.act(x), d.act(dy), d.f32(w), d.f32(b)
        check(lib.vdnn_conv_bwd_filter_bias_sgd(ctx.handle, None, g, 0, dx_.ptr, ddy.ptr, dw.ptr, db.ptr, alpha, None, 0))
        got_w, got_b = dw.download(w.shape), db.download(b.shape)
        assert_close(got_w, oracle.conv_bwd_filter_sgd(og, x, dy, w, alpha), 1e-4, "filter")
        assert_close(got_b, oracle.conv_bwd_bias_sgd(og, dy, b, alpha), 1e-4, "bias")
        dw2 = d.f32(w)
        check(lib.vdnn_conv_bwd_filter_sgd(ctx.handle, None, g, 0, dx_.ptr, ddy.ptr, dw2.ptr, alpha, None, 0))
        assert np.array_equal(dw2.download(w.shape), got_w)
        gw, gb = d.f32(np.full_like(w, 7.0)), d.f32(np.full_like(b, 7.0))
        check(lib.vdnn_conv_bwd_filter_bias(ctx.handle, None, g, 0, dx_.ptr, ddy.ptr, gw.ptr, gb.ptr, None, 0))
        got_db = gb.download(b.shape)
        assert_close(got_db, oracle.conv_bwd_bias_sgd(og, dy, np.zeros_like(b), 1.0), 1e-4, "db")
        check(lib.vdnn_conv_bwd_filter_bias(ctx.handle, None, g, 0, dx_.ptr, ddy.ptr, gw.ptr, gb.ptr, None, 0))
        assert np.array_equal(gb.download(b.shape), got_db)


@pytest.mark.parametrize("geom", drawn_geometries(6, 16), ids=lambda g: "x".join(map(str, g)))
@pytest.mark.parametrize("algo", [0, 1])
def test_conv_bf16_drawn_geometries(ctx, geom, algo):
    test_conv_bf16(ctx, geom, algo)


@pytest.mark.parametrize("n,cin,cout", [(128, 1000, 520), (64, 2304, 512), (5, 41, 33), (72, 264, 136), (128, 12544, 200), (40, 72, 1000)])
def test_fc_bf16(ctx, n, cin, cout):
    rng = np.random.default_rng(n + cin)
    x, dy = rnd(rng, (n, cin)), rnd(rng, (n, cout))
    w = (rng.standard_normal((cout, cin)) / np.sqrt(cin)).astype(np.float32)
    b = rng.standard_normal(cout).astype(np.float32)
    announce("fc bf16", n, cin, cout)
    with Dev(ctx) as d:
        dx_, ddy, dw, db = d.act(x), d.act(dy), d.f32(w), d.f32(b)
        y, gx, gw, gb = d.empty_act((n, cout)), d.empty_act((n, cin)), d.f32(np.zeros_like(w)), d.f32(np.zeros_like(b))
        check(lib.vdnn_fc_fwd(ctx.handle, None, n, cin, cout, dx_.ptr, dw.ptr, db.ptr, y.ptr))
        check(lib.vdnn_fc_bwd_data(ctx.handle, None, n, cin, cout, ddy.ptr, dw.ptr, gx.ptr))
        check(lib.vdnn_fc_bwd_weight(ctx.handle, None, n, cin, cout, dx_.ptr, ddy.ptr, gw.ptr))
        check(lib.vdnn_fc_bwd_bias(ctx.handle, None, n, cout, ddy.ptr, gb.ptr))
        assert_close_bf16(get_act(y, (n, cout)), oracle.fc_fwd(x, oracle.round_bf16(w), b), "fc fwd")
        assert_close_bf16(get_act(gx, (n, cin)), oracle.fc_bwd_data(dy, oracle.round_bf16(w)), "fc bwd data")
        assert_close(gw.download(w.shape), oracle.fc_bwd_weight_sgd(x, dy, np.zeros_like(w), 1.0), 1e-4, "fc dW")
        assert_close(gb.download(b.shape), oracle.fc_bwd_bias_sgd(dy, np.zeros_like(b), 1.0), 1e-4, "fc db")


@pytest.mark.parametrize("count", [1, 7, 4096 * 5 + 3])
def test_elementwise_bf16(ctx, count):
    rng = np.random.default_rng(count)
    x, dy = rnd(rng, count, 2.0), rnd(rng, count)
    x[: min(4, count)] = np.array([0.0, -0.0, np.inf, -1.0], np.float32)[: min(4, count)]
    announce("elementwise bf16", count)
    with Dev(ctx) as d:
        dx_, ddy, y, gx = d.act(x), d.act(dy), d.empty_act(count), d.empty_act(count)
        check(lib.vdnn_relu_fwd(ctx.handle, None, count, dx_.ptr, y.ptr))
        got_y = get_act(y, count)
        assert np.array_equal(got_y.view(np.uint32), oracle.relu_fwd(x).view(np.uint32))
        check(lib.vdnn_relu_bwd(ctx.handle, None, count, dx_.ptr, y.ptr, ddy.ptr, gx.ptr))
        assert np.array_equal(get_act(gx, count), oracle.relu_bwd(x, got_y, dy))
        check(lib.vdnn_relu_bwd(ctx.handle, None, count, None, y.ptr, ddy.ptr, gx.ptr))
        assert np.array_equal(get_act(gx, count), oracle.relu_bwd(x, got_y, dy))
        check(lib.vdnn_sub(ctx.handle, None, count, dx_.ptr, ddy.ptr, y.ptr))
        fin = np.isfinite(x)
        assert np.array_equal(get_act(y, count)[fin], oracle.round_bf16(x - dy)[fin])
        xs = np.where(fin, x, 1.0).astype(np.float32)
        dxs = d.act(xs)
        for name, fwd, bwd in (("tanh", oracle.tanh_fwd, oracle.tanh_bwd), ("sigmoid", oracle.sigmoid_fwd, oracle.sigmoid_bwd)):
            check(getattr(lib, "vdnn_%s_fwd" % name)(ctx.handle, None, count, dxs.ptr, y.ptr))
            gy = get_act(y, count)
            assert_close_bf16(gy, fwd(xs), name)
            check(getattr(lib, "vdnn_%s_bwd" % name)(ctx.handle, None, count, y.ptr, ddy.ptr, gx.ptr))
            assert_close_bf16(get_act(gx, count), bwd(gy, dy), name + " bwd")
        check(lib.vdnn_fill(ctx.handle, None, count, 0.3, y.ptr))
        assert np.all(get_act(y, count) == oracle.round_bf16(np.float32([0.3]))[0])


@pytest.mark.parametrize("n,c,h,w,win,stride", [(2, 8, 16, 16, 2, 2), (2, 5, 13, 13, 3, 2), (3, 4, 6, 10, 2, 2), (1, 3, 8, 12, 2, 2)])
def test_maxpool_bf16_is_exact(ctx, n, c, h, w, win, stride):
    rng = np.random.default_rng(h * w)
    g = be.shape(n, c, h, w, 0, win, win, 0, 0, stride, stride)
    og = oracle.shape(n, c, h, w, 0, win, win, 0, 0, stride, stride)
    x = rnd(rng, (n, c, h, w))
    want = oracle.maxpool_fwd(og, x)
    dy = rnd(rng, want.shape)
    announce("maxpool bf16", n, c, h, w, win, stride)
    with Dev(ctx) as d:
        dx_, ddy, y, gx = d.act(x), d.act(dy), d.empty_act(want.shape), d.empty_act(x.shape)
        check(lib.vdnn_maxpool_fwd(ctx.handle, None, g, dx_.ptr, y.ptr))
        assert np.array_equal(get_act(y, want.shape), want)
        check(lib.vdnn_maxpool_bwd(ctx.handle, None, g, dx_.ptr, y.ptr, ddy.ptr, gx.ptr))
        # overlapping windows add several dy: the sum is rounded once
        assert_close_bf16(get_act(gx, x.shape), oracle.maxpool_bwd(og, x, want, dy), "pool bwd", ulps=0.51)


def test_lrn_softmax_and_loss_bf16(ctx):
    rng = np.random.default_rng(3)
    x, dy = rnd(rng, (3, 24, 5, 7), 20.0), rnd(rng, (3, 24, 5, 7))
    announce("lrn bf16")
    with Dev(ctx) as d:
        dx_, ddy, y, gx = d.act(x), d.act(dy), d.empty_act(x.shape), d.empty_act(x.shape)
        check(lib.vdnn_lrn_fwd(ctx.handle, None, 3, 24, 35, dx_.ptr, y.ptr))
        gy = get_act(y, x.shape)
        assert_close_bf16(gy, oracle.lrn_fwd(x), "lrn fwd")
        check(lib.vdnn_lrn_bwd(ctx.handle, None, 3, 24, 35, dx_.ptr, y.ptr, ddy.ptr, gx.ptr))
        assert_close_bf16(get_act(gx, x.shape), oracle.lrn_bwd(x, gy, dy), "lrn bwd")
    n, classes = 6, 1000
    logits, dyl = rnd(rng, (n, classes), 3.0), rnd(rng, (n, classes))
    labels = rng.integers(0, classes, n).astype(np.int32)
    target = np.zeros((n, classes), np.float32)
    target[np.arange(n), labels] = 1.0
    announce("softmax bf16")
    with Dev(ctx) as d:
        dl, ddy, prob, gx, dt = d.act(logits), d.act(dyl), d.empty_act((n, classes)), d.empty_act((n, classes)), d.act(target)
        loss = d.f32(np.zeros(1, np.float32))
        check(lib.vdnn_softmax_fwd(ctx.handle, None, n, classes, dl.ptr, prob.ptr))
        gp = get_act(prob, (n, classes))
        assert_close_bf16(gp, oracle.softmax_fwd(logits), "softmax fwd")
        check(lib.vdnn_softmax_bwd(ctx.handle, None, n, classes, prob.ptr, ddy.ptr, gx.ptr))
        assert_close_bf16(get_act(gx, (n, classes)), oracle.softmax_bwd(gp, dyl), "softmax bwd")
        check(lib.vdnn_cross_entropy_dense(ctx.handle, None, n, classes, prob.ptr, dt.ptr, loss.ptr))
        want = float(np.mean(-np.log(gp[np.arange(n), labels].astype(np.float64))))
        assert abs(loss.download((1,))[0] - want) <= 1e-5 * abs(want)


def test_bf16_engine_in_a_split_last_round_agrees_with_two_half_batches(ctx):
    """VGG16's 14x14 layers at batch 128 on the bfloat16 engine: 784 tiles for 768 resident workgroups, the last 16
    split along the reduction. No CPU result is affordable at this size; convolution is independent per sample,
    so the two half batches (another launch geometry) must give the same values up to one rounding of the
    differently ordered float sums."""
    geom, half = (128, 512, 14, 14, 512, 3, 3, 1, 1, 1, 1), (64, 512, 14, 14, 512, 3, 3, 1, 1, 1, 1)
    g, gh = be.shape(*geom), be.shape(*half)
    rng = np.random.default_rng(31)
    x = rnd(rng, (128, 512, 14, 14))
    w = (rng.standard_normal((512, 512, 3, 3)) * np.sqrt(2.0 / 4608)).astype(np.float32)
    b = rng.standard_normal(512).astype(np.float32)
    dy = rnd(rng, (128, 512, 14, 14))
    with Dev(ctx) as d:
        dx_, ddy, dw, db = d.act(x), d.act(dy), d.f32(w), d.f32(b)
        y, gx = d.empty_act(x.shape), d.empty_act(x.shape)
        announce("bf16 engine, split last round, whole batch")
        check(lib.vdnn_conv_fwd(ctx.handle, None, g, 0, dx_.ptr, dw.ptr, db.ptr, y.ptr, None, 0))
        check(lib.vdnn_conv_bwd_data(ctx.handle, None, g, 0, ddy.ptr, dw.ptr, gx.ptr, None, 0))
        whole_y, whole_gx = get_act(y, x.shape), get_act(gx, x.shape)
        halves_y, halves_gx = [], []
        for i in range(2):
            hx, hdy = d.act(x[64 * i:64 * i + 64]), d.act(dy[64 * i:64 * i + 64])
            hy, hgx = d.empty_act((64, 512, 14, 14)), d.empty_act((64, 512, 14, 14))
            announce("bf16 engine, split last round, half", i)
            check(lib.vdnn_conv_fwd(ctx.handle, None, gh, 0, hx.ptr, dw.ptr, db.ptr, hy.ptr, None, 0))
            check(lib.vdnn_conv_bwd_data(ctx.handle, None, gh, 0, hdy.ptr, dw.ptr, hgx.ptr, None, 0))
            halves_y.append(get_act(hy, (64, 512, 14, 14))); halves_gx.append(get_act(hgx, (64, 512, 14, 14)))
    assert_close_bf16(whole_y, np.concatenate(halves_y), "forward, whole batch against two halves")
    assert_close_bf16(whole_gx, np.concatenate(halves_gx), "backward data, whole batch against two halves")
    # a few output elements against the definition in double, with the filter rounded to bfloat16
    wr = oracle.round_bf16(w).astype(np.float64)
    for (n, k, p, q) in ((0, 0, 0, 0), (127, 511, 13, 13), (77, 300, 6, 0), (127, 5, 0, 13)):
        acc = float(b[k])
        for r in range(3):
            for s_ in range(3):
                ih, iw = p - 1 + r, q - 1 + s_
                if 0 <= ih < 14 and 0 <= iw < 14:
                    acc += float(np.dot(x[n, :, ih, iw].astype(np.float64), wr[k, :, r, s_]))
        assert abs(whole_y[n, k, p, q] - acc) <= 2.0 ** -7 * max(abs(acc), 1e-3)


def test_conv_bf16_tensors_at_odd_element_offsets(ctx):
    """Activation tensors that start two bytes off a four-byte boundary (a view into a larger buffer): neither the pixel-pair
    loads of forward / backward data nor the eight-pixel loads of backward filter depend on the alignment of the tensor."""
    geom = (3, 64, 12, 16, 96, 3, 3, 1, 1, 1, 1)
    g, og = be.shape(*geom), oracle.shape(*geom)
    rng = np.random.default_rng(77)
    x = rnd(rng, (3, 64, 12, 16))
    w = (rng.standard_normal((96, 64, 3, 3)) * np.sqrt(2.0 / 576)).astype(np.float32)
    b = rng.standard_normal(96).astype(np.float32)
    dy = rnd(rng, (3, 96, 12, 16))
    wr = oracle.round_bf16(w)

    def shifted(d, a):
        """uploads `a` one element into a buffer that is one element longer"""
        bits = np.concatenate([np.zeros(1, np.uint16), to_bf16_bits(a).ravel()])
        buf = d.ctx.to_device(bits, np.uint16)
        d.bufs.append(buf)
        return buf.ptr + 2

    with Dev(ctx) as d:
        px, pdy, dw, db = shifted(d, x), shifted(d, dy), d.f32(w), d.f32(b)
        y, gx = d.raw(dy.size * 2 + 2), d.raw(x.size * 2 + 2)
        announce("conv bf16, tensors at odd element offsets")
        check(lib.vdnn_conv_fwd(ctx.handle, None, g, 0, px, dw.ptr, db.ptr, y.ptr + 2, None, 0))
        check(lib.vdnn_conv_bwd_data(ctx.handle, None, g, 0, pdy, dw.ptr, gx.ptr + 2, None, 0))
        gw = d.f32(np.zeros_like(w))
        check(lib.vdnn_conv_bwd_filter(ctx.handle, None, g, 0, px, pdy, gw.ptr, None, 0))
        got_y = from_bf16_bits(y.download((dy.size + 1,), np.uint16)[1:]).reshape(dy.shape)
        got_gx = from_bf16_bits(gx.download((x.size + 1,), np.uint16)[1:]).reshape(x.shape)
        assert_close_bf16(got_y, oracle.conv_fwd(og, x, wr, b), "fwd")
        assert_close_bf16(got_gx, oracle.conv_bwd_data(og, dy, wr), "bwd data")
        assert_close(gw.download(w.shape), oracle.conv_bwd_filter_sgd(og, x, dy, np.zeros_like(w), 1.0), 1e-4, "bwd filter")
