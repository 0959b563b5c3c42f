"""GPU parity of the fused-rectifier entry points and of networks that use them, through the C ABI.

A fused call must return the bits of the two calls it stands for (the layer, then vdnn_relu_fwd / vdnn_relu_bwd,
layer.cu:766-814): the rectifier is exact, so fusing it changes no rounding. The unfused calls themselves are
held against the CPU checker elsewhere; here a few cases are also checked against it directly.
"""
import numpy as np
import pytest

import oracle
import vdnn_implementation_amd.backend as be
from gpu_util import Dev, _workspace, announce, gpu_conv_bwd_data, gpu_conv_fwd
from test_gpu_network import run_steps, small_specs
from util import assert_close, to_bf16_bits
from vdnn_implementation_amd import (ALEXNET_LRN, BASELINE, OVERFEAT, VDNN_ALL, VDNN_CONV, VDNN_MEMORY_OPT_ALGO, VDNN_NONE,
                                     VDNN_PERF_OPT_ALGO, VGG16_128, enums)
from vdnn_implementation_amd.backend import check, lib
from vdnn_implementation_amd.network import Network

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = be.Context(pool_bytes=6 << 30)
    yield c
    c.close()


def relu(a):
    return np.where(a > 0, a, np.where(np.isnan(a), a, np.float32(0))).astype(np.float32)


FUSED_GEOMS = [
    (2, 64, 14, 14, 64, 3, 3, 1, 1, 1, 1),      # few tiles: the reduction is split, the rectifier sits in the reduction kernel
    (8, 128, 28, 28, 128, 3, 3, 1, 1, 1, 1),    # many tiles: the rectifier sits in the tile kernel's epilogue
    (2, 48, 27, 27, 96, 5, 5, 2, 2, 1, 1),      # AlexNet conv2 geometry
    (1, 16, 20, 24, 32, 3, 5, 1, 2, 2, 1),      # strided, asymmetric
    (2, 70, 9, 13, 130, 3, 3, 1, 1, 1, 1),      # nothing divides the tiles
    (5, 64, 6, 6, 200, 6, 6, 0, 0, 1, 1),       # window = input: the dense route
    (2, 3, 32, 32, 16, 3, 3, 1, 1, 1, 1),       # three input channels: backward data leaves its vector-ALU kernel when masked
]


@pytest.mark.parametrize("algo", [0, 1])
@pytest.mark.parametrize("geom", FUSED_GEOMS, ids=lambda g: "x".join(map(str, g)))
def test_conv_fused_rectifier_gives_the_bits_of_the_separate_calls(ctx, geom, algo):
    rng = np.random.default_rng(hash(geom) % (2 ** 31) + 7)
    g, og = be.shape(*geom), oracle.shape(*geom)
    x = relu(rng.standard_normal((g.n, g.c, g.h, g.w)).astype(np.float32))  # the input is itself a rectifier's output
    w = (rng.standard_normal((g.k, g.c, g.r, g.s)) * np.sqrt(2.0 / (g.c * g.r * g.s))).astype(np.float32)
    b = rng.standard_normal(g.k).astype(np.float32)
    announce("fused conv", geom, "algo", algo, "fwd")
    y = gpu_conv_fwd(ctx, g, x, w, b, algo=algo)
    with Dev(ctx) as d:
        dx_, dw_, db_ = d.up(x), d.up(w), d.up(b)
        yf = d.empty(y.shape)
        ws, nws = _workspace(d, g, algo, 0)
        check(lib.vdnn_conv_fwd_relu(ctx.handle, None, g, algo, dx_.ptr, dw_.ptr, db_.ptr, yf.ptr, ws, nws))
        got = yf.download(y.shape)
    assert np.array_equal(got.view(np.uint32), relu(y).view(np.uint32))
    assert_close(got, relu(oracle.conv_fwd(og, x, w, b)), 2e-5, "fused forward against the checker")
    announce("fused conv", geom, "algo", algo, "bwd_data")
    dy = rng.standard_normal(y.shape).astype(np.float32)
    with Dev(ctx) as d:
        a, bw, xm = d.up(dy), d.up(w), d.up(x)
        gx = d.empty(x.shape)
        ws, nws = _workspace(d, g, algo, 1)
        check(lib.vdnn_conv_bwd_data_relu(ctx.handle, None, g, algo, a.ptr, bw.ptr, xm.ptr, gx.ptr, ws, nws))
        got = gx.download(x.shape)
    want = oracle.conv_bwd_data(og, dy, w) * (x > 0)
    assert_close(got, want, 2e-5, "masked backward data against the checker")
    assert np.all(got[x <= 0] == 0)
    if g.c > 4:  # same kernel with and without the mask: same bits
        plain = gpu_conv_bwd_data(ctx, g, dy, w, algo=algo)
        assert np.array_equal(got.view(np.uint32), np.where(x > 0, plain, np.float32(0)).view(np.uint32))


def test_conv_fused_rectifier_in_a_split_last_round(ctx):
    """VGG16's 14x14 layers at batch 128: 784 tiles for 768 resident workgroups, the last 16 are split and
    summed by a kernel of their own, which then applies the rectifier / the mask."""
    geom = (128, 512, 14, 14, 512, 3, 3, 1, 1, 1, 1)
    g = be.shape(*geom)
    rng = np.random.default_rng(23)
    x = relu(rng.standard_normal((128, 512, 14, 14)).astype(np.float32))
    w = (rng.standard_normal((512, 512, 3, 3)) * np.sqrt(2.0 / 4608)).astype(np.float32)
    b = rng.standard_normal(512).astype(np.float32)
    announce("fused conv, split last round, fwd")
    y = gpu_conv_fwd(ctx, g, x, w, b)
    with Dev(ctx) as d:
        dx_, dw_, db_ = d.up(x), d.up(w), d.up(b)
        yf = d.empty(y.shape)
        check(lib.vdnn_conv_fwd_relu(ctx.handle, None, g, 0, dx_.ptr, dw_.ptr, db_.ptr, yf.ptr, None, 0))
        got = yf.download(y.shape)
    assert np.array_equal(got.view(np.uint32), relu(y).view(np.uint32))
    announce("fused conv, split last round, bwd_data")
    dy = rng.standard_normal(y.shape).astype(np.float32)
    plain = gpu_conv_bwd_data(ctx, g, dy, w)
    with Dev(ctx) as d:
        a, bw, xm = d.up(dy), d.up(w), d.up(x)
        gx = d.empty(x.shape)
        check(lib.vdnn_conv_bwd_data_relu(ctx.handle, None, g, 0, a.ptr, bw.ptr, xm.ptr, gx.ptr, None, 0))
        got = gx.download(x.shape)
    assert np.array_equal(got.view(np.uint32), np.where(x > 0, plain, np.float32(0)).view(np.uint32))


@pytest.mark.parametrize("n,cin,cout", [(4, 192, 20), (128, 4096, 1000), (32, 9216, 4096), (3, 37, 11)])
def test_fc_fused_rectifier_gives_the_bits_of_the_separate_calls(ctx, n, cin, cout):
    rng = np.random.default_rng(n * 1000 + cout)
    x = relu(rng.standard_normal((n, cin)).astype(np.float32))
    w = (rng.standard_normal((cout, cin)) * np.sqrt(2.0 / cin)).astype(np.float32)
    b = rng.standard_normal(cout).astype(np.float32)
    dy = rng.standard_normal((n, cout)).astype(np.float32)
    announce("fused fc", n, cin, cout)
    with Dev(ctx) as d:
        dx_, dw_, db_, ddy = d.up(x), d.up(w), d.up(b), d.up(dy)
        y, yf, gx, gxf = d.empty((n, cout)), d.empty((n, cout)), d.empty((n, cin)), d.empty((n, cin))
        check(lib.vdnn_fc_fwd(ctx.handle, None, n, cin, cout, dx_.ptr, dw_.ptr, db_.ptr, y.ptr))
        check(lib.vdnn_fc_fwd_relu(ctx.handle, None, n, cin, cout, dx_.ptr, dw_.ptr, db_.ptr, yf.ptr))
        check(lib.vdnn_fc_bwd_data(ctx.handle, None, n, cin, cout, ddy.ptr, dw_.ptr, gx.ptr))
        check(lib.vdnn_fc_bwd_data_relu(ctx.handle, None, n, cin, cout, ddy.ptr, dw_.ptr, dx_.ptr, gxf.ptr))
        y, yf, gx, gxf = y.download((n, cout)), yf.download((n, cout)), gx.download((n, cin)), gxf.download((n, cin))
    assert np.array_equal(yf.view(np.uint32), relu(y).view(np.uint32))
    assert np.array_equal(gxf.view(np.uint32), np.where(x > 0, gx, np.float32(0)).view(np.uint32))
    if n * cin * cout <= 2 ** 24:
        assert_close(yf, relu(oracle.fc_fwd(x, w, b)), 2e-5, "fused fc forward against the checker")
        assert_close(gxf, oracle.fc_bwd_data(dy, w) * (x > 0), 2e-5, "masked fc backward data against the checker")


@pytest.mark.parametrize("n,c,h,w,win,stride", [(2, 8, 16, 16, 2, 2), (3, 5, 13, 13, 3, 2), (2, 4, 12, 20, 2, 2), (1, 3, 9, 9, 3, 3),
                                                (1, 2, 130, 121, 3, 2)])
def test_maxpool_backward_masked_by_its_input(ctx, n, c, h, w, win, stride):
    rng = np.random.default_rng(h * 100 + win)
    x = relu(rng.standard_normal((n, c, h, w)).astype(np.float32))  # about half zeros: windows of zeros have ties
    g, og = be.shape(n, c, h, w, 0, win, win, 0, 0, stride, stride), oracle.shape(n, c, h, w, 0, win, win, 0, 0, stride, stride)
    y = oracle.maxpool_fwd(og, x)
    dy = rng.standard_normal(y.shape).astype(np.float32)
    announce("masked pool backward", n, c, h, w, win, stride)
    with Dev(ctx) as d:
        a, b, cdy = d.up(x), d.up(y), d.up(dy)
        gx, gxf = d.empty(x.shape), d.empty(x.shape)
        check(lib.vdnn_maxpool_bwd(ctx.handle, None, g, a.ptr, b.ptr, cdy.ptr, gx.ptr))
        check(lib.vdnn_maxpool_bwd_relu(ctx.handle, None, g, a.ptr, b.ptr, cdy.ptr, gxf.ptr))
        gx, gxf = gx.download(x.shape), gxf.download(x.shape)
    assert np.array_equal(gxf.view(np.uint32), np.where(x > 0, gx, np.float32(0)).view(np.uint32))
    assert np.array_equal(gxf, oracle.relu_bwd(x, x, oracle.maxpool_bwd(og, x, y, dy)))


def test_fused_entry_points_with_bfloat16_storage():
    """bfloat16 activations: the rectifier commutes with the rounding (it keeps signs and zero), so the fused
    call still returns the bits of the separate ones."""
    c = be.Context(pool_bytes=2 << 30)
    try:
        check(lib.vdnn_ctx_set_activation_dtype(c.handle, 1))
        geom = (4, 64, 14, 14, 128, 3, 3, 1, 1, 1, 1)
        g = be.shape(*geom)
        rng = np.random.default_rng(99)
        x = oracle.round_bf16(relu(rng.standard_normal((4, 64, 14, 14)).astype(np.float32)))
        w = (rng.standard_normal((128, 64, 3, 3)) * np.sqrt(2.0 / 576)).astype(np.float32)
        b = rng.standard_normal(128).astype(np.float32)
        dy = oracle.round_bf16(rng.standard_normal((4, 128, 14, 14)).astype(np.float32))
        announce("fused conv bf16")
        bufs = []
        def act(a):
            t = c.to_device(to_bf16_bits(a), np.uint16); bufs.append(t); return t
        def f32(a):
            t = c.to_device(a, np.float32); bufs.append(t); return t
        def empty(count):
            t = c.alloc(count * 2); bufs.append(t); return t
        dx_, dw_, db_, ddy = act(x), f32(w), f32(b), act(dy)
        y, yr, yf = empty(dy.size), empty(dy.size), empty(dy.size)
        gx, gxr, gxf = empty(x.size), empty(x.size), empty(x.size)
        check(lib.vdnn_conv_fwd(c.handle, None, g, 0, dx_.ptr, dw_.ptr, db_.ptr, y.ptr, None, 0))
        check(lib.vdnn_relu_fwd(c.handle, None, dy.size, y.ptr, yr.ptr))
        check(lib.vdnn_conv_fwd_relu(c.handle, None, g, 0, dx_.ptr, dw_.ptr, db_.ptr, yf.ptr, None, 0))
        check(lib.vdnn_conv_bwd_data(c.handle, None, g, 0, ddy.ptr, dw_.ptr, gx.ptr, None, 0))
        check(lib.vdnn_relu_bwd(c.handle, None, x.size, dx_.ptr, dx_.ptr, gx.ptr, gxr.ptr))
        check(lib.vdnn_conv_bwd_data_relu(c.handle, None, g, 0, ddy.ptr, dw_.ptr, dx_.ptr, gxf.ptr, None, 0))
        assert np.array_equal(yf.download((dy.size,), np.uint16), yr.download((dy.size,), np.uint16))
        assert np.array_equal(gxf.download((x.size,), np.uint16), gxr.download((x.size,), np.uint16))
        for t in bufs:
            t.free()
    finally:
        c.close()


CONVS = (enums.CONV, enums.FC_CONV)


def fusion_plan(specs, offloaded=()):
    """(producers, elided, gated, elided in backward) as the network derives them from its layer table and from the
    layers whose input is offloaded: a CONV / FC layer that gets its input back by prefetch does not mask by it"""
    prod, elided, gated, elided_bwd = set(), set(), set(), set()
    for l in range(1, len(specs)):
        if specs[l].type != enums.RELU or specs[l - 1].type not in CONVS + (enums.FC_GEMM,):
            continue
        prod.add(l - 1); elided.add(l)
        if l + 1 < len(specs):
            t = specs[l + 1].type
            if t != enums.POOL and (l + 1) in offloaded:
                continue
            if (t in CONVS and specs[l + 1].c > 4) or t in (enums.FC_GEMM, enums.POOL):
                gated.add(l + 1); elided_bwd.add(l)
    return prod, elided, gated, elided_bwd


def assert_fused_matches(fused, plain, specs, what, offloaded=()):
    prod, elided, gated, _ = fusion_plan(specs, offloaded)
    assert prod, "the table has nothing to fuse"
    eq = lambda x, y: np.array_equal(x.view(np.uint32), y.view(np.uint32))
    assert [x.tobytes() for x in fused["loss"]] == [x.tobytes() for x in plain["loss"]], what + ": loss"
    for s in range(len(plain["loss"])):
        for l in range(len(specs)):
            # a producer's output is the rectified tensor, a masked layer's input gradient the ReLU's
            want_dst = plain["dsts"][s][l + 1] if l in prod else plain["dsts"][s][l]
            want_grad = plain["grads"][s][l - 1] if l in gated else plain["grads"][s][l]
            assert eq(fused["dsts"][s][l], want_dst), "%s: step %d output of layer %d" % (what, s, l)
            assert eq(fused["grads"][s][l], want_grad), "%s: step %d gradient of layer %d" % (what, s, l)
    for i, ((wa, ba), (wb, bb)) in enumerate(zip(fused["params"], plain["params"])):
        assert eq(wa, wb) and eq(ba, bb), "%s: params %d" % (what, i)
    assert eq(fused["input"], plain["input"]), what + ": input after the step"


@pytest.mark.parametrize("cnn,batch,algo,bf16", [(None, 4, VDNN_MEMORY_OPT_ALGO, False), (ALEXNET_LRN, 4, VDNN_MEMORY_OPT_ALGO, False),
                                                 (OVERFEAT, 3, VDNN_MEMORY_OPT_ALGO, False), (VGG16_128, 2, VDNN_PERF_OPT_ALGO, False),
                                                 (VGG16_128, 2, VDNN_MEMORY_OPT_ALGO, True)])
def test_networks_with_fused_rectifiers_keep_every_bit(cnn, batch, algo, bf16):
    def make(policy, **kw):
        if cnn is None:
            return Network(layers=small_specs(batch), policy=policy, algo=algo, capture=True, seed=3, bf16=bf16, **kw)
        return Network(cnn, policy, algo, batch, capture=True, seed=3, bf16=bf16, **kw)

    announce("fused networks", cnn, batch, "BASELINE unfused")
    with make(BASELINE) as net:
        plain = run_steps(net, 2)
        specs = list(net.specs)
        plain_peak = net.stats()["peak_bytes_in_use"]
    assert all(np.isfinite(v) for v in plain["loss"])
    for policy, kw in ((BASELINE, {}), (VDNN_NONE, {}), (VDNN_CONV, {}), (VDNN_ALL, {}), (VDNN_ALL, {"host_sync": True}),
                       (VDNN_CONV, {"refined": True}), (VDNN_ALL, {"refined": True}),
                       (VDNN_ALL, {"refined": True, "offload_lag": 6, "prefetch_depth": 3}),
                       (VDNN_CONV, {"offload_lag": 3, "prefetch_depth": 2}), (VDNN_ALL, {"unfused_optimizer": True})):
        announce("fused networks", cnn, batch, "policy", policy, kw)
        with make(policy, fuse=True, **kw) as net:
            got = run_steps(net, 2)
            peak = net.stats()["peak_bytes_in_use"]
            offloaded = {l for l in range(net.num_layers) if net.is_offloaded(l)}
        assert_fused_matches(got, plain, specs, "policy %d %s" % (policy, kw), offloaded)
        if policy == BASELINE:
            assert peak < plain_peak  # the elided layers own no output tensor
