"""Pins the CPU checker's layer math: torch-CPU golden fixtures, brute force, closed forms,
adjoint identities. No GPU."""
import numpy as np
import pytest

import oracle
from util import assert_close, golden, rel_err, shape_from_geom

CONV = ["vgg_3x3_p1", "alex_11x11_s4", "alex_5x5_p2", "overfeat_5x5_p0", "overfeat_6x6_to_1x1",
        "overfeat_1x1", "odd_3x3_s2_p1"]
TOL = 2e-6  # fp32 accumulation over <= 400 terms against float64 expectations


@pytest.fixture(params=[False, True], ids=["acc32", "acc64"])
def acc(request):
    oracle.set_accumulate_double(request.param)
    yield request.param
    oracle.set_accumulate_double(False)


@pytest.mark.parametrize("name", CONV)
def test_conv_against_torch(name, acc):
    f = golden("conv_" + name)
    g = shape_from_geom(oracle, f["geom"])
    assert oracle.conv_out_shape(g) == f["y"].shape
    assert_close(oracle.conv_fwd(g, f["x"], f["w"], f["b"]), f["y"], TOL, "fwd")
    assert_close(oracle.conv_bwd_data(g, f["dy"], f["w"]), f["dx"], TOL, "bwd data")
    # the reference fuses SGD into the filter and bias gradients: w + alpha * dW
    alpha = np.float32(-0.37)
    assert_close(oracle.conv_bwd_filter_sgd(g, f["x"], f["dy"], f["w"], alpha), f["w"] + alpha * f["dw"], TOL, "bwd filter")
    assert_close(oracle.conv_bwd_bias_sgd(g, f["dy"], f["b"], alpha), f["b"] + alpha * f["db"], TOL, "bwd bias")


@pytest.mark.parametrize("name", CONV)
def test_conv_brute_force_agrees(name):
    f = golden("conv_" + name)
    g = shape_from_geom(oracle, f["geom"])
    assert_close(oracle.conv_fwd(g, f["x"], f["w"], f["b"], brute=True), f["y"], 1e-6, "brute fwd")
    assert_close(oracle.conv_bwd_data(g, f["dy"], f["w"], brute=True), f["dx"], 1e-6, "brute bwd data")
    assert_close(oracle.conv_bwd_filter_brute(g, f["x"], f["dy"]), f["dw"], 1e-6, "brute bwd filter")


@pytest.fixture
def blocked():
    oracle.set_blocked_gemm(True)
    yield
    oracle.set_blocked_gemm(False)


@pytest.mark.parametrize("name", [n for n in CONV if "_s4" not in n and "_s2" not in n])
def test_blocked_gemm_convolutions_against_torch(name, blocked):
    """The im2col + blocked-SGEMM route (what the CPU baseline times) on the stride-1 fixtures: the same torch
    expectations, the tolerance of float accumulation in another order."""
    f = golden("conv_" + name)
    g = shape_from_geom(oracle, f["geom"])
    assert_close(oracle.conv_fwd(g, f["x"], f["w"], f["b"]), f["y"], 5e-6, "fwd")
    assert_close(oracle.conv_bwd_data(g, f["dy"], f["w"]), f["dx"], 5e-6, "bwd data")
    alpha = np.float32(-0.37)
    assert_close(oracle.conv_bwd_filter_sgd(g, f["x"], f["dy"], f["w"], alpha), f["w"] + alpha * f["dw"], 5e-6, "bwd filter")


@pytest.mark.parametrize("geom", [(3, 5, 9, 20, 7, 3, 3, 1, 1, 1, 1),     # nothing divides the 6 x 16 tiles
                                  (2, 70, 14, 14, 130, 3, 3, 1, 1, 1, 1),  # several reduction blocks, rows shorter than a strip
                                  (5, 16, 40, 36, 33, 3, 3, 1, 1, 1, 1),   # more than one pixel block per sample
                                  (2, 6, 11, 13, 9, 5, 4, 2, 0, 1, 1),     # asymmetric window and padding
                                  (4, 8, 10, 12, 12, 3, 3, 1, 1, 2, 1)])   # strided: falls back to the direct loops
def test_blocked_gemm_convolutions_against_the_direct_loops(geom, blocked):
    rng = np.random.default_rng(sum(geom))
    g = oracle.shape(*geom)
    x = rng.standard_normal((g.n, g.c, g.h, g.w)).astype(np.float32)
    w = rng.standard_normal((g.k, g.c, g.r, g.s)).astype(np.float32)
    b = rng.standard_normal(g.k).astype(np.float32)
    got_y = oracle.conv_fwd(g, x, w, b)
    dy = rng.standard_normal(got_y.shape).astype(np.float32)
    got = (got_y, oracle.conv_bwd_data(g, dy, w), oracle.conv_bwd_filter_sgd(g, x, dy, w, np.float32(0.5)))
    oracle.set_blocked_gemm(False)
    oracle.set_accumulate_double(True)
    try:
        want = (oracle.conv_fwd(g, x, w, b), oracle.conv_bwd_data(g, dy, w), oracle.conv_bwd_filter_sgd(g, x, dy, w, np.float32(0.5)))
    finally:
        oracle.set_accumulate_double(False)
    for a, e, what in zip(got, want, ("fwd", "bwd data", "bwd filter")):
        assert_close(a, e, 1e-5, what)


def test_conv_without_bias_and_zero_alpha():
    f = golden("conv_vgg_3x3_p1")
    g = shape_from_geom(oracle, f["geom"])
    y0 = oracle.conv_fwd(g, f["x"], f["w"], None)
    assert_close(y0 + f["b"][None, :, None, None], f["y"], TOL)
    assert np.array_equal(oracle.conv_bwd_filter_sgd(g, f["x"], f["dy"], f["w"], 0.0), f["w"])


@pytest.mark.parametrize("geom", [(2, 3, 8, 9, 4, 3, 3, 1, 1, 1, 1), (1, 2, 12, 11, 3, 5, 4, 2, 1, 2, 3),
                                  (2, 2, 9, 9, 3, 3, 3, 0, 0, 4, 4)])
def test_conv_adjoint_identities(geom):
    """<conv(x,w), dy> = <x, bwdData(dy,w)> = <w, bwdFilter(x,dy)> in float64 accumulation."""
    rng = np.random.default_rng(7)
    g = oracle.shape(*geom)
    oracle.set_accumulate_double(True)
    try:
        x = rng.standard_normal((g.n, g.c, g.h, g.w)).astype(np.float32)
        w = rng.standard_normal((g.k, g.c, g.r, g.s)).astype(np.float32)
        y = oracle.conv_fwd(g, x, w)
        dy = rng.standard_normal(y.shape).astype(np.float32)
        lhs = np.sum(y.astype(np.float64) * dy)
        dx = oracle.conv_bwd_data(g, dy, w)
        dw = oracle.conv_bwd_filter_sgd(g, x, dy, np.zeros_like(w), 1.0)
        assert abs(lhs - np.sum(x.astype(np.float64) * dx)) <= 1e-5 * abs(lhs) + 1e-4
        assert abs(lhs - np.sum(w.astype(np.float64) * dw)) <= 1e-5 * abs(lhs) + 1e-4
    finally:
        oracle.set_accumulate_double(False)


def test_out_dim_matches_the_network_tables():
    # extents the reference's tables state for the next layer (network.cu:156-813)
    assert oracle.out_dim(227, 0, 11, 4) == 55 and oracle.out_dim(55, 0, 3, 2) == 27
    assert oracle.out_dim(27, 2, 5, 1) == 27 and oracle.out_dim(27, 0, 3, 2) == 13 and oracle.out_dim(13, 0, 3, 2) == 6
    assert oracle.out_dim(231, 0, 11, 4) == 56 and oracle.out_dim(28, 0, 5, 1) == 24 and oracle.out_dim(6, 0, 6, 1) == 1
    assert oracle.out_dim(224, 1, 3, 1) == 224 and oracle.out_dim(224, 0, 2, 2) == 112


def test_fc_against_torch_and_numpy(acc):
    f = golden("fc")
    assert_close(oracle.fc_fwd(f["x"], f["w"], f["b"]), f["y"], TOL)
    assert_close(oracle.fc_bwd_data(f["dy"], f["w"]), f["dx"], TOL)
    alpha = np.float32(0.21)
    assert_close(oracle.fc_bwd_weight_sgd(f["x"], f["dy"], f["w"], alpha), f["w"] + alpha * f["dw"], TOL)
    assert_close(oracle.fc_bwd_bias_sgd(f["dy"], f["b"], alpha), f["b"] + alpha * f["db"], TOL)
    rng = np.random.default_rng(3)
    x = rng.standard_normal((5, 300)).astype(np.float32)
    w = rng.standard_normal((40, 300)).astype(np.float32)
    assert_close(oracle.fc_fwd(x, w), x.astype(np.float64) @ w.astype(np.float64).T, 2e-6)


def test_relu_against_torch_and_special_values():
    f = golden("relu")
    assert np.array_equal(oracle.relu_fwd(f["x"]), f["y"])
    assert np.array_equal(oracle.relu_bwd(f["x"], f["y"], f["dy"]), f["dx"])
    assert np.array_equal(oracle.relu_bwd(None, f["y"], f["dy"]), f["dx"])  # y > 0 selects the same set
    x = np.array([-0.0, 0.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45], np.float32)
    y = oracle.relu_fwd(x)
    assert np.array_equal(y[[0, 1, 2, 3, 5, 6]], np.array([0, 0, np.inf, 0, 1e-45, 0], np.float32))
    assert np.isnan(y[4])  # CUDNN_PROPAGATE_NAN (layer.cu:380-385)
    assert not np.signbit(y[0])
    dx = oracle.relu_bwd(x, y, np.ones_like(x))
    assert np.array_equal(dx, np.array([0, 0, 1, 0, 0, 1, 0], np.float32))


@pytest.mark.parametrize("name", ["pool_3x3_s2", "pool_2x2_s2", "pool_2x2_s2_odd"])
def test_maxpool_against_torch(name):
    f = golden(name)
    g = shape_from_geom(oracle, f["geom"])
    y = oracle.maxpool_fwd(g, f["x"])
    assert np.array_equal(y, f["y"])
    assert_close(oracle.maxpool_bwd(g, f["x"], y, f["dy"]), f["dx"], 1e-7)


def test_maxpool_tie_rule_and_nan():
    g = oracle.shape(1, 1, 4, 4, 0, 2, 2, 0, 0, 2, 2)
    x = np.zeros((1, 1, 4, 4), np.float32)  # every window is a four-way tie
    y = oracle.maxpool_fwd(g, x)
    dy = np.arange(1, 5, dtype=np.float32).reshape(1, 1, 2, 2)
    dx = oracle.maxpool_bwd(g, x, y, dy)
    want = np.zeros_like(x)
    want[0, 0, 0, 0], want[0, 0, 0, 2], want[0, 0, 2, 0], want[0, 0, 2, 2] = 1, 2, 3, 4  # first in row-major order
    assert np.array_equal(dx, want)
    x[0, 0, 0, 0] = np.nan
    x[0, 0, 1, 1] = 3.0
    assert oracle.maxpool_fwd(g, x)[0, 0, 0, 0] == 3.0  # NOT_PROPAGATE_NAN (layer.cu:419)
    # overlapping windows accumulate
    g3 = oracle.shape(1, 1, 5, 5, 0, 3, 3, 0, 0, 2, 2)
    x3 = np.zeros((1, 1, 5, 5), np.float32)
    x3[0, 0, 2, 2] = 9.0
    dx3 = oracle.maxpool_bwd(g3, x3, oracle.maxpool_fwd(g3, x3), np.ones((1, 1, 2, 2), np.float32))
    assert dx3[0, 0, 2, 2] == 4.0 and dx3.sum() == 4.0


@pytest.mark.parametrize("name", ["lrn", "lrn_large_inputs"])
def test_lrn_against_torch(name):
    f = golden(name)
    y = oracle.lrn_fwd(f["x"])
    assert_close(y, f["y"], 2e-6)
    assert_close(oracle.lrn_bwd(f["x"], f["y"], f["dy"]), f["dx"], 5e-6)


def test_lrn_finite_differences():
    rng = np.random.default_rng(11)
    x = (rng.standard_normal((1, 7, 2, 2)) * 40).astype(np.float32)
    dy = rng.standard_normal(x.shape).astype(np.float32)
    y = oracle.lrn_fwd(x)
    dx = oracle.lrn_bwd(x, y, dy)
    for idx in [(0, 0, 0, 0), (0, 3, 1, 0), (0, 6, 1, 1)]:
        h = 0.25
        xp, xm = x.copy(), x.copy()
        xp[idx] += h
        xm[idx] -= h
        fd = np.sum((oracle.lrn_fwd(xp).astype(np.float64) - oracle.lrn_fwd(xm)) * dy) / (2 * h)
        assert abs(fd - dx[idx]) <= 2e-3 * max(1.0, abs(fd))


def test_softmax_against_torch_and_invariants():
    f = golden("softmax")
    y = oracle.softmax_fwd(f["x"])
    assert_close(y, f["y"], 1e-6)
    assert np.allclose(y.sum(axis=1), 1.0, atol=1e-6)
    assert_close(oracle.softmax_fwd(f["x"] + 100.0), f["y"], 2e-5)  # shift invariance
    dx = oracle.softmax_bwd(f["y"], f["dy"])
    assert_close(dx, f["dx"], 2e-6)
    assert np.allclose(dx.sum(axis=1), 0.0, atol=1e-6)
    big = np.array([[1e4, 0.0, -1e4]], np.float32)  # ACCURATE mode: no overflow (layer.cu:826)
    assert np.array_equal(oracle.softmax_fwd(big), np.array([[1, 0, 0]], np.float32))


def test_softmax_ce_against_torch():
    f = golden("softmax_ce")
    prob, loss = oracle.softmax_ce_fwd(f["x"], f["labels"])
    assert_close(prob, f["prob"], 1e-6)
    assert abs(loss - f["loss"][0]) <= 1e-6 * abs(f["loss"][0])
    assert_close(oracle.softmax_ce_bwd(prob, f["labels"]), f["dx"], 2e-6)
    onehot = np.eye(f["x"].shape[1], dtype=np.float32)[f["labels"]]
    assert abs(oracle.cross_entropy_dense(prob, onehot) - loss) <= 1e-6


def test_sub():
    a = np.array([1.5, -2.0, 3.25], np.float32)
    b = np.array([0.5, 2.0, -1.0], np.float32)
    r = np.empty(3, np.float32)
    oracle.lib.orc_sub(3, oracle._p(a), oracle._p(b), oracle._p(r))
    assert np.array_equal(r, a - b)


_M64 = (1 << 64) - 1


def _mix64(z):
    z = (z + 0x9E3779B97F4A7C15) & _M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    return z ^ (z >> 31)


def _rng(seed, stream, i):
    return _mix64((_mix64(seed ^ _mix64(stream)) + i * 0x9E3779B97F4A7C15) & _M64)


def test_seeded_generator_is_pinned():
    # the mixer is splitmix64's output function: its published first output for state 0
    assert _mix64(0) == 0xE220A8397B1DCDAF
    for seed, stream, i in [(1234, 1, 0), (1234, 1, 1), (1234, 1, 2), (0, 0, 0), (2 ** 63, 101, 10 ** 12)]:
        assert oracle.lib.orc_rng_u64(seed, stream, i) == _rng(seed, stream, i)
    assert oracle.lib.orc_rng_u64(1234, 1, 0) == 0xA1DB23A44940BAA2
    # Box-Muller restated in numpy float64; libm and numpy may differ in the last bit of log/cos
    want = []
    for i in range(64):
        u1 = ((_rng(1234, 1, 2 * i) >> 11) + 0.5) / 2.0 ** 53
        u2 = ((_rng(1234, 1, 2 * i + 1) >> 11) + 0.5) / 2.0 ** 53
        want.append(np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2))
    got = oracle.fill_normal(64, 1234, 1)
    assert np.allclose(got, np.array(want), rtol=3e-7, atol=1e-7)
    assert got[:2].tolist() == [-0.7955732345581055, -1.840828776359558]
    assert oracle.fill_labels(6, 1234, 2, 1000).tolist() == [76, 552, 549, 713, 594, 75]
    assert [(_rng(1234, 2, i) >> 32) * 1000 >> 32 for i in range(6)] == [76, 552, 549, 713, 594, 75]
    n = oracle.fill_normal(400000, 99, 1)
    assert abs(n.mean()) < 5e-3 and abs(n.std() - 1.0) < 5e-3
    assert abs(((n - n.mean()) ** 3).mean()) < 2e-2 and abs(((n - n.mean()) ** 4).mean() - 3.0) < 5e-2
    assert np.array_equal(n[:1000], oracle.fill_normal(1000, 99, 1))  # element i depends on i only
    assert not np.array_equal(n[:1000], oracle.fill_normal(1000, 99, 2))
    u = oracle.fill_uniform(200000, 5, 3, -0.01, 0.01)
    assert u.min() >= -0.01 and u.max() <= 0.01 and abs(u.mean()) < 1e-4
    lab = oracle.fill_labels(100000, 5, 2, 1000)
    assert lab.min() >= 0 and lab.max() <= 999 and len(np.unique(lab)) == 1000
    he = oracle.fill_normal(300000, 5, 100, 0.0, float(np.sqrt(2.0 / 576)))
    assert abs(he.std() - np.sqrt(2.0 / 576)) < 2e-4


def test_tanh_and_sigmoid_against_torch_and_identities():
    import torch
    rng = np.random.default_rng(21)
    x = (rng.standard_normal(4099) * 3).astype(np.float32)
    dy = rng.standard_normal(4099).astype(np.float32)
    for fwd, bwd, ref in ((oracle.tanh_fwd, oracle.tanh_bwd, torch.tanh), (oracle.sigmoid_fwd, oracle.sigmoid_bwd, torch.sigmoid)):
        xt = torch.tensor(x.astype(np.float64), requires_grad=True)
        yt = ref(xt)
        yt.backward(torch.tensor(dy.astype(np.float64)))
        y = fwd(x)
        assert_close(y, yt.detach().numpy(), 1e-7, "forward")
        # backward is a function of the (float32) output, as the library call is handed y
        y64 = y.astype(np.float64)
        want = dy * (1 - y64 * y64) if ref is torch.tanh else dy * y64 * (1 - y64)
        assert_close(bwd(y, dy), want, 1e-7, "backward from y")
        assert_close(bwd(y, dy), xt.grad.numpy(), 1e-5, "backward against autograd")
    special = np.array([0.0, -0.0, np.inf, -np.inf, 200.0, -200.0], np.float32)
    assert np.array_equal(oracle.tanh_fwd(special), np.array([0, -0.0, 1, -1, 1, -1], np.float32))
    assert np.array_equal(oracle.sigmoid_fwd(special), np.array([0.5, 0.5, 1, 0, 1, 0], np.float32))
    assert np.isnan(oracle.tanh_fwd(np.array([np.nan], np.float32))[0]) and np.isnan(oracle.sigmoid_fwd(np.array([np.nan], np.float32))[0])
    assert np.array_equal(oracle.tanh_fwd(-x), -oracle.tanh_fwd(x))
    assert_close(oracle.sigmoid_fwd(x).astype(np.float64) + oracle.sigmoid_fwd(-x), np.ones_like(x), 1e-7, "sigmoid(x) + sigmoid(-x)")


def test_bf16_rounding_against_torch():
    import torch
    rng = np.random.default_rng(8)
    x = np.concatenate([
        (rng.standard_normal(20000) * 10.0 ** rng.integers(-30, 30, 20000)).astype(np.float32),
        np.array([0.0, -0.0, 1.0, np.inf, -np.inf, 3.4028235e38, 1e-45, -1e-40], np.float32),
        # exact ties: 1 + 2^-8 (even below: rounds down), 1 + 3*2^-8 (odd below: rounds up), and just past a tie
        np.array([1.00390625, 1.01171875, np.nextafter(np.float32(1.00390625), np.float32(2))], np.float32)])
    want = torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()
    got = oracle.round_bf16(x)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert got[-3] == 1.0 and got[-2] == np.float32(1.015625) and got[-1] == np.float32(1.0078125)
    assert np.isinf(oracle.round_bf16(np.array([3.4028235e38], np.float32))[0])
    n = oracle.round_bf16(np.array([np.nan], np.float32))
    assert np.isnan(n[0]) and not (n.view(np.uint32)[0] & 0xFFFF)
    assert np.array_equal(oracle.round_bf16(got).view(np.uint32), got.view(np.uint32))  # idempotent


def _drawn_small_geometries(seed, count):
    """Convolution geometries from a seeded generator, small enough for torch in float64 on the CPU: windows 1 to 5,
    strides 1 to 3, with and without padding, channel counts on both sides of the blocked GEMM's panel widths."""
    import random
    rnd = random.Random(seed)
    out = []
    while len(out) < count:
        n, c, k = rnd.randint(1, 4), rnd.choice([1, 2, 3, 5, 8, 16, 17, 33]), rnd.choice([1, 2, 4, 7, 16, 24, 40])
        r, s = rnd.choice([1, 2, 3, 3, 5]), rnd.choice([1, 2, 3, 3, 5])
        h, w = rnd.randint(r, 19), rnd.randint(s, 19)
        ph, pw = rnd.choice([0, r // 2, r - 1]), rnd.choice([0, s // 2, s - 1])
        sh, sw = rnd.choice([1, 1, 2, 3]), rnd.choice([1, 1, 2, 3])
        out.append((n, c, h, w, k, r, s, ph, pw, sh, sw))
    return out


@pytest.mark.parametrize("geom", _drawn_small_geometries(3, 24), ids=lambda g: "x".join(map(str, g)))
def test_conv_drawn_geometries_against_torch_autograd(geom, acc):
    """The checker's four convolution passes against torch's float64 convolution and its autograd on geometries drawn
    from a seeded generator (the fixtures hold seven hand-picked ones): asymmetric windows, strides that leave columns
    unread, paddings up to window - 1."""
    import torch
    n, c, h, w_, k, r, s, ph, pw, sh, sw = geom
    g = oracle.shape(*geom)
    rng = np.random.default_rng(sum(geom))
    x = rng.standard_normal((n, c, h, w_)).astype(np.float32)
    w = (rng.standard_normal((k, c, r, s)) / np.sqrt(c * r * s)).astype(np.float32)
    b = rng.standard_normal(k).astype(np.float32)
    xt = torch.tensor(x.astype(np.float64), requires_grad=True)
    wt = torch.tensor(w.astype(np.float64), requires_grad=True)
    bt = torch.tensor(b.astype(np.float64), requires_grad=True)
    yt = torch.nn.functional.conv2d(xt, wt, bt, stride=(sh, sw), padding=(ph, pw))
    dy = rng.standard_normal(tuple(yt.shape)).astype(np.float32)
    yt.backward(torch.tensor(dy.astype(np.float64)))
    assert oracle.conv_out_shape(g) == tuple(yt.shape)
    assert_close(oracle.conv_fwd(g, x, w, b), yt.detach().numpy(), TOL, "fwd")
    assert_close(oracle.conv_bwd_data(g, dy, w), xt.grad.numpy(), TOL, "bwd data")
    alpha = np.float32(0.5)
    assert_close(oracle.conv_bwd_filter_sgd(g, x, dy, w, alpha), w + alpha * wt.grad.numpy(), TOL, "bwd filter")
    assert_close(oracle.conv_bwd_bias_sgd(g, dy, b, alpha), b + alpha * bt.grad.numpy(), TOL, "bwd bias")


@pytest.mark.parametrize("case", [(2, 3, 9, 11, 2, 2), (1, 5, 13, 13, 3, 2), (3, 2, 8, 12, 2, 1), (2, 4, 7, 7, 3, 3), (1, 1, 6, 10, 3, 1)])
def test_maxpool_drawn_shapes_against_torch_autograd(case):
    """Unpadded max pooling with distinct values (no ties): forward and the gradient's route against torch."""
    import torch
    n, c, h, w_, win, stride = case
    g = oracle.shape(n, c, h, w_, 0, win, win, 0, 0, stride, stride)
    rng = np.random.default_rng(sum(case))
    x = rng.permutation(n * c * h * w_).astype(np.float32).reshape(n, c, h, w_) / 7.0
    xt = torch.tensor(x.astype(np.float64), requires_grad=True)
    yt = torch.nn.functional.max_pool2d(xt, win, stride)
    dy = rng.standard_normal(tuple(yt.shape)).astype(np.float32)
    yt.backward(torch.tensor(dy.astype(np.float64)))
    y = oracle.maxpool_fwd(g, x)
    assert np.array_equal(y, yt.detach().numpy().astype(np.float32))
    assert_close(oracle.maxpool_bwd(g, x, y, dy), xt.grad.numpy(), 1e-6, "bwd")
