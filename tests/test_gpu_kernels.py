"""GPU parity: every HIP kernel against the CPU checker, through the C ABI.

Tolerances: convolution and FC results are fp32 MFMA sums compared with the checker's float64
accumulation: relative error (max |a-b| / max |b|) <= 1e-4, the bound the hot path is specified to.
ReLU, max-pool, subtraction and fills are exact (bit-identical).
"""
import ctypes as C

import numpy as np
import pytest

import oracle
import vdnn_implementation_amd.backend as be
from gpu_util import Dev, announce, conv_shape, gpu_conv_bwd_bias, gpu_conv_bwd_data, gpu_conv_bwd_filter, gpu_conv_fwd
from util import assert_close, golden
from vdnn_implementation_amd.backend import check, lib

pytestmark = pytest.mark.gpu
TOL = 1e-4


@pytest.fixture(scope="module")
def ctx():
    c = be.Context(pool_bytes=6 << 30)
    yield c
    c.close()


@pytest.fixture(autouse=True)
def accurate_oracle():
    oracle.set_accumulate_double(True)
    yield
    oracle.set_accumulate_double(False)


@pytest.fixture
def winograd_variant():
    """The perf-optimal mode takes Winograd where it applies (its default is the split-bfloat16 kernels)."""
    before = lib.vdnn_conv_perf_variant(1)
    yield
    lib.vdnn_conv_perf_variant(before)


CONV_GOLDEN = ["vgg_3x3_p1", "alex_11x11_s4", "alex_5x5_p2", "overfeat_5x5_p0", "overfeat_6x6_to_1x1",
               "overfeat_1x1", "odd_3x3_s2_p1"]


@pytest.mark.parametrize("name", CONV_GOLDEN)
def test_conv_golden(ctx, name):
    f = golden("conv_" + name)
    g = conv_shape(f["geom"])
    announce("conv golden", name, "fwd")
    assert_close(gpu_conv_fwd(ctx, g, f["x"], f["w"], f["b"]), f["y"], TOL, "fwd")
    announce("conv golden", name, "bwd_data")
    assert_close(gpu_conv_bwd_data(ctx, g, f["dy"], f["w"]), f["dx"], TOL, "bwd data")
    alpha = np.float32(-0.37)
    announce("conv golden", name, "bwd_filter")
    assert_close(gpu_conv_bwd_filter(ctx, g, f["x"], f["dy"], f["w"], alpha), f["w"] + alpha * f["dw"], TOL, "bwd filter")
    announce("conv golden", name, "bwd_bias")
    assert_close(gpu_conv_bwd_bias(ctx, g, f["dy"], f["b"], alpha), f["b"] + alpha * f["db"], TOL, "bwd bias")


# (n, c, h, w, k, r, s, pad_h, pad_w, stride_h, stride_w): tile edges, several reduction slices, split reductions
CONV_RANDOM = [
    (3, 64, 28, 28, 64, 3, 3, 1, 1, 1, 1),     # VGG-like, M = 64 tile
    (2, 128, 14, 14, 256, 3, 3, 1, 1, 1, 1),   # M > 128: two row tiles
    (2, 3, 32, 32, 64, 3, 3, 1, 1, 1, 1),      # first layer: 27-deep reduction, 3-row backward-data
    (2, 70, 9, 13, 130, 3, 3, 1, 1, 1, 1),     # nothing divides the tiles
    (2, 3, 67, 67, 96, 11, 11, 0, 0, 4, 4),    # AlexNet conv1 geometry
    (2, 48, 27, 27, 96, 5, 5, 2, 2, 1, 1),     # AlexNet conv2 geometry
    (2, 40, 12, 12, 72, 5, 5, 0, 0, 1, 1),     # OverFeat conv2 geometry
    (5, 64, 6, 6, 200, 6, 6, 0, 0, 1, 1),      # OverFeat 6x6 -> 1x1
    (9, 300, 1, 1, 150, 1, 1, 0, 0, 1, 1),     # OverFeat 1x1 on 1x1
    (1, 16, 20, 24, 32, 3, 5, 1, 2, 2, 1),     # asymmetric everything
    (2, 4, 17, 19, 8, 3, 3, 1, 1, 2, 2),       # four input channels, strided: the vector-ALU filter gradient
    (3, 1, 9, 9, 12, 3, 3, 0, 0, 1, 1),        # one input channel, no padding
    (7, 3, 40, 36, 16, 3, 3, 1, 1, 1, 1),      # three input channels, several pixel chunks per sample
    # backward filter with one filter row and 64 input channels per workgroup (3x3, stride 1, padding 1, W % 4 == 0, C % 64 == 0)
    (2, 64, 4, 16, 64, 3, 3, 1, 1, 1, 1),      # 64-row tile, one reduction split (results stored directly), rows one slice long
    (7, 128, 6, 20, 192, 3, 3, 1, 1, 1, 1),    # two channel blocks, a ragged second row tile, splits that straddle samples, slices that straddle rows
    (3, 64, 56, 56, 130, 3, 3, 1, 1, 1, 1),    # VGG-sized rows; two rows in the last tile
    (3, 64, 6, 28, 96, 3, 3, 1, 1, 1, 1),      # plane not a multiple of the slice: slices straddle samples
    (3, 64, 6, 18, 96, 3, 3, 1, 1, 1, 1),      # rows of four and a half groups: every other row begins in the middle of a group
    (4, 64, 14, 14, 64, 3, 3, 1, 1, 1, 1),     # 14 x 14: rows shorter than a slice, two row wraps per slice
    (3, 2, 6, 20, 96, 3, 3, 1, 1, 1, 1),       # two input channels, 96 output channels (a ragged second row tile), slices that straddle samples
    (2, 3, 11, 140, 32, 3, 3, 1, 1, 1, 1),     # three input channels, rows wider than a backward-data column block, strips of eight and three rows
]


@pytest.mark.parametrize("geom", CONV_RANDOM, ids=lambda g: "x".join(map(str, g)))
def test_conv_random_against_oracle(ctx, geom):
    rng = np.random.default_rng(hash(geom) % (2 ** 31))
    g, og = be.shape(*geom), oracle.shape(*geom)
    x = rng.standard_normal((g.n, g.c, g.h, g.w)).astype(np.float32)
    w = (rng.standard_normal((g.k, g.c, g.r, g.s)) * np.sqrt(2.0 / (g.c * g.r * g.s))).astype(np.float32)
    b = rng.standard_normal(g.k).astype(np.float32)
    want_y = oracle.conv_fwd(og, x, w, b)
    announce("conv random", geom, "fwd")
    assert_close(gpu_conv_fwd(ctx, g, x, w, b), want_y, TOL, "fwd")
    dy = rng.standard_normal(want_y.shape).astype(np.float32)
    announce("conv random", geom, "bwd_data")
    assert_close(gpu_conv_bwd_data(ctx, g, dy, w), oracle.conv_bwd_data(og, dy, w), TOL, "bwd data")
    # compare gradients, not weights: alpha = 1 on a zero filter
    announce("conv random", geom, "bwd_filter")
    zero = np.zeros_like(w)
    assert_close(gpu_conv_bwd_filter(ctx, g, x, dy, zero, np.float32(1.0)), oracle.conv_bwd_filter_sgd(og, x, dy, zero, 1.0), TOL, "bwd filter")
    announce("conv random", geom, "bwd_filter sgd")
    got = gpu_conv_bwd_filter(ctx, g, x, dy, w, np.float32(-1e-5))
    assert_close(got, oracle.conv_bwd_filter_sgd(og, x, dy, w, -1e-5), 1e-6, "fused sgd")
    announce("conv random", geom, "bwd_bias")
    assert_close(gpu_conv_bwd_bias(ctx, g, dy, b, np.float32(-0.5)), oracle.conv_bwd_bias_sgd(og, dy, b, -0.5), TOL, "bwd bias")


def drawn_geometries(seed, count, budget=2.5e8):
    """Convolution geometries drawn from a seeded generator: channel counts around the kernels' tile and block sizes,
    windows of 1 to 5, strides, paddings, planes around the sizes the vector loaders distinguish; small enough
    (budget multiply-adds) for the checker."""
    import random
    rnd = random.Random(seed)
    channels = [1, 2, 3, 4, 8, 16, 24, 32, 48, 64, 64, 64, 96, 128, 128, 130, 192, 256]
    out = []
    while len(out) < count:
        n, c, k = rnd.randint(1, 6), rnd.choice(channels), rnd.choice(channels)
        if rnd.random() < 0.6:
            r = s = 3
        else:
            r, s = rnd.choice([1, 3, 5, 2]), rnd.choice([1, 3, 5, 2])
        h = rnd.choice([rnd.randint(r, 40), rnd.choice([4, 6, 7, 8, 12, 14, 16, 28, 56])])
        w = rnd.choice([rnd.randint(s, 40), rnd.choice([4, 8, 12, 14, 16, 20, 28, 32, 56, 64])])
        ph, pw = rnd.choice([0, r // 2, r // 2, r // 2]), rnd.choice([0, s // 2, s // 2, s // 2])
        sh = sw = 1
        if rnd.random() < 0.2:
            sh, sw = rnd.choice([1, 2]), rnd.choice([1, 2, 3])
        if h < r or w < s:
            continue
        p, q = (h + 2 * ph - r) // sh + 1, (w + 2 * pw - s) // sw + 1
        if p < 1 or q < 1 or n * c * k * r * s * p * q > budget:
            continue
        out.append((n, c, h, w, k, r, s, ph, pw, sh, sw))
    return out


@pytest.mark.parametrize("geom", drawn_geometries(5, 24), ids=lambda g: "x".join(map(str, g)))
def test_conv_drawn_geometries_against_oracle(ctx, geom):
    test_conv_random_against_oracle(ctx, geom)


PERF_OPT_GEOMS = [
    (3, 64, 28, 28, 64, 3, 3, 1, 1, 1, 1),
    (2, 128, 14, 14, 256, 3, 3, 1, 1, 1, 1),
    (2, 48, 27, 27, 96, 5, 5, 2, 2, 1, 1),
    (1, 16, 20, 24, 32, 3, 5, 1, 2, 2, 1),     # strided: forward packs, backward data does not
    (2, 3, 32, 32, 64, 3, 3, 1, 1, 1, 1),      # three input channels: only backward filter has a variant
    (128, 512, 28, 28, 512, 3, 3, 1, 1, 1, 1), # backward filter asks for more staging than the context owns
]


def winograd_workspace(geom, bwd, chunk_bytes=512 << 20):
    """Bytes the Winograd variant of the perf-optimal mode takes for forward (bwd False) or backward data, 0 where the
    variant does not apply: 3x3 / stride 1 / padding 1, at least 128 reduced channels (a multiple of 16), more than 64
    produced ones. The transformed filter (36 x rows x reduced), then the transformed input (reduced x 36 x Tpad) and
    output (rows x 36 x Tpad) of one chunk of samples, each rounded up to 256 bytes; Tpad = the chunk's 4x4 tiles rounded
    up to 128; chunks of equal size whose input + output stay within chunk_bytes."""
    n, c, h, w, k, r, s, ph, pw, sh, sw = geom
    rows, red = (c, k) if bwd else (k, c)
    if (r, s, ph, pw, sh, sw) != (3, 3, 1, 1, 1, 1) or red < 128 or red % 16 or rows <= 64 or h < 4 or w < 4:
        return 0
    per = ((h + 3) // 4) * ((w + 3) // 4)
    most = max(1, min(n, chunk_bytes // ((rows + red) * 36 * per * 4)))
    chunks = -(-n // most)
    nc = -(-n // chunks)
    tpad = -(-nc * per // 128) * 128
    up = lambda b: -(-b // 256) * 256
    return up(36 * rows * red * 4) + up(red * 36 * tpad * 4) + up(rows * 36 * tpad * 4)


def winograd_wgrad_applies(geom):
    """Backward filter as Winograd F(3x3, 4x4): 3x3 / stride 1 / padding 1, input channels a multiple of 128, more than
    64 output channels."""
    n, c, h, w, k, r, s, ph, pw, sh, sw = geom
    return (r, s, ph, pw, sh, sw) == (3, 3, 1, 1, 1, 1) and c % 128 == 0 and k > 64 and h >= 4 and w >= 4


@pytest.mark.parametrize("geom", PERF_OPT_GEOMS, ids=lambda g: "x".join(map(str, g)))
def test_conv_perf_opt_variants(ctx, geom, winograd_variant):
    """The workspace-using variants. Wide 3x3 layers run forward and backward data as Winograd F(4x4, 3x3): other sums,
    held to the tolerance against the checker (or, at sizes the checker cannot afford, against the workspace-free
    kernels). Elsewhere forward and backward data read a re-laid-out filter bank in the same reduction order and return
    the bits of the workspace-free kernels. Backward filter may split the reduction differently and is held to the
    tolerance."""
    rng = np.random.default_rng(hash(geom) % (2 ** 31) + 1)
    g, og = be.shape(*geom), oracle.shape(*geom)
    n, c, h, w_, k, r, s_ = geom[:7]
    filter_bytes = k * c * r * s_ * 4
    fwd_ok = r * s_ <= 32 and c % 16 == 0
    bwd_ok = c > 4 and geom[9] == 1 and geom[10] == 1 and r * s_ <= 32 and k % 16 == 0
    wino = winograd_workspace(geom, False), winograd_workspace(geom, True)
    assert lib.vdnn_conv_workspace_bytes(g, 0, 0) == lib.vdnn_conv_workspace_bytes(g, 0, 1) == lib.vdnn_conv_workspace_bytes(g, 0, 2) == 0
    assert lib.vdnn_conv_workspace_bytes(g, 1, 0) == (wino[0] or (filter_bytes if fwd_ok else 0))
    assert lib.vdnn_conv_workspace_bytes(g, 1, 1) == (wino[1] or (filter_bytes if bwd_ok else 0))
    # with bfloat16 activations the variant does not apply: the packed filter's size, as before
    assert lib.vdnn_conv_workspace_bytes_dtype(g, 1, 0, 1) == (filter_bytes if fwd_ok else 0)
    wino_filter = winograd_wgrad_applies(geom)
    if wino_filter:
        # the transformed input and output gradient of a chunk of samples and at least one partial result
        tpad = -(-((h + 3) // 4) * ((w_ + 3) // 4) // 128) * 128
        assert lib.vdnn_conv_workspace_bytes(g, 1, 2) >= (c + k) * 36 * tpad * 4 + 36 * k * c * 4
    else:
        assert lib.vdnn_conv_workspace_bytes(g, 1, 2) % filter_bytes == 0
    assert lib.vdnn_conv_workspace_bytes_dtype(g, 1, 2, 1) % filter_bytes == 0
    if geom[0] == 128:
        assert lib.vdnn_conv_workspace_bytes(g, 1, 2) > (64 << 20)
    x = rng.standard_normal((g.n, g.c, g.h, g.w)).astype(np.float32)
    w = (rng.standard_normal((g.k, g.c, g.r, g.s)) * np.sqrt(2.0 / (g.c * g.r * g.s))).astype(np.float32)
    b = rng.standard_normal(g.k).astype(np.float32)
    announce("conv perf-opt", geom, "fwd")
    y0, y1 = gpu_conv_fwd(ctx, g, x, w, b, algo=0), gpu_conv_fwd(ctx, g, x, w, b, algo=1)
    if wino[0]:
        assert_close(y1, y0, TOL, "fwd, Winograd against direct")
        assert not np.array_equal(y0, y1)
    else:
        assert np.array_equal(y0, y1)
    dy = rng.standard_normal(y0.shape).astype(np.float32)
    announce("conv perf-opt", geom, "bwd_data")
    d0, d1 = gpu_conv_bwd_data(ctx, g, dy, w, algo=0), gpu_conv_bwd_data(ctx, g, dy, w, algo=1)
    if wino[1]:
        assert_close(d1, d0, TOL, "bwd data, Winograd against direct")
        assert not np.array_equal(d0, d1)
    else:
        assert np.array_equal(d0, d1)
    announce("conv perf-opt", geom, "bwd_filter")
    zero = np.zeros_like(w)
    got = gpu_conv_bwd_filter(ctx, g, x, dy, zero, np.float32(1.0), algo=1)
    if n * c * h * w_ * k <= 2 ** 28:  # sizes the checker finishes in seconds
        assert_close(got, oracle.conv_bwd_filter_sgd(og, x, dy, zero, 1.0), TOL, "bwd filter")
        assert_close(y1, oracle.conv_fwd(og, x, w, b), TOL, "fwd")
        assert_close(d1, oracle.conv_bwd_data(og, dy, w), TOL, "bwd data")
    else:
        assert_close(got, gpu_conv_bwd_filter(ctx, g, x, dy, zero, np.float32(1.0), algo=0), TOL, "bwd filter, two split counts")


def drawn_perf_geometries(seed, count, budget=2.5e8):
    """Geometries for the perf-optimal mode's routes: channel counts at and beside the multiples of 16 / 64 / 128 its
    kernels ask for, mostly 3x3 / stride 1 / padding 1 with rows of whole and broken pixel groups, the rest other
    windows, strides and paddings."""
    import random
    rnd = random.Random(seed)
    channels = [3, 8, 16, 16, 32, 48, 64, 64, 65, 80, 96, 128, 128, 130, 144, 192, 256]
    out = []
    while len(out) < count:
        n, c, k = rnd.choice([1, 2, 3, 5, 9]), rnd.choice(channels), rnd.choice(channels)
        if rnd.random() < 0.6:
            r, s, ph, pw, sh, sw = 3, 3, 1, 1, 1, 1
            h, w = rnd.choice([4, 6, 7, 12, 14, 16, 28]), rnd.choice([4, 6, 8, 10, 13, 14, 16, 18, 20, 28, 36])
        else:
            r, s = rnd.choice([(1, 1), (1, 3), (2, 2), (3, 3), (3, 5), (5, 5), (4, 7)])
            ph, pw = rnd.choice([0, r // 2, r - 1]), rnd.choice([0, s // 2, s - 1])
            sh, sw = rnd.choice([(1, 1), (1, 1), (1, 1), (2, 2), (2, 1)])
            h, w = rnd.randint(max(1, r - 2 * ph), 30), rnd.randint(max(1, s - 2 * pw), 30)
        p, q = (h + 2 * ph - r) // sh + 1, (w + 2 * pw - s) // sw + 1
        if p < 1 or q < 1 or n * c * k * r * s * p * q > budget:
            continue
        out.append((n, c, h, w, k, r, s, ph, pw, sh, sw))
    return out


@pytest.mark.parametrize("variant", [0, 1], ids=["split-bf16", "winograd"])
@pytest.mark.parametrize("geom", drawn_perf_geometries(11, 20), ids=lambda g: "x".join(map(str, g)))
def test_conv_perf_opt_drawn_geometries_against_oracle(ctx, geom, variant):
    """Whatever kernels the perf-optimal mode picks for a drawn geometry, with the workspace it asks for: forward,
    backward data, backward filter applied to a filter, against the checker to the mode's tolerance."""
    before = lib.vdnn_conv_perf_variant(variant)
    try:
        rng = np.random.default_rng(hash(geom) % (2 ** 31) + 13)
        g, og = be.shape(*geom), oracle.shape(*geom)
        x = rng.standard_normal((g.n, g.c, g.h, g.w)).astype(np.float32)
        w = (rng.standard_normal((g.k, g.c, g.r, g.s)) * np.sqrt(2.0 / (g.c * g.r * g.s))).astype(np.float32)
        b = rng.standard_normal(g.k).astype(np.float32)
        announce("conv perf-opt drawn", geom, "fwd variant %d" % variant)
        want_y = oracle.conv_fwd(og, x, w, b)
        assert_close(gpu_conv_fwd(ctx, g, x, w, b, algo=1), want_y, TOL, "fwd")
        dy = rng.standard_normal(want_y.shape).astype(np.float32)
        announce("conv perf-opt drawn", geom, "bwd_data variant %d" % variant)
        assert_close(gpu_conv_bwd_data(ctx, g, dy, w, algo=1), oracle.conv_bwd_data(og, dy, w), TOL, "bwd data")
        announce("conv perf-opt drawn", geom, "bwd_filter variant %d" % variant)
        zero = np.zeros_like(w)
        assert_close(gpu_conv_bwd_filter(ctx, g, x, dy, zero, np.float32(1.0), algo=1),
                     oracle.conv_bwd_filter_sgd(og, x, dy, zero, 1.0), TOL, "bwd filter")
        got = gpu_conv_bwd_filter(ctx, g, x, dy, w, np.float32(-1e-5), algo=1)
        assert_close(got, oracle.conv_bwd_filter_sgd(og, x, dy, w, -1e-5), 1e-6, "fused sgd")
    finally:
        lib.vdnn_conv_perf_variant(before)


# Winograd F(4x4, 3x3): planes that are whole 4x4 tiles and planes that are not (tiles stored in part, rows that are not
# whole groups of four pixels take the scalar loads), channel counts at and beside the limits
WINOGRAD_GEOMS = [
    (3, 128, 8, 8, 128, 3, 3, 1, 1, 1, 1),
    (2, 128, 14, 14, 256, 3, 3, 1, 1, 1, 1),   # 14 x 14: 4 x 4 tiles, the last ones half outside
    (3, 144, 7, 9, 80, 3, 3, 1, 1, 1, 1),      # odd plane; 80 produced rows: one ragged row tile; backward data does not apply (80 < 128)
    (2, 256, 13, 20, 96, 3, 3, 1, 1, 1, 1),    # rows of whole groups, a ragged last tile row
    (5, 160, 4, 4, 65, 3, 3, 1, 1, 1, 1),      # one tile per sample, 65 rows
    (1, 512, 28, 28, 192, 3, 3, 1, 1, 1, 1),
]


@pytest.mark.parametrize("geom", WINOGRAD_GEOMS, ids=lambda g: "x".join(map(str, g)))
@pytest.mark.parametrize("small_chunks", [False, True], ids=["one-chunk", "small-chunks"])
def test_conv_winograd_against_oracle(ctx, geom, small_chunks, winograd_variant):
    """Forward (with and without the fused rectifier) and backward data (plain, gated, and written over the gating
    input) of the perf-optimal mode's Winograd variant against the checker; with small chunks the batch is processed in
    several pieces (two samples at a time), the last one shorter."""
    per_sample = (geom[1] + geom[4]) * 36 * ((geom[2] + 3) // 4) * ((geom[3] + 3) // 4) * 4
    chunk_bytes = int(2.5 * per_sample) if small_chunks else 0
    rng = np.random.default_rng(hash(geom) % (2 ** 31) + 3)
    g, og = be.shape(*geom), oracle.shape(*geom)
    x = rng.standard_normal((g.n, g.c, g.h, g.w)).astype(np.float32)
    w = (rng.standard_normal((g.k, g.c, 3, 3)) * np.sqrt(2.0 / (g.c * 9))).astype(np.float32)
    b = rng.standard_normal(g.k).astype(np.float32)
    want_y = oracle.conv_fwd(og, x, w, b)
    dy = rng.standard_normal(want_y.shape).astype(np.float32)
    want_dx = oracle.conv_bwd_data(og, dy, w)
    lib.vdnn_conv_winograd_chunk_bytes(chunk_bytes)
    try:
        fwd_bytes, bwd_bytes = int(lib.vdnn_conv_workspace_bytes(g, 1, 0)), int(lib.vdnn_conv_workspace_bytes(g, 1, 1))
        assert fwd_bytes == winograd_workspace(geom, False, chunk_bytes or 512 << 20) > 0
        bwd_applies = winograd_workspace(geom, True, chunk_bytes or 512 << 20) > 0
        if bwd_applies:
            assert bwd_bytes == winograd_workspace(geom, True, chunk_bytes or 512 << 20)
        with Dev(ctx) as d:
            dx_, dw, db, ddy = d.up(x), d.up(w), d.up(b), d.up(dy)
            y, gx = d.empty(want_y.shape), d.empty(x.shape)
            ws = d.empty((max(fwd_bytes, bwd_bytes) // 4,))
            announce("winograd", geom, chunk_bytes, "fwd")
            check(lib.vdnn_conv_fwd(ctx.handle, None, g, 1, dx_.ptr, dw.ptr, db.ptr, y.ptr, ws.ptr, fwd_bytes))
            assert_close(y.download(want_y.shape), want_y, TOL, "fwd")
            announce("winograd", geom, chunk_bytes, "fwd + relu")
            check(lib.vdnn_conv_fwd_relu(ctx.handle, None, g, 1, dx_.ptr, dw.ptr, db.ptr, y.ptr, ws.ptr, fwd_bytes))
            got = y.download(want_y.shape)
            assert_close(got, np.maximum(want_y, 0), TOL, "fwd + relu")
            assert np.all(got >= 0)
            # a workspace that is too small: the memory-optimal kernels run instead
            check(lib.vdnn_conv_fwd(ctx.handle, None, g, 1, dx_.ptr, dw.ptr, db.ptr, y.ptr, ws.ptr, fwd_bytes - 256))
            assert_close(y.download(want_y.shape), want_y, TOL, "fwd, short workspace")
            announce("winograd", geom, chunk_bytes, "bwd_data")
            check(lib.vdnn_conv_bwd_data(ctx.handle, None, g, 1, ddy.ptr, dw.ptr, gx.ptr, ws.ptr, bwd_bytes))
            assert_close(gx.download(x.shape), want_dx, TOL, "bwd data")
            announce("winograd", geom, chunk_bytes, "bwd_data gated")
            check(lib.vdnn_conv_bwd_data_relu(ctx.handle, None, g, 1, ddy.ptr, dw.ptr, dx_.ptr, gx.ptr, ws.ptr, bwd_bytes))
            gated = gx.download(x.shape)
            assert_close(gated, np.where(x > 0, want_dx, 0), TOL, "bwd data gated")
            assert np.all(gated[x <= 0] == 0)
            if winograd_wgrad_applies(geom):
                # before the input is overwritten below: the filter gradient alone, then applied to the filter
                announce("winograd", geom, chunk_bytes, "bwd_filter")
                flt_bytes = int(lib.vdnn_conv_workspace_bytes(g, 1, 2))
                assert flt_bytes > 0
                ws2, gw, wu = d.empty((flt_bytes // 4,)), d.empty(w.shape), d.up(w)
                check(lib.vdnn_conv_bwd_filter(ctx.handle, None, g, 1, dx_.ptr, ddy.ptr, gw.ptr, ws2.ptr, flt_bytes))
                want_dw = oracle.conv_bwd_filter_sgd(og, x, dy, np.zeros_like(w), 1.0)
                assert_close(gw.download(w.shape), want_dw, TOL, "bwd filter")
                check(lib.vdnn_conv_bwd_filter_sgd(ctx.handle, None, g, 1, dx_.ptr, ddy.ptr, wu.ptr, np.float32(-0.37), ws2.ptr, flt_bytes))
                assert_close(wu.download(w.shape), oracle.conv_bwd_filter_sgd(og, x, dy, w, -0.37), TOL, "bwd filter + sgd")
                # twice the same bits: the sums have a fixed order
                first = gw.download(w.shape)
                check(lib.vdnn_conv_bwd_filter(ctx.handle, None, g, 1, dx_.ptr, ddy.ptr, gw.ptr, ws2.ptr, flt_bytes))
                assert np.array_equal(gw.download(w.shape), first)
            announce("winograd", geom, chunk_bytes, "bwd_data over the gating input")
            assert lib.vdnn_conv_bwd_data_in_place_ok(g)
            check(lib.vdnn_conv_bwd_data_relu(ctx.handle, None, g, 1, ddy.ptr, dw.ptr, dx_.ptr, dx_.ptr, ws.ptr, bwd_bytes))
            assert np.array_equal(dx_.download(x.shape), gated)
    finally:
        lib.vdnn_conv_winograd_chunk_bytes(0)


# The perf-optimal mode's default for 3x3 / stride 1 / padding 1 float layers: operands as two bfloat16 parts, three
# matrix instructions per product. Forward needs C % 16 == 0, backward data K % 16 == 0, both an even W; backward filter
# W % 4 == 0, W >= 16, H*W % 8 == 0 and C % 64 == 0. Tile edges, ragged row tiles, split and tail reductions, rows that
# are not whole groups of eight pixels.
SPLIT_GEOMS = [
    (3, 64, 16, 16, 64, 3, 3, 1, 1, 1, 1),
    (2, 128, 28, 28, 96, 3, 3, 1, 1, 1, 1),     # 96 rows: a ragged second row tile
    (2, 64, 12, 20, 130, 3, 3, 1, 1, 1, 1),     # rows of two and a half groups; 130 output channels: backward data takes another kernel
    (5, 16, 6, 10, 32, 3, 3, 1, 1, 1, 1),       # one slice of channels; backward filter takes another kernel
    (1, 512, 28, 28, 192, 3, 3, 1, 1, 1, 1),    # deep reduction, few tiles: split
    (3, 64, 56, 56, 130, 3, 3, 1, 1, 1, 1),     # several pixel tiles per sample, tiles that straddle samples
    (7, 128, 6, 20, 192, 3, 3, 1, 1, 1, 1),     # planes smaller than a pixel tile
    (2, 64, 16, 36, 64, 3, 3, 1, 1, 1, 1),      # rows of four and a half groups
    (130, 32, 14, 14, 48, 3, 3, 1, 1, 1, 1),    # more tiles than one round: the tail round is split
]


def split_applies(geom):
    """(forward, backward data, backward filter) of the split-bfloat16 variant."""
    n, c, h, w, k, r, s, ph, pw, sh, sw = geom
    base = (r, s, ph, pw, sh, sw) == (3, 3, 1, 1, 1, 1) and w % 2 == 0 and c > 4
    return (base and c % 16 == 0, base and k % 16 == 0,
            (r, s, ph, pw, sh, sw) == (3, 3, 1, 1, 1, 1) and w % 4 == 0 and w >= 16 and (h * w) % 8 == 0 and c % 64 == 0)


@pytest.mark.parametrize("geom", SPLIT_GEOMS, ids=lambda g: "x".join(map(str, g)))
def test_conv_split_bf16_against_oracle(ctx, geom):
    """Forward (with and without the fused rectifier), backward data (plain, gated, written over the gating input) and
    backward filter (alone, applied, with the bias gradient) of the perf-optimal mode's default variant against the
    checker. Its error is that of two dropped low-order terms per product, about 5e-6 of the largest output: held to
    3e-5 here where the mode's bound is 1e-4. The same bits twice."""
    tight = 3e-5
    fwd_ok, bwd_ok, flt_ok = split_applies(geom)
    rng = np.random.default_rng(hash(geom) % (2 ** 31) + 5)
    g, og = be.shape(*geom), oracle.shape(*geom)
    filter_bytes = g.k * g.c * 9 * 4
    x = rng.standard_normal((g.n, g.c, g.h, g.w)).astype(np.float32)
    w = (rng.standard_normal((g.k, g.c, 3, 3)) * np.sqrt(2.0 / (g.c * 9))).astype(np.float32)
    b = rng.standard_normal(g.k).astype(np.float32)
    want_y = oracle.conv_fwd(og, x, w, b)
    dy = (rng.standard_normal(want_y.shape) + 0.25).astype(np.float32)
    want_dx = oracle.conv_bwd_data(og, dy, w)
    assert lib.vdnn_conv_perf_variant(-1) == 0
    fwd_bytes, bwd_bytes, flt_bytes = (int(lib.vdnn_conv_workspace_bytes(g, 1, p)) for p in range(3))
    if fwd_ok:
        assert fwd_bytes == filter_bytes
    if bwd_ok:
        assert bwd_bytes == filter_bytes
    with Dev(ctx) as d:
        dx_, dw, db, ddy = d.up(x), d.up(w), d.up(b), d.up(dy)
        y, gx = d.empty(want_y.shape), d.empty(x.shape)
        ws = d.empty((max(fwd_bytes, bwd_bytes, flt_bytes, 4) // 4,))
        announce("split bf16", geom, "fwd")
        check(lib.vdnn_conv_fwd(ctx.handle, None, g, 1, dx_.ptr, dw.ptr, db.ptr, y.ptr, ws.ptr, fwd_bytes))
        first = y.download(want_y.shape)
        assert_close(first, want_y, tight, "fwd")
        if fwd_ok:
            y0 = d.empty(want_y.shape)
            check(lib.vdnn_conv_fwd(ctx.handle, None, g, 0, dx_.ptr, dw.ptr, db.ptr, y0.ptr, None, 0))
            assert not np.array_equal(y0.download(want_y.shape), first)   # (the variant ran)
        check(lib.vdnn_conv_fwd(ctx.handle, None, g, 1, dx_.ptr, dw.ptr, db.ptr, y.ptr, ws.ptr, fwd_bytes))
        assert np.array_equal(y.download(want_y.shape), first)
        announce("split bf16", geom, "fwd + relu")
        check(lib.vdnn_conv_fwd_relu(ctx.handle, None, g, 1, dx_.ptr, dw.ptr, db.ptr, y.ptr, ws.ptr, fwd_bytes))
        assert np.array_equal(y.download(want_y.shape), np.maximum(first, 0))
        if fwd_bytes:
            # a workspace that is too small: the memory-optimal kernels run instead
            check(lib.vdnn_conv_fwd(ctx.handle, None, g, 1, dx_.ptr, dw.ptr, db.ptr, y.ptr, ws.ptr, fwd_bytes - 256))
            assert_close(y.download(want_y.shape), want_y, tight, "fwd, short workspace")
        announce("split bf16", geom, "bwd_data")
        check(lib.vdnn_conv_bwd_data(ctx.handle, None, g, 1, ddy.ptr, dw.ptr, gx.ptr, ws.ptr, bwd_bytes))
        plain = gx.download(x.shape)
        assert_close(plain, want_dx, tight, "bwd data")
        announce("split bf16", geom, "bwd_data gated")
        check(lib.vdnn_conv_bwd_data_relu(ctx.handle, None, g, 1, ddy.ptr, dw.ptr, dx_.ptr, gx.ptr, ws.ptr, bwd_bytes))
        gated = gx.download(x.shape)
        assert np.array_equal(gated, np.where(x > 0, plain, 0))
        announce("split bf16", geom, "bwd_filter")
        assert bool(lib.vdnn_conv_bwd_filter_sums_bias(g, 1, 0)) or not flt_ok
        gw, gb, wu, bu = d.empty(w.shape), d.empty(b.shape), d.up(w), d.up(b)
        fws = ws.ptr if flt_bytes else None
        check(lib.vdnn_conv_bwd_filter_bias(ctx.handle, None, g, 1, dx_.ptr, ddy.ptr, gw.ptr, gb.ptr, fws, flt_bytes))
        got_dw, got_db = gw.download(w.shape), gb.download(b.shape)
        assert_close(got_dw, oracle.conv_bwd_filter_sgd(og, x, dy, np.zeros_like(w), 1.0), tight, "bwd filter")
        assert_close(got_db, oracle.conv_bwd_bias_sgd(og, dy, np.zeros_like(b), 1.0), tight, "bias gradient")
        alpha = np.float32(-0.37)
        check(lib.vdnn_conv_bwd_filter_bias_sgd(ctx.handle, None, g, 1, dx_.ptr, ddy.ptr, wu.ptr, bu.ptr, alpha, fws, flt_bytes))
        assert_close(wu.download(w.shape), oracle.conv_bwd_filter_sgd(og, x, dy, w, alpha), tight, "bwd filter + sgd")
        assert_close(bu.download(b.shape), oracle.conv_bwd_bias_sgd(og, dy, b, alpha), tight, "bias + sgd")
        check(lib.vdnn_conv_bwd_filter(ctx.handle, None, g, 1, dx_.ptr, ddy.ptr, gw.ptr, fws, flt_bytes))
        assert np.array_equal(gw.download(w.shape), got_dw)
        if flt_ok:
            g0 = d.empty(w.shape)
            check(lib.vdnn_conv_bwd_filter(ctx.handle, None, g, 0, dx_.ptr, ddy.ptr, g0.ptr, None, 0))
            assert not np.array_equal(g0.download(w.shape), got_dw)   # (the variant ran)
        announce("split bf16", geom, "bwd_data over the gating input")
        assert lib.vdnn_conv_bwd_data_in_place_ok(g)
        check(lib.vdnn_conv_bwd_data_relu(ctx.handle, None, g, 1, ddy.ptr, dw.ptr, dx_.ptr, dx_.ptr, ws.ptr, bwd_bytes))
        assert np.array_equal(dx_.download(x.shape), gated)


# The same products through the general bfloat16 engine: stride-1 layers the windowed kernel does not take (and strided
# forward), reduced channels a multiple of 16, at most 32 taps.
SPLIT_GENERAL_GEOMS = [
    (2, 48, 27, 27, 96, 5, 5, 2, 2, 1, 1),      # AlexNet conv2 geometry
    (2, 64, 12, 12, 80, 5, 5, 0, 0, 1, 1),      # no padding; 80 rows: a ragged row tile
    (3, 32, 13, 13, 48, 3, 3, 1, 1, 1, 1),      # odd planes, too narrow for Winograd
    (2, 96, 13, 15, 64, 3, 3, 1, 1, 1, 1),      # 64 rows: the 64 x 256 tile, two items per thread
    (1, 16, 20, 24, 32, 3, 5, 1, 2, 2, 1),      # strided: forward only
    (3, 64, 9, 9, 128, 1, 1, 0, 0, 1, 1),       # one tap
    (130, 16, 7, 7, 16, 3, 3, 1, 1, 1, 1),      # samples smaller than a tile: tiles over several samples
    (2, 512, 6, 6, 160, 3, 3, 0, 0, 1, 1),      # deep reduction, few tiles: split
    (2, 256, 13, 13, 384, 3, 3, 1, 1, 1, 1),    # AlexNet conv3 geometry: Winograd applies too, this variant is taken
]


@pytest.mark.parametrize("geom", SPLIT_GENERAL_GEOMS, ids=lambda g: "x".join(map(str, g)))
def test_conv_split_general_against_oracle(ctx, geom):
    """Forward (with the rectifier too) and backward data (plain and gated) of the perf-optimal mode through the general
    bfloat16 engine with float operands as two bfloat16 parts, against the checker: held to 3e-5 (the mode's bound is
    1e-4), other bits than the memory-optimal kernels' (the variant ran), the same bits twice."""
    tight = 3e-5
    n, c, h, w_, k, r, s_, ph, pw, sh, sw = geom
    rng = np.random.default_rng(hash(geom) % (2 ** 31) + 9)
    g, og = be.shape(*geom), oracle.shape(*geom)
    filter_bytes = k * c * r * s_ * 4
    x = rng.standard_normal((g.n, g.c, g.h, g.w)).astype(np.float32)
    w = (rng.standard_normal((g.k, g.c, g.r, g.s)) * np.sqrt(2.0 / (g.c * g.r * g.s))).astype(np.float32)
    b = rng.standard_normal(g.k).astype(np.float32)
    want_y = oracle.conv_fwd(og, x, w, b)
    dy = rng.standard_normal(want_y.shape).astype(np.float32)
    want_dx = oracle.conv_bwd_data(og, dy, w)
    assert lib.vdnn_conv_perf_variant(-1) == 0
    assert int(lib.vdnn_conv_workspace_bytes(g, 1, 0)) == filter_bytes
    bwd_applies = (sh, sw) == (1, 1) and k % 16 == 0
    if bwd_applies:
        assert int(lib.vdnn_conv_workspace_bytes(g, 1, 1)) == filter_bytes
    with Dev(ctx) as d:
        dx_, dw, db, ddy = d.up(x), d.up(w), d.up(b), d.up(dy)
        y, y0, gx, gx0 = d.empty(want_y.shape), d.empty(want_y.shape), d.empty(x.shape), d.empty(x.shape)
        ws = d.empty((filter_bytes // 4,))
        announce("split general", geom, "fwd")
        check(lib.vdnn_conv_fwd(ctx.handle, None, g, 1, dx_.ptr, dw.ptr, db.ptr, y.ptr, ws.ptr, filter_bytes))
        first = y.download(want_y.shape)
        assert_close(first, want_y, tight, "fwd")
        check(lib.vdnn_conv_fwd(ctx.handle, None, g, 0, dx_.ptr, dw.ptr, db.ptr, y0.ptr, None, 0))
        assert not np.array_equal(y0.download(want_y.shape), first)
        check(lib.vdnn_conv_fwd_relu(ctx.handle, None, g, 1, dx_.ptr, dw.ptr, db.ptr, y.ptr, ws.ptr, filter_bytes))
        assert np.array_equal(y.download(want_y.shape), np.maximum(first, 0))
        announce("split general", geom, "bwd_data")
        check(lib.vdnn_conv_bwd_data(ctx.handle, None, g, 1, ddy.ptr, dw.ptr, gx.ptr, ws.ptr, filter_bytes))
        plain = gx.download(x.shape)
        assert_close(plain, want_dx, tight, "bwd data")
        check(lib.vdnn_conv_bwd_data(ctx.handle, None, g, 0, ddy.ptr, dw.ptr, gx0.ptr, None, 0))
        assert np.array_equal(gx0.download(x.shape), plain) != bwd_applies
        check(lib.vdnn_conv_bwd_data_relu(ctx.handle, None, g, 1, ddy.ptr, dw.ptr, dx_.ptr, gx.ptr, ws.ptr, filter_bytes))
        assert np.array_equal(gx.download(x.shape), np.where(x > 0, plain, 0))
        check(lib.vdnn_conv_bwd_data(ctx.handle, None, g, 1, ddy.ptr, dw.ptr, gx.ptr, ws.ptr, filter_bytes))
        assert np.array_equal(gx.download(x.shape), plain)


# (geometry, algorithm mode, whether the filter-gradient kernel of the shape adds up the bias gradient itself)
FILTER_BIAS_GEOMS = [
    ((7, 3, 40, 36, 16, 3, 3, 1, 1, 1, 1), 0, True),       # first-layer kernel: the product's spare column multiplies dy by one
    ((2, 2, 16, 64, 70, 3, 3, 1, 1, 1, 1), 0, True),       # two input channels, a ragged second block of output channels
    ((3, 64, 56, 56, 130, 3, 3, 1, 1, 1, 1), 0, True),     # filter-row kernel, three row tiles, the last ragged, many splits
    ((4, 64, 14, 14, 64, 3, 3, 1, 1, 1, 1), 0, True),      # filter-row kernel, 64-row tile, groups across image rows
    ((7, 128, 6, 20, 192, 3, 3, 1, 1, 1, 1), 0, True),     # two channel blocks: only the first block's workgroups sum
    ((2, 128, 14, 14, 256, 3, 3, 1, 1, 1, 1), 1, True),    # Winograd: the dy transform sums what it reads
    ((3, 128, 9, 7, 80, 3, 3, 1, 1, 1, 1), 1, True),       # Winograd, ragged tiles, odd rows (scalar loads)
    ((2, 48, 27, 27, 96, 5, 5, 2, 2, 1, 1), 0, False),     # tile engine: the bias kernels run behind the filter gradient
    ((2, 70, 9, 13, 130, 3, 3, 1, 1, 1, 1), 1, False),
    ((5, 64, 6, 6, 200, 6, 6, 0, 0, 1, 1), 0, False),      # one dense product
]


@pytest.mark.parametrize("geom,algo,inside", FILTER_BIAS_GEOMS, ids=lambda v: "x".join(map(str, v)) if isinstance(v, tuple) else str(v))
def test_conv_bwd_filter_with_the_bias_gradient(ctx, geom, algo, inside):
    """vdnn_conv_bwd_filter_bias_sgd / _bias / _then_bias_sgd (layer.cu:631-660 in one call) against the checker's two
    reductions: the filter as with the separate call (same bits), the bias gradient within the tolerance (its sums take
    another order inside the filter-gradient kernel), twice the same bits."""
    rng = np.random.default_rng(hash(geom) % (2 ** 31) + 11)
    g, og = be.shape(*geom), oracle.shape(*geom)
    assert bool(lib.vdnn_conv_bwd_filter_sums_bias(g, algo, 0)) == inside
    x = rng.standard_normal((g.n, g.c, g.h, g.w)).astype(np.float32)
    w = (rng.standard_normal((g.k, g.c, g.r, g.s)) * np.sqrt(2.0 / (g.c * g.r * g.s))).astype(np.float32)
    b = rng.standard_normal(g.k).astype(np.float32)
    P, Q = lib.vdnn_out_dim(g.h, g.pad_h, g.r, g.stride_h), lib.vdnn_out_dim(g.w, g.pad_w, g.s, g.stride_w)
    dy = (rng.standard_normal((g.n, g.k, P, Q)) + 0.25).astype(np.float32)   # a mean: the bias gradient is not a sum that cancels
    alpha = np.float32(-0.37)
    want_w, want_b = oracle.conv_bwd_filter_sgd(og, x, dy, w, alpha), oracle.conv_bwd_bias_sgd(og, dy, b, alpha)
    want_dw = oracle.conv_bwd_filter_sgd(og, x, dy, np.zeros_like(w), 1.0)
    want_db = oracle.conv_bwd_bias_sgd(og, dy, np.zeros_like(b), 1.0)
    nws = int(lib.vdnn_conv_workspace_bytes(g, algo, 2))
    with Dev(ctx) as d:
        dx_, ddy = d.up(x), d.up(dy)
        ws = d.empty((max(nws, 4) // 4,)).ptr if nws else None
        announce("bwd filter + bias", geom, algo, "sgd")
        dw, db = d.up(w), d.up(b)
        check(lib.vdnn_conv_bwd_filter_bias_sgd(ctx.handle, None, g, algo, dx_.ptr, ddy.ptr, dw.ptr, db.ptr, alpha, ws, nws))
        got_w, got_b = dw.download(w.shape), db.download(b.shape)
        assert_close(got_w, want_w, TOL, "filter")
        assert_close(got_b, want_b, TOL, "bias")
        assert not np.array_equal(got_b, b)
        # the filter's bits are those of the call without the bias
        dw2 = d.up(w)
        check(lib.vdnn_conv_bwd_filter_sgd(ctx.handle, None, g, algo, dx_.ptr, ddy.ptr, dw2.ptr, alpha, ws, nws))
        assert np.array_equal(dw2.download(w.shape), got_w)
        announce("bwd filter + bias", geom, algo, "gradients")
        gw, gb = d.up(np.full_like(w, 7.0)), d.up(np.full_like(b, 7.0))
        check(lib.vdnn_conv_bwd_filter_bias(ctx.handle, None, g, algo, dx_.ptr, ddy.ptr, gw.ptr, gb.ptr, ws, nws))
        got_dw, got_db = gw.download(w.shape), gb.download(b.shape)
        assert_close(got_dw, want_dw, TOL, "dW")
        assert_close(got_db, want_db, TOL, "db")
        # db applied afterwards = the fused update (one fused multiply-add either way)
        b2 = d.up(b)
        check(lib.vdnn_sgd_apply(ctx.handle, None, g.k, alpha, gb.ptr, b2.ptr))
        assert np.array_equal(b2.download(b.shape), got_b)
        announce("bwd filter + bias", geom, algo, "gradient, then the bias step")
        gw3, b3 = d.up(np.zeros_like(w)), d.up(b)
        check(lib.vdnn_conv_bwd_filter_then_bias_sgd(ctx.handle, None, g, algo, dx_.ptr, ddy.ptr, gw3.ptr, b3.ptr, alpha, ws, nws))
        assert np.array_equal(gw3.download(w.shape), got_dw)
        assert np.array_equal(b3.download(b.shape), got_b)
        # repeatable
        check(lib.vdnn_conv_bwd_filter_bias(ctx.handle, None, g, algo, dx_.ptr, ddy.ptr, gw.ptr, gb.ptr, ws, nws))
        assert np.array_equal(gb.download(b.shape), got_db) and np.array_equal(gw.download(w.shape), got_dw)


def test_conv_tail_round_is_split_and_agrees_with_two_half_batches(ctx):
    """VGG16's 14x14 layers at batch 128 make 784 output tiles for 768 resident workgroups: the 16 tiles of
    the last round are split along the reduction. No CPU result is affordable at this size; convolution is
    independent per sample, so the two half batches (392 tiles each, a different launch geometry) must
    give the same values to float rounding."""
    geom = (128, 512, 14, 14, 512, 3, 3, 1, 1, 1, 1)
    half = (64,) + geom[1:]
    rng = np.random.default_rng(17)
    x = rng.standard_normal((128, 512, 14, 14)).astype(np.float32)
    w = (rng.standard_normal((512, 512, 3, 3)) * np.sqrt(2.0 / 4608)).astype(np.float32)
    b = rng.standard_normal(512).astype(np.float32)
    announce("tail round", geom, "fwd")
    y = gpu_conv_fwd(ctx, be.shape(*geom), x, w, b)
    y2 = np.concatenate([gpu_conv_fwd(ctx, be.shape(*half), x[:64], w, b), gpu_conv_fwd(ctx, be.shape(*half), x[64:], w, b)])
    assert_close(y, y2, 1e-5, "forward, whole batch against two halves")
    # a few output elements against the definition, in float64
    for (n, k, p, q) in ((0, 0, 0, 0), (127, 511, 13, 13), (77, 300, 6, 0), (127, 5, 0, 13)):
        acc = float(b[k])
        for r in range(3):
            for s_ in range(3):
                ih, iw = p - 1 + r, q - 1 + s_
                if 0 <= ih < 14 and 0 <= iw < 14:
                    acc += float(np.dot(x[n, :, ih, iw].astype(np.float64), w[k, :, r, s_].astype(np.float64)))
        assert abs(y[n, k, p, q] - acc) <= 1e-4 * max(1.0, abs(acc))
    announce("tail round", geom, "bwd_data")
    dy = rng.standard_normal(y.shape).astype(np.float32)
    dx = gpu_conv_bwd_data(ctx, be.shape(*geom), dy, w)
    dx2 = np.concatenate([gpu_conv_bwd_data(ctx, be.shape(*half), dy[:64], w), gpu_conv_bwd_data(ctx, be.shape(*half), dy[64:], w)])
    assert_close(dx, dx2, 1e-5, "backward data, whole batch against two halves")


def test_conv_results_do_not_depend_on_the_run(ctx):
    """Split reductions are ordered: two runs give identical bits."""
    geom = (4, 64, 28, 28, 64, 3, 3, 1, 1, 1, 1)
    rng = np.random.default_rng(5)
    g = be.shape(*geom)
    x = rng.standard_normal((4, 64, 28, 28)).astype(np.float32)
    dy = rng.standard_normal((4, 64, 28, 28)).astype(np.float32)
    w = rng.standard_normal((64, 64, 3, 3)).astype(np.float32)
    announce("determinism bwd_filter")
    a = gpu_conv_bwd_filter(ctx, g, x, dy, w, np.float32(-1e-3))
    b = gpu_conv_bwd_filter(ctx, g, x, dy, w, np.float32(-1e-3))
    assert np.array_equal(a, b)
    announce("determinism bwd_bias")
    assert np.array_equal(gpu_conv_bwd_bias(ctx, g, dy, w[:, 0, 0, 0], np.float32(1.0)), gpu_conv_bwd_bias(ctx, g, dy, w[:, 0, 0, 0], np.float32(1.0)))


def _fc_all(ctx, x, w, b, dy, alpha):
    n, cin = x.shape
    cout = w.shape[0]
    with Dev(ctx) as d:
        dx_, dw_, db_, ddy = d.up(x), d.up(w), d.up(b), d.up(dy)
        y, gx = d.empty((n, cout)), d.empty((n, cin))
        check(lib.vdnn_fc_fwd(ctx.handle, None, n, cin, cout, dx_.ptr, dw_.ptr, db_.ptr, y.ptr))
        check(lib.vdnn_fc_bwd_data(ctx.handle, None, n, cin, cout, ddy.ptr, dw_.ptr, gx.ptr))
        check(lib.vdnn_fc_bwd_weight_sgd(ctx.handle, None, n, cin, cout, dx_.ptr, ddy.ptr, dw_.ptr, alpha))
        check(lib.vdnn_fc_bwd_bias_sgd(ctx.handle, None, n, cout, ddy.ptr, db_.ptr, alpha))
        return y.download((n, cout)), gx.download((n, cin)), dw_.download(w.shape), db_.download(b.shape)


def test_fc_golden(ctx):
    f = golden("fc")
    alpha = np.float32(0.21)
    announce("fc golden")
    y, dx, w2, b2 = _fc_all(ctx, f["x"], f["w"], f["b"], f["dy"], alpha)
    assert_close(y, f["y"], TOL)
    assert_close(dx, f["dx"], TOL)
    assert_close(w2, f["w"] + alpha * f["dw"], TOL)
    assert_close(b2, f["b"] + alpha * f["db"], TOL)


@pytest.mark.parametrize("n,cin,cout", [(128, 1000, 520), (64, 2304, 512), (32, 777, 1000), (5, 40, 33)])
def test_fc_random_against_oracle(ctx, n, cin, cout):
    rng = np.random.default_rng(n * 7 + cin)
    x = rng.standard_normal((n, cin)).astype(np.float32)
    w = (rng.standard_normal((cout, cin)) * np.sqrt(2.0 / cin)).astype(np.float32)
    b = rng.standard_normal(cout).astype(np.float32)
    dy = rng.standard_normal((n, cout)).astype(np.float32)
    alpha = np.float32(-0.01)
    announce("fc random", n, cin, cout)
    y, dx, w2, b2 = _fc_all(ctx, x, w, b, dy, alpha)
    assert_close(y, oracle.fc_fwd(x, w, b), TOL, "fwd")
    assert_close(dx, oracle.fc_bwd_data(dy, w), TOL, "bwd data")
    assert_close((w2.astype(np.float64) - w) / alpha, (oracle.fc_bwd_weight_sgd(x, dy, w, alpha).astype(np.float64) - w) / alpha, 1e-3, "dW")
    assert_close(w2, oracle.fc_bwd_weight_sgd(x, dy, w, alpha), 1e-6, "fused sgd")
    assert_close(b2, oracle.fc_bwd_bias_sgd(dy, b, alpha), 1e-6, "bias")


@pytest.mark.parametrize("count", [1, 3, 4, 1023, 4096 * 33 + 5])
def test_relu_is_exact(ctx, count):
    rng = np.random.default_rng(count)
    x = rng.standard_normal(count).astype(np.float32)
    x[::7] = 0.0
    if count > 16:
        x[3], x[5], x[6], x[9] = np.nan, np.inf, -np.inf, -0.0
    dy = rng.standard_normal(count).astype(np.float32)
    announce("relu", count)
    with Dev(ctx) as d:
        a, g = d.up(x), d.up(dy)
        y, dx, dx2 = d.empty(count), d.empty(count), d.empty(count)
        check(lib.vdnn_relu_fwd(ctx.handle, None, count, a.ptr, y.ptr))
        check(lib.vdnn_relu_bwd(ctx.handle, None, count, a.ptr, y.ptr, g.ptr, dx.ptr))
        check(lib.vdnn_relu_bwd(ctx.handle, None, count, None, y.ptr, g.ptr, dx2.ptr))
        gy, gdx, gdx2 = y.download(count), dx.download(count), dx2.download(count)
    wy = oracle.relu_fwd(x)
    assert np.array_equal(gy.view(np.uint32), wy.view(np.uint32))
    wdx = oracle.relu_bwd(x, wy, dy)
    assert np.array_equal(gdx, wdx)
    assert np.array_equal(gdx2, wdx)  # from y alone: same elements selected


@pytest.mark.parametrize("count", [1, 5, 4096 * 9 + 3])
def test_tanh_and_sigmoid(ctx, count):
    rng = np.random.default_rng(count)
    x = (rng.standard_normal(count) * 3).astype(np.float32)
    x[: min(count, 4)] = np.array([0.0, 30.0, -30.0, -0.0], np.float32)[: min(count, 4)]
    dy = rng.standard_normal(count).astype(np.float32)
    for name, fwd, bwd in (("tanh", oracle.tanh_fwd, oracle.tanh_bwd), ("sigmoid", oracle.sigmoid_fwd, oracle.sigmoid_bwd)):
        announce(name, count)
        with Dev(ctx) as d:
            dx_, ddy, y, gx = d.up(x), d.up(dy), d.empty((count,)), d.empty((count,))
            check(getattr(lib, "vdnn_%s_fwd" % name)(ctx.handle, None, count, dx_.ptr, y.ptr))
            check(getattr(lib, "vdnn_%s_bwd" % name)(ctx.handle, None, count, y.ptr, ddy.ptr, gx.ptr))
            got_y, got_dx = y.download((count,)), gx.download((count,))
        # float32 library functions against the checker's double evaluation: a few units in the last place
        assert_close(got_y, fwd(x), 1e-6, name + " forward")
        assert_close(got_dx, bwd(got_y, dy), 1e-6, name + " backward")


POOLS = [(2, 3, 13, 15, 3, 2), (2, 3, 12, 12, 2, 2), (1, 2, 7, 9, 2, 2), (3, 5, 8, 16, 2, 2), (2, 4, 27, 27, 3, 2), (1, 2, 6, 10, 2, 2),
         (3, 7, 55, 55, 3, 2),     # AlexNet's first pool: one plane per workgroup in LDS
         (2, 37, 13, 13, 3, 2),    # several planes per workgroup, the last group short
         (1, 2, 130, 121, 3, 2),   # planes too large for LDS: the gather kernel
         (2, 3, 20, 20, 3, 1)]     # stride 1: every input in up to nine windows


@pytest.mark.parametrize("n,c,h,w,win,stride", POOLS)
@pytest.mark.parametrize("ties", [False, True])
def test_maxpool_is_exact(ctx, n, c, h, w, win, stride, ties):
    rng = np.random.default_rng(h * 31 + w)
    x = rng.standard_normal((n, c, h, w)).astype(np.float32)
    if ties:
        x = np.maximum(np.round(x), 0).astype(np.float32)  # post-ReLU-like data full of equal values
    g, og = be.shape(n, c, h, w, 0, win, win, 0, 0, stride, stride), oracle.shape(n, c, h, w, 0, win, win, 0, 0, stride, stride)
    wy = oracle.maxpool_fwd(og, x)
    dy = rng.standard_normal(wy.shape).astype(np.float32)
    announce("maxpool", (n, c, h, w, win, stride), "ties" if ties else "")
    with Dev(ctx) as d:
        a, gdy = d.up(x), d.up(dy)
        y, dx = d.empty(wy.shape), d.empty(x.shape)
        check(lib.vdnn_maxpool_fwd(ctx.handle, None, g, a.ptr, y.ptr))
        check(lib.vdnn_maxpool_bwd(ctx.handle, None, g, a.ptr, y.ptr, gdy.ptr, dx.ptr))
        gy, gdx = y.download(wy.shape), dx.download(x.shape)
    assert np.array_equal(gy, wy)
    assert np.array_equal(gdx, oracle.maxpool_bwd(og, x, wy, dy))


def test_maxpool_golden(ctx):
    for name in ("pool_3x3_s2", "pool_2x2_s2", "pool_2x2_s2_odd"):
        f = golden(name)
        g = conv_shape(f["geom"])
        announce("maxpool golden", name)
        with Dev(ctx) as d:
            a, gdy = d.up(f["x"]), d.up(f["dy"])
            y, dx = d.empty(f["y"].shape), d.empty(f["x"].shape)
            check(lib.vdnn_maxpool_fwd(ctx.handle, None, g, a.ptr, y.ptr))
            check(lib.vdnn_maxpool_bwd(ctx.handle, None, g, a.ptr, y.ptr, gdy.ptr, dx.ptr))
            assert np.array_equal(y.download(f["y"].shape), f["y"])
            assert_close(dx.download(f["x"].shape), f["dx"], 1e-7)


@pytest.mark.parametrize("shape,scale", [((2, 9, 4, 5), 1.0), ((2, 9, 4, 5), 60.0), ((3, 96, 11, 13), 30.0), ((1, 3, 5, 5), 10.0),
                                         ((2, 37, 7, 9), 20.0), ((1, 16, 3, 3), 5.0), ((2, 17, 3, 3), 5.0), ((1, 1, 4, 4), 50.0)])
def test_lrn(ctx, shape, scale):
    rng = np.random.default_rng(int(scale) + shape[1])
    x = (rng.standard_normal(shape) * scale).astype(np.float32)
    dy = rng.standard_normal(shape).astype(np.float32)
    wy = oracle.lrn_fwd(x)
    n, c, hw = shape[0], shape[1], shape[2] * shape[3]
    announce("lrn", shape, scale)
    with Dev(ctx) as d:
        a, gdy = d.up(x), d.up(dy)
        y, dx = d.empty(shape), d.empty(shape)
        check(lib.vdnn_lrn_fwd(ctx.handle, None, n, c, hw, a.ptr, y.ptr))
        check(lib.vdnn_lrn_bwd(ctx.handle, None, n, c, hw, a.ptr, y.ptr, gdy.ptr, dx.ptr))
        gy, gdx = y.download(shape), dx.download(shape)
    assert_close(gy, wy, 1e-5, "fwd")
    assert_close(gdx, oracle.lrn_bwd(x, wy, dy), 1e-5, "bwd")
    if shape == (2, 9, 4, 5):
        f = golden("lrn" if scale == 1.0 else "lrn_large_inputs")
        with Dev(ctx) as d:
            a, gdy, gy_ = d.up(f["x"]), d.up(f["dy"]), d.up(f["y"])
            y, dx = d.empty(shape), d.empty(shape)
            check(lib.vdnn_lrn_fwd(ctx.handle, None, n, c, hw, a.ptr, y.ptr))
            check(lib.vdnn_lrn_bwd(ctx.handle, None, n, c, hw, a.ptr, gy_.ptr, gdy.ptr, dx.ptr))
            assert_close(y.download(shape), f["y"], 1e-5, "golden fwd")
            assert_close(dx.download(shape), f["dx"], 1e-5, "golden bwd")


@pytest.mark.parametrize("n,classes", [(5, 17), (128, 1000), (3, 1), (2, 257)])
def test_softmax(ctx, n, classes):
    rng = np.random.default_rng(classes)
    x = (rng.standard_normal((n, classes)) * 4).astype(np.float32)
    dy = rng.standard_normal((n, classes)).astype(np.float32)
    wy = oracle.softmax_fwd(x)
    announce("softmax", n, classes)
    with Dev(ctx) as d:
        a, gdy = d.up(x), d.up(dy)
        y, dx = d.empty(x.shape), d.empty(x.shape)
        check(lib.vdnn_softmax_fwd(ctx.handle, None, n, classes, a.ptr, y.ptr))
        check(lib.vdnn_softmax_bwd(ctx.handle, None, n, classes, y.ptr, gdy.ptr, dx.ptr))
        gy, gdx = y.download(x.shape), dx.download(x.shape)
    assert_close(gy, wy, 1e-5, "fwd")
    assert np.allclose(gy.sum(axis=1), 1.0, atol=1e-5)
    assert_close(gdx, oracle.softmax_bwd(gy, dy), 1e-5, "bwd")


def test_softmax_golden_and_ce(ctx):
    f = golden("softmax")
    n, classes = f["x"].shape
    announce("softmax golden")
    with Dev(ctx) as d:
        a, gdy, gy = d.up(f["x"]), d.up(f["dy"]), d.up(f["y"])
        y, dx = d.empty(f["x"].shape), d.empty(f["x"].shape)
        check(lib.vdnn_softmax_fwd(ctx.handle, None, n, classes, a.ptr, y.ptr))
        check(lib.vdnn_softmax_bwd(ctx.handle, None, n, classes, gy.ptr, gdy.ptr, dx.ptr))
        assert_close(y.download(f["x"].shape), f["y"], 1e-5)
        assert_close(dx.download(f["x"].shape), f["dx"], 1e-5)
    f = golden("softmax_ce")
    n, classes = f["x"].shape
    announce("softmax-ce golden")
    with Dev(ctx) as d:
        a, lab = d.up(f["x"]), d.up(f["labels"], np.int32)
        prob, dlog, loss, loss2, onehot = d.empty(f["x"].shape), d.empty(f["x"].shape), d.empty(1), d.empty(1), d.up(np.eye(classes, dtype=np.float32)[f["labels"]])
        check(lib.vdnn_softmax_ce_fwd(ctx.handle, None, n, classes, a.ptr, lab.ptr, prob.ptr, loss.ptr))
        check(lib.vdnn_softmax_ce_bwd(ctx.handle, None, n, classes, prob.ptr, lab.ptr, dlog.ptr))
        check(lib.vdnn_cross_entropy_dense(ctx.handle, None, n, classes, prob.ptr, onehot.ptr, loss2.ptr))
        assert_close(prob.download(f["x"].shape), f["prob"], 1e-5)
        assert abs(loss.download(1)[0] - f["loss"][0]) <= 1e-5 * abs(f["loss"][0])
        assert abs(loss2.download(1)[0] - f["loss"][0]) <= 1e-5 * abs(f["loss"][0])
        assert_close(dlog.download(f["x"].shape), f["dx"], 1e-5)


def test_sub_fill_bias_add_are_exact(ctx):
    rng = np.random.default_rng(0)
    a = rng.standard_normal(100003).astype(np.float32)
    b = rng.standard_normal(100003).astype(np.float32)
    announce("sub/fill/bias_add")
    with Dev(ctx) as d:
        da, db, r, f = d.up(a), d.up(b), d.empty(a.shape), d.empty(777)
        check(lib.vdnn_sub(ctx.handle, None, a.size, da.ptr, db.ptr, r.ptr))
        check(lib.vdnn_fill(ctx.handle, None, 777, 1.0, f.ptr))
        assert np.array_equal(r.download(a.shape), a - b)
        assert np.array_equal(f.download(777), np.ones(777, np.float32))
        y = rng.standard_normal((3, 5, 7, 2)).astype(np.float32)
        bias = rng.standard_normal(5).astype(np.float32)
        dy_, dbias = d.up(y), d.up(bias)
        check(lib.vdnn_bias_add(ctx.handle, None, 3, 5, 14, dbias.ptr, dy_.ptr))
        assert np.array_equal(dy_.download(y.shape), y + bias[None, :, None, None])


def test_offload_prefetch_round_trip_is_byte_identical(ctx):
    """offloadSrcData / prefetchPreviousSrcData (layer.cu:969-987): D2H into pinned memory on the
    copy stream, H2D back into a fresh block; the bytes must survive unchanged."""
    import zlib
    rng = np.random.default_rng(1)
    nbytes = 32 << 20
    src = rng.integers(0, 256, nbytes, dtype=np.uint8)
    h = ctx.handle
    announce("offload/prefetch round trip")
    with Dev(ctx) as d:
        a = d.up(src, np.uint8)
        host = C.c_void_p()
        check(lib.vdnn_host_alloc_pinned(h, C.byref(host), nbytes))
        ev = C.c_void_p()
        check(lib.vdnn_event_create(h, C.byref(ev), 0))
        check(lib.vdnn_memcpy_d2h_async(h, host, a.ptr, nbytes, lib.vdnn_ctx_stream_d2h(h)))
        check(lib.vdnn_event_record(h, ev, lib.vdnn_ctx_stream_d2h(h)))
        check(lib.vdnn_stream_wait_event(h, lib.vdnn_ctx_stream_h2d(h), ev))
        b = d.empty(nbytes, np.uint8)
        check(lib.vdnn_memcpy_h2d_async(h, b.ptr, host, nbytes, lib.vdnn_ctx_stream_h2d(h)))
        check(lib.vdnn_stream_synchronize(h, lib.vdnn_ctx_stream_h2d(h)))
        staged = np.ctypeslib.as_array(C.cast(host, C.POINTER(C.c_uint8)), shape=(nbytes,)).copy()
        back = b.download(nbytes, np.uint8)
        check(lib.vdnn_event_destroy(h, ev))
        check(lib.vdnn_host_free_pinned(h, host))
    assert zlib.crc32(staged.tobytes()) == zlib.crc32(src.tobytes())
    assert np.array_equal(back, src)
