"""GPU parity: a seeded sweep of 3x3 / stride 1 / padding 1 geometries through the kernels written for them (the windowed
forward / backward data of bfloat16 layers, the row-per-workgroup backward filter in both element types, the streaming
first-layer kernels), against the CPU checker through the C ABI.

The shapes are drawn so that every variant is met several times: rows of whole groups of eight, four and two pixels,
rows shorter and longer than a slice and than a tile, planes that are and are not multiples of the slice, one to three
input channels, channel counts of one and several blocks, ragged output-channel tiles, reductions short enough for one
split and long enough for many. Tolerances as in test_gpu_kernels.py / test_gpu_bf16.py.
"""
import numpy as np
import pytest

import oracle
import vdnn_implementation_amd.backend as be
from gpu_util import announce, gpu_conv_bwd_data, gpu_conv_bwd_filter, gpu_conv_fwd
from test_gpu_bf16 import Dev, get_act, rnd
from util import assert_close, assert_close_bf16
from vdnn_implementation_amd.backend import check, lib

pytestmark = pytest.mark.gpu
TOL = 1e-4


@pytest.fixture(scope="module")
def ctx():
    c = be.Context(pool_bytes=4 << 30)
    yield c
    c.close()


@pytest.fixture(autouse=True)
def accurate_oracle():
    oracle.set_accumulate_double(True)
    yield
    oracle.set_accumulate_double(False)


def sweep(seed, count):
    rng = np.random.default_rng(seed)
    out = []
    widths = [14, 16, 18, 20, 24, 28, 30, 32, 36, 40, 44, 56, 64, 72, 130]
    while len(out) < count:
        w = int(rng.choice(widths))
        h = int(rng.integers(2, 13))
        if rng.random() < 0.25:
            c = int(rng.integers(1, 4))                   # the first-layer kernels
            k = int(rng.choice([8, 16, 32, 40, 64]))
        else:
            c = int(rng.choice([32, 64, 64, 128, 192]))
            k = int(rng.choice([32, 64, 96, 128, 130, 192]))
        n = int(rng.integers(1, 6))
        if n * c * h * w * k * 9 > 6e8:                   # keeps the checker within a second or two per case
            continue
        out.append((n, c, h, w, k, 3, 3, 1, 1, 1, 1))
    return out


@pytest.mark.parametrize("geom", sweep(20240611, 48), ids=lambda g: "x".join(map(str, g[:5])))
def test_conv3x3_sweep_float(ctx, geom):
    rng = np.random.default_rng(abs(hash(geom)) % (2 ** 31))
    g, og = be.shape(*geom), oracle.shape(*geom)
    x = rng.standard_normal((g.n, g.c, g.h, g.w)).astype(np.float32)
    w = (rng.standard_normal((g.k, g.c, 3, 3)) * np.sqrt(2.0 / (g.c * 9))).astype(np.float32)
    b = rng.standard_normal(g.k).astype(np.float32)
    want_y = oracle.conv_fwd(og, x, w, b)
    announce("conv sweep float", geom, "fwd")
    assert_close(gpu_conv_fwd(ctx, g, x, w, b), want_y, TOL, "fwd")
    dy = rng.standard_normal(want_y.shape).astype(np.float32)
    announce("conv sweep float", geom, "bwd_data")
    assert_close(gpu_conv_bwd_data(ctx, g, dy, w), oracle.conv_bwd_data(og, dy, w), TOL, "bwd data")
    announce("conv sweep float", geom, "bwd_filter")
    zero = np.zeros_like(w)
    assert_close(gpu_conv_bwd_filter(ctx, g, x, dy, zero, np.float32(1.0)), oracle.conv_bwd_filter_sgd(og, x, dy, zero, 1.0), TOL, "bwd filter")


@pytest.mark.parametrize("geom", sweep(977, 48), ids=lambda g: "x".join(map(str, g[:5])))
def test_conv3x3_sweep_bfloat16(ctx, geom):
    rng = np.random.default_rng(abs(hash(geom)) % (2 ** 31) + 1)
    g, og = be.shape(*geom), oracle.shape(*geom)
    x = rnd(rng, (g.n, g.c, g.h, g.w))
    w = (rng.standard_normal((g.k, g.c, 3, 3)) * np.sqrt(2.0 / (g.c * 9))).astype(np.float32)
    b = rng.standard_normal(g.k).astype(np.float32)
    wr = oracle.round_bf16(w)  # forward and backward data multiply the filter rounded to bfloat16
    want_y = oracle.conv_fwd(og, x, wr, b)
    dy = rnd(rng, want_y.shape)
    check(lib.vdnn_ctx_set_activation_dtype(ctx.handle, 1))
    try:
        with Dev(ctx) as d:
            dx_, ddy, dw, db = d.act(x), d.act(dy), d.f32(w), d.f32(b)
            y, gx = d.empty_act(want_y.shape), d.empty_act(x.shape)
            announce("conv sweep bf16", geom, "fwd")
            check(lib.vdnn_conv_fwd(ctx.handle, None, g, 0, dx_.ptr, dw.ptr, db.ptr, y.ptr, None, 0))
            assert_close_bf16(get_act(y, want_y.shape), want_y, "fwd")
            announce("conv sweep bf16", geom, "bwd_data")
            check(lib.vdnn_conv_bwd_data(ctx.handle, None, g, 0, ddy.ptr, dw.ptr, gx.ptr, None, 0))
            assert_close_bf16(get_act(gx, x.shape), oracle.conv_bwd_data(og, dy, wr), "bwd data")
            announce("conv sweep bf16", geom, "bwd_filter")
            gw = d.f32(np.zeros_like(w))
            check(lib.vdnn_conv_bwd_filter(ctx.handle, None, g, 0, dx_.ptr, ddy.ptr, gw.ptr, None, 0))
            assert_close(gw.download(w.shape), oracle.conv_bwd_filter_sgd(og, x, dy, np.zeros_like(w), 1.0), 1e-4, "bwd filter")
    finally:
        check(lib.vdnn_ctx_set_activation_dtype(ctx.handle, 0))
