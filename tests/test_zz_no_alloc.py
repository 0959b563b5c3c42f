"""vdnn_conv_bwd_bias_sgd_noalloc, the entry point that allocates nothing, against vdnn_conv_bwd_bias_sgd through the
C ABI: the same bits on two calls in a row (the second with a smaller input, so stale partial sums of the first
sit in the shared scratch array), with float and bfloat16 gradients, and a clear refusal beyond the array's size."""
import ctypes as C

import numpy as np
import pytest

import vdnn_implementation_amd.backend as be
from gpu_util import announce
from util import to_bf16_bits
from vdnn_implementation_amd.backend import check, lib

pytestmark = pytest.mark.gpu
ALPHA = np.float32(-1e-5 * 300)  # large enough that the update changes the leading bits of a bias


def both_ways(ctx, geom, seed, bf16):
    n, k, h, w = geom
    g = be.shape(n, 3, h, w, k, 1, 1, 0, 0, 1, 1)   # 1x1 window, stride 1: dy is n x k x h x w
    rng = np.random.default_rng(seed)
    dy = rng.standard_normal((n, k, h, w)).astype(np.float32)
    bias = rng.standard_normal(k).astype(np.float32)
    if bf16:
        dy = (dy.view(np.uint32) & 0xFFFF0000).view(np.float32)
        dy_dev = ctx.to_device(to_bf16_bits(dy), np.uint16)
    else:
        dy_dev = ctx.to_device(dy)
    want_dev, got_dev = ctx.to_device(bias), ctx.to_device(bias)
    check(lib.vdnn_ctx_set_activation_dtype(ctx.handle, 1 if bf16 else 0))
    announce("conv_bwd_bias_sgd", geom, "bf16" if bf16 else "f32")
    check(lib.vdnn_conv_bwd_bias_sgd(ctx.handle, None, g, dy_dev.ptr, want_dev.ptr, ALPHA))
    announce("conv_bwd_bias_sgd_noalloc", geom, "bf16" if bf16 else "f32")
    check(lib.vdnn_conv_bwd_bias_sgd_noalloc(lib.vdnn_ctx_stream_compute(ctx.handle), g, 1 if bf16 else 0, dy_dev.ptr, got_dev.ptr, ALPHA))
    ctx.synchronize()
    want, got = want_dev.download((k,)), got_dev.download((k,))
    check(lib.vdnn_ctx_set_activation_dtype(ctx.handle, 0))
    for b in (dy_dev, want_dev, got_dev):
        b.free()
    # the reference value: bias + alpha * sum over n, h, w
    ref = bias.astype(np.float64) + np.float64(ALPHA) * dy.astype(np.float64).sum(axis=(0, 2, 3))
    assert np.max(np.abs(want - ref)) <= 1e-4 * np.max(np.abs(ref))
    assert not np.array_equal(want, bias)
    return want, got


@pytest.mark.parametrize("bf16", [False, True])
def test_noalloc_bias_gradient_gives_the_bits_of_the_context_entry_point(bf16):
    with be.Context(pool_bytes=512 << 20) as ctx:
        # a large call, then a smaller one (fewer channels, fewer batch slices, a plane that is not a multiple of four)
        for geom, seed in (((32, 64, 14, 14), 1), ((3, 10, 7, 7), 2), ((16, 512, 28, 28), 3)):
            want, got = both_ways(ctx, geom, seed, bf16)
            assert np.array_equal(want.view(np.uint32), got.view(np.uint32)), geom


def test_noalloc_bias_gradient_rejects_what_its_scratch_cannot_hold():
    with be.Context(pool_bytes=512 << 20) as ctx:
        k = 70000   # one batch slice of 70000 channels: 280000 bytes of partial sums, the array holds 262144
        g = be.shape(1, 3, 1, 1, k, 1, 1, 0, 0, 1, 1)
        dy, bias = ctx.to_device(np.ones(k, np.float32)), ctx.to_device(np.zeros(k, np.float32))
        rc = lib.vdnn_conv_bwd_bias_sgd_noalloc(None, g, 0, dy.ptr, bias.ptr, ALPHA)
        assert rc == be.VDNN_EINVAL
        msg = lib.vdnn_last_error().decode()
        assert "280000" in msg and "262144" in msg
        assert lib.vdnn_conv_bwd_bias_sgd_noalloc(None, g, 7, dy.ptr, bias.ptr, ALPHA) == be.VDNN_EINVAL
        assert lib.vdnn_conv_bwd_bias_sgd_noalloc(None, g, 0, None, bias.ptr, ALPHA) == be.VDNN_EINVAL
        ctx.synchronize()
        assert np.array_equal(bias.download((k,)), np.zeros(k, np.float32)), "a refused call writes nothing"
        # the context entry point takes the same shape
        check(lib.vdnn_conv_bwd_bias_sgd(ctx.handle, None, g, dy.ptr, bias.ptr, ALPHA))
        ctx.synchronize()
        assert np.array_equal(bias.download((k,)), np.full(k, ALPHA, np.float32))
