"""Helpers for the GPU parity tests: every call goes through the C ABI of libvdnn_amd.so."""
import sys

import numpy as np

import vdnn_implementation_amd.backend as be
from vdnn_implementation_amd.backend import check, lib

LR_ALPHA = np.float32(-1e-5)


def announce(*what):
    """Names the case on stdout before the GPU step, so a fault can be attributed."""
    print("[gpu-case]", *what, flush=True)
    sys.stdout.flush()


def conv_shape(geom):
    return be.shape(*[int(v) for v in geom])


class Dev:
    """Uploads arrays, runs one kernel, downloads the result; frees everything on exit."""

    def __init__(self, ctx):
        self.ctx = ctx
        self.bufs = []

    def up(self, a, dtype=np.float32):
        b = self.ctx.to_device(a, dtype)
        self.bufs.append(b)
        return b

    def empty(self, shape, dtype=np.float32):
        b = self.ctx.alloc(max(int(np.prod(shape)) * np.dtype(dtype).itemsize, 4))
        self.bufs.append(b)
        return b

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        for b in self.bufs:
            b.free()


def _workspace(d, g, algo, which):
    """The pass's workspace as the layer code provides it: sized by the library, taken from the pool."""
    nbytes = int(lib.vdnn_conv_workspace_bytes(g, algo, which))
    if nbytes == 0:
        return None, 0
    return d.empty((nbytes // 4,)).ptr, nbytes


def gpu_conv_fwd(ctx, g, x, w, b, algo=0):
    P, Q = lib.vdnn_out_dim(g.h, g.pad_h, g.r, g.stride_h), lib.vdnn_out_dim(g.w, g.pad_w, g.s, g.stride_w)
    with Dev(ctx) as d:
        dx_, dw_, db_ = d.up(x), d.up(w), (d.up(b) if b is not None else None)
        y = d.empty((g.n, g.k, P, Q))
        ws, nws = _workspace(d, g, algo, 0)
        check(lib.vdnn_conv_fwd(ctx.handle, None, g, algo, dx_.ptr, dw_.ptr, db_.ptr if db_ else None, y.ptr, ws, nws))
        return y.download((g.n, g.k, P, Q))


def gpu_conv_bwd_data(ctx, g, dy, w, algo=0):
    with Dev(ctx) as d:
        a, b = d.up(dy), d.up(w)
        dx = d.empty((g.n, g.c, g.h, g.w))
        ws, nws = _workspace(d, g, algo, 1)
        check(lib.vdnn_conv_bwd_data(ctx.handle, None, g, algo, a.ptr, b.ptr, dx.ptr, ws, nws))
        return dx.download((g.n, g.c, g.h, g.w))


def gpu_conv_bwd_filter(ctx, g, x, dy, w, alpha, algo=0):
    with Dev(ctx) as d:
        a, b, c = d.up(x), d.up(dy), d.up(w)
        ws, nws = _workspace(d, g, algo, 2)
        check(lib.vdnn_conv_bwd_filter_sgd(ctx.handle, None, g, algo, a.ptr, b.ptr, c.ptr, alpha, ws, nws))
        return c.download(np.shape(w))


def gpu_conv_bwd_bias(ctx, g, dy, bias, alpha):
    with Dev(ctx) as d:
        a, b = d.up(dy), d.up(bias)
        check(lib.vdnn_conv_bwd_bias_sgd(ctx.handle, None, g, a.ptr, b.ptr, alpha))
        return b.download(np.shape(bias))
