"""ctypes binding of the device back end's C ABI (include/vdnn_backend.h)."""
import ctypes as C
import os

import numpy as np

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libvdnn_amd.so")

VDNN_OK, VDNN_OOM, VDNN_EINVAL, VDNN_EDEVICE = 0, -1, -2, -3
VDNN_CTX_PLAN_ONLY = 1


class BackendError(RuntimeError):
    def __init__(self, status, message):
        super().__init__("vdnn status %d: %s" % (status, message))
        self.status = status


class OutOfMemory(BackendError):
    pass


def load_library():
    """Loads the native library built in-tree. No fallback: a missing library is an error."""
    if not os.path.exists(LIB_PATH):
        raise ImportError("%s is missing: build it with `python -m vdnn_implementation_amd.build` "
                          "(there is no CPU or pure-Python path)" % LIB_PATH)
    return C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)


lib = load_library()


class Shape(C.Structure):
    _fields_ = [(k, C.c_int) for k in ("n", "c", "h", "w", "k", "r", "s", "pad_h", "pad_w", "stride_h", "stride_w")]


def shape(n, c, h, w, k=0, r=0, s=0, pad_h=0, pad_w=0, stride_h=1, stride_w=1):
    return Shape(n, c, h, w, k, r, s, pad_h, pad_w, stride_h, stride_w)


class ProfileEntry(C.Structure):
    _fields_ = [("name", C.c_char * 48), ("launches", C.c_ulonglong), ("ms", C.c_double), ("flops", C.c_double),
                ("bytes", C.c_double)]


class ProfileInterval(C.Structure):
    _fields_ = [("name", C.c_char * 48), ("stream", C.c_int), ("start_ms", C.c_double), ("stop_ms", C.c_double)]


_vp, _sz, _i, _f = C.c_void_p, C.c_size_t, C.c_int, C.c_float
_S = C.POINTER(Shape)
_psz = C.POINTER(C.c_size_t)

# name -> (restype, argtypes); every symbol include/vdnn_backend.h declares
BACKEND_SYMBOLS = {
    "vdnn_ctx_create": (_i, [C.POINTER(_vp), _i, _i]),
    "vdnn_ctx_destroy": (_i, [_vp]),
    "vdnn_ctx_set_activation_dtype": (_i, [_vp, _i]),
    "vdnn_ctx_activation_dtype": (_i, [_vp]),
    "vdnn_last_error": (C.c_char_p, []),
    "vdnn_device_mem_info": (_i, [_vp, _psz, _psz]),
    "vdnn_device_synchronize": (_i, [_vp]),
    "vdnn_ctx_stream_compute": (_vp, [_vp]),
    "vdnn_ctx_stream_d2h": (_vp, [_vp]),
    "vdnn_ctx_stream_h2d": (_vp, [_vp]),
    "vdnn_ctx_stream_pack": (_vp, [_vp]),
    "vdnn_pool_init": (_i, [_vp, _sz]),
    "vdnn_pool_finalize": (_i, [_vp]),
    "vdnn_pool_malloc": (_i, [_vp, C.POINTER(_vp), _sz]),
    "vdnn_pool_free": (_i, [_vp, _vp]),
    "vdnn_pool_info": (_i, [_vp, _psz, _psz]),
    "vdnn_pool_peak": (_i, [_vp, _psz, _psz]),
    "vdnn_pool_reset_peak": (_i, [_vp]),
    "vdnn_pool_set_cap": (_i, [_vp, _sz]),
    "vdnn_pool_live_blocks": (_i, [_vp, _psz]),
    "vdnn_stream_synchronize": (_i, [_vp, _vp]),
    "vdnn_event_create": (_i, [_vp, C.POINTER(_vp), _i]),
    "vdnn_event_destroy": (_i, [_vp, _vp]),
    "vdnn_event_record": (_i, [_vp, _vp, _vp]),
    "vdnn_stream_wait_event": (_i, [_vp, _vp, _vp]),
    "vdnn_event_synchronize": (_i, [_vp, _vp]),
    "vdnn_event_elapsed_ms": (_i, [_vp, _vp, _vp, C.POINTER(_f)]),
    "vdnn_host_alloc_pinned": (_i, [_vp, C.POINTER(_vp), _sz]),
    "vdnn_host_free_pinned": (_i, [_vp, _vp]),
    "vdnn_memcpy_d2h_async": (_i, [_vp, _vp, _vp, _sz, _vp]),
    "vdnn_memcpy_h2d_async": (_i, [_vp, _vp, _vp, _sz, _vp]),
    "vdnn_zvc_buffer_bytes": (_sz, [_sz, _i]),
    "vdnn_zvc_offload_async": (_i, [_vp, _vp, _vp, _sz, _i, _vp]),
    "vdnn_zvc_offload_staged_async": (_i, [_vp, _vp, _vp, _sz, _vp, _sz, _i, _vp, _vp, _vp, _vp, _i]),
    "vdnn_zvc_prefetch_staged_async": (_i, [_vp, _vp, _vp, _sz, _vp, _sz, _i, _vp]),
    "vdnn_zvc_prefetch_async": (_i, [_vp, _vp, _vp, _sz, _i, _vp]),
    "vdnn_zvc_traffic": (_i, [_vp, C.POINTER(C.c_ulonglong), C.POINTER(C.c_ulonglong)]),
    "vdnn_memcpy_d2h": (_i, [_vp, _vp, _vp, _sz]),
    "vdnn_memcpy_h2d": (_i, [_vp, _vp, _vp, _sz]),
    "vdnn_memcpy_d2d_async": (_i, [_vp, _vp, _vp, _sz, _vp]),
    "vdnn_out_dim": (_i, [_i, _i, _i, _i]),
    "vdnn_conv_workspace_bytes": (_sz, [_S, _i, _i]),
    "vdnn_conv_workspace_bytes_dtype": (_sz, [_S, _i, _i, _i]),
    "vdnn_conv_winograd_chunk_bytes": (_sz, [_sz]),
    "vdnn_conv_perf_variant": (_i, [_i]),
    "vdnn_conv_fwd": (_i, [_vp, _vp, _S, _i, _vp, _vp, _vp, _vp, _vp, _sz]),
    "vdnn_bias_add": (_i, [_vp, _vp, _i, _i, _i, _vp, _vp]),
    "vdnn_conv_bwd_data": (_i, [_vp, _vp, _S, _i, _vp, _vp, _vp, _vp, _sz]),
    "vdnn_conv_fwd_relu": (_i, [_vp, _vp, _S, _i, _vp, _vp, _vp, _vp, _vp, _sz]),
    "vdnn_conv_bwd_data_relu": (_i, [_vp, _vp, _S, _i, _vp, _vp, _vp, _vp, _vp, _sz]),
    "vdnn_fc_fwd_relu": (_i, [_vp, _vp, _i, _i, _i, _vp, _vp, _vp, _vp]),
    "vdnn_fc_bwd_data_relu": (_i, [_vp, _vp, _i, _i, _i, _vp, _vp, _vp, _vp]),
    "vdnn_maxpool_bwd_relu": (_i, [_vp, _vp, _S, _vp, _vp, _vp, _vp]),
    "vdnn_conv_bwd_data_in_place_ok": (_i, [_S]),
    "vdnn_maxpool_bwd_in_place_ok": (_i, [_S]),
    "vdnn_conv_bwd_bias_sgd": (_i, [_vp, _vp, _S, _vp, _vp, _f]),
    "vdnn_conv_bwd_bias_sgd_noalloc": (_i, [_vp, _S, _i, _vp, _vp, _f]),
    "vdnn_conv_bwd_bias_sgd_noalloc_prepare": (_i, []),
    "vdnn_conv_bwd_filter_sgd": (_i, [_vp, _vp, _S, _i, _vp, _vp, _vp, _f, _vp, _sz]),
    "vdnn_fc_fwd": (_i, [_vp, _vp, _i, _i, _i, _vp, _vp, _vp, _vp]),
    "vdnn_fc_bwd_data": (_i, [_vp, _vp, _i, _i, _i, _vp, _vp, _vp]),
    "vdnn_fc_bwd_weight_sgd": (_i, [_vp, _vp, _i, _i, _i, _vp, _vp, _vp, _f]),
    "vdnn_fc_bwd_bias_sgd": (_i, [_vp, _vp, _i, _i, _vp, _vp, _f]),
    "vdnn_conv_bwd_bias": (_i, [_vp, _vp, _S, _vp, _vp]),
    "vdnn_conv_bwd_filter": (_i, [_vp, _vp, _S, _i, _vp, _vp, _vp, _vp, _sz]),
    "vdnn_conv_bwd_filter_sums_bias": (_i, [_S, _i, _i]),
    "vdnn_conv_bwd_filter_bias_sgd": (_i, [_vp, _vp, _S, _i, _vp, _vp, _vp, _vp, _f, _vp, _sz]),
    "vdnn_conv_bwd_filter_bias": (_i, [_vp, _vp, _S, _i, _vp, _vp, _vp, _vp, _vp, _sz]),
    "vdnn_conv_bwd_filter_then_bias_sgd": (_i, [_vp, _vp, _S, _i, _vp, _vp, _vp, _vp, _f, _vp, _sz]),
    "vdnn_fc_bwd_weight": (_i, [_vp, _vp, _i, _i, _i, _vp, _vp, _vp]),
    "vdnn_fc_bwd_bias": (_i, [_vp, _vp, _i, _i, _vp, _vp]),
    "vdnn_sgd_apply": (_i, [_vp, _vp, _sz, _f, _vp, _vp]),
    "vdnn_tanh_fwd": (_i, [_vp, _vp, _sz, _vp, _vp]),
    "vdnn_tanh_bwd": (_i, [_vp, _vp, _sz, _vp, _vp, _vp]),
    "vdnn_sigmoid_fwd": (_i, [_vp, _vp, _sz, _vp, _vp]),
    "vdnn_sigmoid_bwd": (_i, [_vp, _vp, _sz, _vp, _vp, _vp]),
    "vdnn_relu_fwd": (_i, [_vp, _vp, _sz, _vp, _vp]),
    "vdnn_relu_bwd": (_i, [_vp, _vp, _sz, _vp, _vp, _vp, _vp]),
    "vdnn_maxpool_fwd": (_i, [_vp, _vp, _S, _vp, _vp]),
    "vdnn_maxpool_bwd": (_i, [_vp, _vp, _S, _vp, _vp, _vp, _vp]),
    "vdnn_lrn_fwd": (_i, [_vp, _vp, _i, _i, _i, _vp, _vp]),
    "vdnn_lrn_bwd": (_i, [_vp, _vp, _i, _i, _i, _vp, _vp, _vp, _vp]),
    "vdnn_softmax_fwd": (_i, [_vp, _vp, _i, _i, _vp, _vp]),
    "vdnn_softmax_bwd": (_i, [_vp, _vp, _i, _i, _vp, _vp, _vp]),
    "vdnn_sub": (_i, [_vp, _vp, _sz, _vp, _vp, _vp]),
    "vdnn_fill": (_i, [_vp, _vp, _sz, _f, _vp]),
    "vdnn_softmax_ce_fwd": (_i, [_vp, _vp, _i, _i, _vp, _vp, _vp, _vp]),
    "vdnn_softmax_ce_bwd": (_i, [_vp, _vp, _i, _i, _vp, _vp, _vp]),
    "vdnn_cross_entropy_dense": (_i, [_vp, _vp, _i, _i, _vp, _vp, _vp]),
    "vdnn_profile_enable": (_i, [_vp, _i]),
    "vdnn_profile_collect": (_i, [_vp, C.POINTER(ProfileEntry), _i, C.POINTER(_i)]),
    "vdnn_profile_intervals": (_i, [_vp, C.POINTER(ProfileInterval), _i, C.POINTER(_i)]),
}

for _name, (_res, _args) in BACKEND_SYMBOLS.items():
    _fn = getattr(lib, _name)
    _fn.restype = _res
    _fn.argtypes = _args


def check(status):
    if status == VDNN_OK:
        return
    msg = lib.vdnn_last_error().decode("utf-8", "replace")
    if status == VDNN_OOM:
        raise OutOfMemory(status, msg)
    raise BackendError(status, msg)


def profile_enable(ctx_handle, on):
    check(lib.vdnn_profile_enable(ctx_handle, int(on)))


def profile_collect(ctx_handle):
    """{kernel class: {launches, ms, flops, bytes}} since profiling was enabled (synchronises)."""
    arr = (ProfileEntry * 64)()
    n = _i()
    check(lib.vdnn_profile_collect(ctx_handle, arr, 64, C.byref(n)))
    return {arr[i].name.decode(): {"launches": int(arr[i].launches), "ms": arr[i].ms, "flops": arr[i].flops, "bytes": arr[i].bytes}
            for i in range(min(n.value, 64))}


def profile_intervals(ctx_handle, capacity=4096):
    """[(kernel class, stream 0..4, start ms, stop ms)] of the launches timed since profiling was enabled (synchronises)."""
    arr = (ProfileInterval * capacity)()
    n = _i()
    check(lib.vdnn_profile_intervals(ctx_handle, arr, capacity, C.byref(n)))
    return [(arr[i].name.decode(), arr[i].stream, arr[i].start_ms, arr[i].stop_ms) for i in range(min(n.value, capacity))]


def zvc_traffic(ctx_handle):
    """(bytes of the tensors offloaded with zero-value compression, bytes that crossed the link for them)"""
    t, l = C.c_ulonglong(), C.c_ulonglong()
    check(lib.vdnn_zvc_traffic(ctx_handle, C.byref(t), C.byref(l)))
    return t.value, l.value


class DeviceBuffer:
    """A block of the context's pool."""

    def __init__(self, ctx, nbytes):
        self.ctx = ctx
        self.nbytes = int(nbytes)
        p = _vp()
        check(lib.vdnn_pool_malloc(ctx.handle, C.byref(p), self.nbytes))
        self.ptr = p.value

    def free(self):
        if self.ptr:
            check(lib.vdnn_pool_free(self.ctx.handle, self.ptr))
            self.ptr = None

    def upload(self, array):
        a = np.ascontiguousarray(array)
        assert a.nbytes <= self.nbytes
        check(lib.vdnn_memcpy_h2d(self.ctx.handle, self.ptr, a.ctypes.data, a.nbytes))
        return self

    def download(self, shape, dtype=np.float32):
        out = np.empty(shape, dtype)
        assert out.nbytes <= self.nbytes
        check(lib.vdnn_memcpy_d2h(self.ctx.handle, out.ctypes.data, self.ptr, out.nbytes))
        return out


class Context:
    """One device context: streams + pool. plan_only=True touches no device."""

    def __init__(self, device=0, pool_bytes=2 << 30, plan_only=False):
        h = _vp()
        check(lib.vdnn_ctx_create(C.byref(h), device, VDNN_CTX_PLAN_ONLY if plan_only else 0))
        self.handle = h.value
        self.plan_only = plan_only
        if pool_bytes:
            check(lib.vdnn_pool_init(self.handle, int(pool_bytes)))

    def close(self):
        if self.handle:
            lib.vdnn_ctx_destroy(self.handle)
            self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def alloc(self, nbytes):
        return DeviceBuffer(self, nbytes)

    def to_device(self, array, dtype=np.float32):
        a = np.ascontiguousarray(array, dtype)
        return DeviceBuffer(self, max(a.nbytes, 4)).upload(a)

    def synchronize(self):
        check(lib.vdnn_device_synchronize(self.handle))

    def pool_info(self):
        f, t = C.c_size_t(), C.c_size_t()
        check(lib.vdnn_pool_info(self.handle, C.byref(f), C.byref(t)))
        return f.value, t.value

    def pool_peak(self):
        a, b = C.c_size_t(), C.c_size_t()
        check(lib.vdnn_pool_peak(self.handle, C.byref(a), C.byref(b)))
        return a.value, b.value

    def live_blocks(self):
        n = C.c_size_t()
        check(lib.vdnn_pool_live_blocks(self.handle, C.byref(n)))
        return n.value
