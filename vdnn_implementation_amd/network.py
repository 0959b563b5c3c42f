"""Python mirror of the reference's host interface: class Network with forwardPropagation /
backwardPropagation (network.h:18-58), over the C ABI of include/vdnn_capi.h."""
import ctypes as C

import numpy as np

from . import enums
from .backend import lib

_vp, _sz, _i = C.c_void_p, C.c_size_t, C.c_int
_fp = C.POINTER(C.c_float)
_ip = C.POINTER(C.c_int32)


class Options(C.Structure):
    _fields_ = [("seed", C.c_uint64), ("pool_bytes", _sz), ("cap_bytes", _sz), ("plan_only", _i), ("host_sync", _i),
                ("capture", _i), ("verbose", _i), ("device", _i), ("refined_lifetimes", _i),
                ("unfused_optimizer", _i), ("defer_optimizer", _i), ("offload_lag", _i), ("prefetch_depth", _i), ("data_type", _i),
                ("fuse_activations", _i), ("keep_tail_bytes", _sz), ("prefetch_within_peak", _i), ("keep_packed_on_device", _i),
                ("plan_packed_fraction", C.c_double),
                ("compress_offload", _i), ("hbm_budget_bytes", _sz), ("in_place_backward", _i), ("recompute_first_layer", _i),
                ("plan_link_bytes", _sz)]


class LayerSpec(C.Structure):
    _fields_ = [(k, _i) for k in ("type", "n", "c", "h", "w", "pad_h", "pad_w", "stride_h", "stride_w", "k", "r", "s",
                                  "n_out", "c_out", "h_out", "w_out")]


class Stats(C.Structure):
    _fields_ = [(k, _sz) for k in ("peak_bytes_in_use", "peak_extent", "offload_bytes", "prefetch_bytes", "pinned_bytes",
                                   "pool_bytes", "weight_bytes")]


# every symbol include/vdnn_capi.h declares
CAPI_SYMBOLS = {
    "vdnn_network_default_options": (None, [C.POINTER(Options)]),
    "vdnn_network_create": (_vp, [_i, _i, _i, _i, C.POINTER(Options)]),
    "vdnn_network_create_custom": (_vp, [C.POINTER(LayerSpec), _i, _i, _i, C.POINTER(Options)]),
    "vdnn_network_destroy": (None, [_vp]),
    "vdnn_network_forward": (_i, [_vp, _i]),
    "vdnn_network_backward": (_i, [_vp, _i]),
    "vdnn_network_synchronize": (None, [_vp]),
    "vdnn_network_loss": (C.c_float, [_vp]),
    "vdnn_network_num_layers": (_i, [_vp]),
    "vdnn_network_batch": (_i, [_vp]),
    "vdnn_network_policy": (_i, [_vp]),
    "vdnn_network_algo": (_i, [_vp]),
    "vdnn_network_layer_spec": (_i, [_vp, _i, C.POINTER(LayerSpec)]),
    "vdnn_network_input_size": (_sz, [_vp]),
    "vdnn_network_output_size": (_sz, [_vp]),
    "vdnn_network_set_input": (None, [_vp, _fp]),
    "vdnn_network_get_input": (None, [_vp, _fp]),
    "vdnn_network_set_labels": (None, [_vp, _ip]),
    "vdnn_network_set_label_tensor": (None, [_vp, _fp]),
    "vdnn_network_set_layer_params": (_i, [_vp, _i, _fp, _fp]),
    "vdnn_network_get_layer_params": (_i, [_vp, _i, _fp, _fp]),
    "vdnn_network_get_layer_gradients": (_i, [_vp, _i, _fp, _fp]),
    "vdnn_network_apply_gradients": (_i, [_vp]),
    "vdnn_network_train": (_i, [_vp, _i, _i, _fp]),
    "vdnn_network_filter_count": (_sz, [_vp, _i]),
    "vdnn_network_bias_count": (_sz, [_vp, _i]),
    "vdnn_network_captured_dst": (_sz, [_vp, _i, _fp, _sz]),
    "vdnn_network_captured_grad": (_sz, [_vp, _i, _fp, _sz]),
    "vdnn_network_stats_get": (None, [_vp, C.POINTER(Stats)]),
    "vdnn_network_reset_peak": (None, [_vp]),
    "vdnn_network_is_offloaded": (_i, [_vp, _i]),
    "vdnn_network_grad_over_src": (_i, [_vp, _i]),
    "vdnn_network_offload_lag": (_i, [_vp]),
    "vdnn_network_recomputed_layer": (_i, [_vp]),
    "vdnn_network_placement": (_i, [_vp, _i]),
    "vdnn_network_plan_feasible": (_i, [_vp]),
    "vdnn_network_plan_peak_bytes": (_sz, [_vp]),
    "vdnn_network_prefetch_trace": (_i, [_vp, C.POINTER(_i), C.POINTER(_i), _i]),
    "vdnn_network_max_dxdy_bytes": (_sz, [_vp]),
    "vdnn_network_max_workspace_bytes": (_sz, [_vp]),
    "vdnn_network_context": (_vp, [_vp]),
    "vdnn_parse_cnn": (_i, [C.c_char_p, C.POINTER(_i)]),
    "vdnn_parse_policy": (_i, [C.c_char_p, C.POINTER(_i)]),
    "vdnn_parse_algo": (_i, [C.c_char_p, C.POINTER(_i)]),
    "vdnn_seeded_fill_normal": (None, [_fp, _sz, C.c_uint64, C.c_uint64, C.c_float, C.c_float]),
    "vdnn_seeded_fill_labels": (None, [_ip, _sz, C.c_uint64, C.c_uint64, _i]),
}
for _name, (_res, _args) in CAPI_SYMBOLS.items():
    _fn = getattr(lib, _name)
    _fn.restype = _res
    _fn.argtypes = _args


def layer_spec(type, n, c, h, w, pad=0, stride=0, k=0, r=0, s=None):
    return LayerSpec(type, n, c, h, w, pad, pad, stride, stride, k, r, r if s is None else s, 0, 0, 0, 0)


def _f32(a):
    return np.ascontiguousarray(a, np.float32)


class Network:
    """Network(cnnType, vdnnType, algoMode, batchSize) as in network.h:18-22; `layers` builds from an
    explicit table instead of one of the built-in networks."""

    def __init__(self, cnn=None, policy=enums.BASELINE, algo=enums.VDNN_MEMORY_OPT_ALGO, batch=0, layers=None, seed=1,
                 pool_bytes=0, cap_bytes=0, plan_only=False, host_sync=False, capture=False, verbose=False, device=0,
                 refined=False, unfused_optimizer=False, defer_optimizer=False, bf16=False, offload_lag=0, prefetch_depth=1,
                 fuse=False, compress=False, keep_tail_bytes=0, prefetch_within_peak=False, keep_packed=False,
                 plan_packed_fraction=0.0, hbm_budget_bytes=0, in_place=False, recompute_first=False, plan_link_bytes=0):
        o = Options()
        lib.vdnn_network_default_options(C.byref(o))
        o.seed, o.pool_bytes, o.cap_bytes = seed, int(pool_bytes), int(cap_bytes)
        o.plan_only, o.host_sync, o.capture, o.verbose, o.device = int(plan_only), int(host_sync), int(capture), int(verbose), device
        o.refined_lifetimes = int(refined)
        o.unfused_optimizer, o.defer_optimizer = int(unfused_optimizer), int(defer_optimizer)
        o.data_type = 1 if bf16 else 0  # VDNN_DTYPE_BF16 / VDNN_DTYPE_F32
        o.offload_lag, o.prefetch_depth = int(offload_lag), int(prefetch_depth)
        o.fuse_activations = int(fuse)
        o.compress_offload = int(compress)
        o.keep_tail_bytes = int(keep_tail_bytes)
        o.prefetch_within_peak = int(prefetch_within_peak)
        o.keep_packed_on_device = int(keep_packed)
        o.plan_packed_fraction = float(plan_packed_fraction)
        o.hbm_budget_bytes = int(hbm_budget_bytes)
        o.in_place_backward = int(in_place)
        o.recompute_first_layer = int(recompute_first)
        o.plan_link_bytes = int(plan_link_bytes)
        if layers is not None:
            arr = (LayerSpec * len(layers))(*layers)
            self._h = lib.vdnn_network_create_custom(arr, len(layers), policy, algo, C.byref(o))
        else:
            self._h = lib.vdnn_network_create(int(cnn), policy, algo, int(batch), C.byref(o))
        if not self._h:
            raise ValueError("unsupported network")
        self.num_layers = lib.vdnn_network_num_layers(self._h)
        self.specs = []
        for l in range(self.num_layers):
            s = LayerSpec()
            lib.vdnn_network_layer_spec(self._h, l, C.byref(s))
            self.specs.append(s)

    def close(self):
        if getattr(self, "_h", None):
            lib.vdnn_network_destroy(self._h)
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        self.close()

    # ---- the reference's interface ----
    def forwardPropagation(self, isDynamic=False):
        return lib.vdnn_network_forward(self._h, int(isDynamic))

    def backwardPropagation(self, isDynamic=False):
        return lib.vdnn_network_backward(self._h, int(isDynamic))

    def getInputSize(self):
        return lib.vdnn_network_input_size(self._h)

    def getOutputSize(self):
        return lib.vdnn_network_output_size(self._h)

    def findMaxDxDySize(self):
        return lib.vdnn_network_max_dxdy_bytes(self._h)

    def findMaxWorkSpaceSize(self):
        return lib.vdnn_network_max_workspace_bytes(self._h)

    # ---- additions ----
    @property
    def batch(self):
        return lib.vdnn_network_batch(self._h)

    @property
    def policy(self):
        return lib.vdnn_network_policy(self._h)

    @property
    def algo(self):
        return lib.vdnn_network_algo(self._h)

    @property
    def context(self):
        return lib.vdnn_network_context(self._h)

    def src_shape(self, l):
        s = self.specs[l]
        return (s.n, s.c, s.h, s.w)

    def dst_shape(self, l):
        s = self.specs[l]
        return (s.n_out, s.c_out, s.h_out, s.w_out)

    def synchronize(self):
        lib.vdnn_network_synchronize(self._h)

    def loss(self):
        return float(lib.vdnn_network_loss(self._h))

    def set_input(self, x):
        x = _f32(x)
        assert x.size == self.getInputSize()
        lib.vdnn_network_set_input(self._h, x.ctypes.data_as(_fp))

    def get_input(self):
        x = np.empty(self.src_shape(0), np.float32)
        lib.vdnn_network_get_input(self._h, x.ctypes.data_as(_fp))
        return x

    def set_labels(self, labels):
        labels = np.ascontiguousarray(labels, np.int32)
        assert labels.size == self.batch
        lib.vdnn_network_set_labels(self._h, labels.ctypes.data_as(_ip))

    def set_label_tensor(self, t):
        t = _f32(t)
        assert t.size == self.getOutputSize()
        lib.vdnn_network_set_label_tensor(self._h, t.ctypes.data_as(_fp))

    def has_params(self, l):
        return lib.vdnn_network_filter_count(self._h, l) > 0

    def get_params(self, l):
        s = self.specs[l]
        w = np.empty((s.k, s.c, s.r, s.s), np.float32)
        b = np.empty(lib.vdnn_network_bias_count(self._h, l), np.float32)
        assert w.size == lib.vdnn_network_filter_count(self._h, l)
        lib.vdnn_network_get_layer_params(self._h, l, w.ctypes.data_as(_fp), b.ctypes.data_as(_fp))
        return w, b

    def get_gradients(self, l):
        """dW, db of layer l from the last backward (needs unfused_optimizer)."""
        s = self.specs[l]
        w = np.empty((s.k, s.c, s.r, s.s), np.float32)
        b = np.empty(lib.vdnn_network_bias_count(self._h, l), np.float32)
        if lib.vdnn_network_get_layer_gradients(self._h, l, w.ctypes.data_as(_fp), b.ctypes.data_as(_fp)) != 0:
            raise ValueError("layer %d keeps no gradients" % l)
        return w, b

    def applyGradients(self):
        return lib.vdnn_network_apply_gradients(self._h)

    def train(self, steps, is_dynamic=False):
        """`steps` training steps; the loss seen by each step's forward."""
        out = np.zeros(steps, np.float32)
        done = lib.vdnn_network_train(self._h, int(steps), int(is_dynamic), out.ctypes.data_as(_fp))
        return out[:done]

    def set_params(self, l, w=None, b=None):
        w = None if w is None else _f32(w)
        b = None if b is None else _f32(b)
        if w is not None:
            assert w.size == lib.vdnn_network_filter_count(self._h, l)
        if b is not None:
            assert b.size == lib.vdnn_network_bias_count(self._h, l)
        rc = lib.vdnn_network_set_layer_params(self._h, l, w.ctypes.data_as(_fp) if w is not None else None,
                                               b.ctypes.data_as(_fp) if b is not None else None)
        assert rc == 0

    def captured_dst(self, l):
        out = np.empty(self.dst_shape(l), np.float32)
        n = lib.vdnn_network_captured_dst(self._h, l, out.ctypes.data_as(_fp), out.size)
        assert n == out.size, "nothing captured for layer %d (capture=True and a step are needed)" % l
        return out

    def captured_grad(self, l):
        out = np.empty(self.src_shape(l), np.float32)
        n = lib.vdnn_network_captured_grad(self._h, l, out.ctypes.data_as(_fp), out.size)
        assert n == out.size, "nothing captured for layer %d" % l
        return out

    def stats(self):
        s = Stats()
        lib.vdnn_network_stats_get(self._h, C.byref(s))
        return {k: getattr(s, k) for k, _ in Stats._fields_}

    def reset_peak(self):
        lib.vdnn_network_reset_peak(self._h)

    def is_offloaded(self, l):
        return bool(lib.vdnn_network_is_offloaded(self._h, l))

    def grad_over_src(self, l):
        """in_place: layer l's backward writes its input gradient over its input"""
        return bool(lib.vdnn_network_grad_over_src(self._h, l))

    def offload_lag(self):
        """the offload lag in use (offload_lag, or what the placement plan chose where that is negative)"""
        return lib.vdnn_network_offload_lag(self._h)

    def recomputed_layer(self):
        """recompute_first: the layer whose input layer 0 computes again before that layer's backward, or -1"""
        return lib.vdnn_network_recomputed_layer(self._h)

    def placement(self):
        """hbm_budget_bytes: per layer, 0 = outside the plan, 1 = on the device, 2 = packed on the device, 3 = host memory."""
        return [lib.vdnn_network_placement(self._h, l) for l in range(self.num_layers)]

    def plan_feasible(self):
        return bool(lib.vdnn_network_plan_feasible(self._h))

    def plan_peak_bytes(self):
        return lib.vdnn_network_plan_peak_bytes(self._h)

    def prefetch_trace(self):
        a = (_i * 64)()
        b = (_i * 64)()
        n = lib.vdnn_network_prefetch_trace(self._h, a, b, 64)
        return [(a[i], b[i]) for i in range(n)]


def parse(model, policy, algo):
    """parseVdnnInputs (vdnn.cu:8-54): the three words of the command line to enum values."""
    out = []
    for fn, word in ((lib.vdnn_parse_cnn, model), (lib.vdnn_parse_policy, policy), (lib.vdnn_parse_algo, algo)):
        v = _i()
        if fn(word.encode(), C.byref(v)) != 0:
            raise ValueError("unknown word %r" % word)
        out.append(v.value)
    return tuple(out)
