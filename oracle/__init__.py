"""TEST INFRASTRUCTURE: ctypes binding of the CPU checker (oracle/liboracle.so).

Only tests, the smoke check and the bench's cpu_baseline leg may import this package. It restates the
reference's layer math on the CPU (see vdnn_oracle.h for what each function follows and what pins it).
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")


def build():
    """Compile the checker with gcc (make -C oracle)."""
    subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"], stdout=subprocess.DEVNULL)


def build_description():
    """How the checker was compiled, for whoever reports its speed."""
    flags = "?"
    for line in open(os.path.join(_HERE, "Makefile")):
        if line.startswith("CFLAGS"):
            flags = line.split("=", 1)[1].strip()
    how = ("stride-1 convolutions as im2col + cache-blocked SGEMM (6x16 AVX2/FMA micro-kernel, packed panels, OpenMP over samples x pixel blocks)"
           if lib.orc_get_blocked_gemm() else "direct loops with OpenMP over output planes")
    return "C port of the layer math, %s, gcc %s" % (how, flags)


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    return C.CDLL(_LIB_PATH)


lib = _load()


class Shape(C.Structure):
    _fields_ = [(k, C.c_int) for k in ("n", "c", "h", "w", "k", "r", "s", "pad_h", "pad_w", "stride_h", "stride_w")]


class LayerDesc(C.Structure):
    _fields_ = [("type", C.c_int), ("g", Shape), ("n_out", C.c_int), ("c_out", C.c_int),
                ("h_out", C.c_int), ("w_out", C.c_int)]


_f = C.POINTER(C.c_float)
_i = C.POINTER(C.c_int32)
_S = C.POINTER(Shape)


def _sig(name, res, *args):
    fn = getattr(lib, name)
    fn.restype = res
    fn.argtypes = list(args)
    return fn


_sig("orc_set_accumulate_double", None, C.c_int)
_sig("orc_get_accumulate_double", C.c_int)
_sig("orc_set_blocked_gemm", None, C.c_int)
_sig("orc_get_blocked_gemm", C.c_int)
_sig("orc_set_threads", None, C.c_int)
_sig("orc_get_threads", C.c_int)
_sig("orc_out_dim", C.c_int, C.c_int, C.c_int, C.c_int, C.c_int)
_sig("orc_conv_fwd", None, _S, _f, _f, _f, _f)
_sig("orc_conv_bwd_data", None, _S, _f, _f, _f)
_sig("orc_conv_bwd_bias_sgd", None, _S, _f, _f, C.c_float)
_sig("orc_conv_bwd_filter_sgd", None, _S, _f, _f, _f, C.c_float)
_sig("orc_conv_fwd_brute", None, _S, _f, _f, _f, _f)
_sig("orc_conv_bwd_data_brute", None, _S, _f, _f, _f)
_sig("orc_conv_bwd_filter_brute", None, _S, _f, _f, _f)
_sig("orc_fc_fwd", None, C.c_int, C.c_int, C.c_int, _f, _f, _f, _f)
_sig("orc_fc_bwd_data", None, C.c_int, C.c_int, C.c_int, _f, _f, _f)
_sig("orc_fc_bwd_weight_sgd", None, C.c_int, C.c_int, C.c_int, _f, _f, _f, C.c_float)
_sig("orc_fc_bwd_bias_sgd", None, C.c_int, C.c_int, _f, _f, C.c_float)
_sig("orc_relu_fwd", None, C.c_size_t, _f, _f)
_sig("orc_relu_bwd", None, C.c_size_t, _f, _f, _f, _f)
for _name in ("orc_tanh_fwd", "orc_sigmoid_fwd", "orc_round_bf16"):
    _sig(_name, None, C.c_size_t, _f, _f)
for _name in ("orc_tanh_bwd", "orc_sigmoid_bwd"):
    _sig(_name, None, C.c_size_t, _f, _f, _f)
_sig("orc_maxpool_fwd", None, _S, _f, _f)
_sig("orc_maxpool_bwd", None, _S, _f, _f, _f, _f)
_sig("orc_lrn_fwd", None, C.c_int, C.c_int, C.c_int, _f, _f)
_sig("orc_lrn_bwd", None, C.c_int, C.c_int, C.c_int, _f, _f, _f, _f)
_sig("orc_softmax_fwd", None, C.c_int, C.c_int, _f, _f)
_sig("orc_softmax_bwd", None, C.c_int, C.c_int, _f, _f, _f)
_sig("orc_sub", None, C.c_size_t, _f, _f, _f)
_sig("orc_softmax_ce_fwd", C.c_float, C.c_int, C.c_int, _f, _i, _f)
_sig("orc_softmax_ce_bwd", None, C.c_int, C.c_int, _f, _i, _f)
_sig("orc_cross_entropy_dense", C.c_float, C.c_int, C.c_int, _f, _f)
_sig("orc_rng_u64", C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64)
_sig("orc_fill_normal", None, _f, C.c_size_t, C.c_uint64, C.c_uint64, C.c_float, C.c_float)
_sig("orc_fill_uniform", None, _f, C.c_size_t, C.c_uint64, C.c_uint64, C.c_float, C.c_float)
_sig("orc_fill_labels", None, _i, C.c_size_t, C.c_uint64, C.c_uint64, C.c_int)
_sig("orc_net_create", C.c_void_p, C.c_int, C.c_int)
_sig("orc_net_create_custom", C.c_void_p, C.POINTER(LayerDesc), C.c_int)
_sig("orc_net_destroy", None, C.c_void_p)
_sig("orc_net_num_layers", C.c_int, C.c_void_p)
_sig("orc_net_layer_desc", None, C.c_void_p, C.c_int, C.POINTER(LayerDesc))
_sig("orc_net_init_seeded", None, C.c_void_p, C.c_uint64)
_sig("orc_net_set_bf16", None, C.c_void_p, C.c_int)
_sig("orc_net_filter_count", C.c_size_t, C.c_void_p, C.c_int)
_sig("orc_net_bias_count", C.c_size_t, C.c_void_p, C.c_int)
for _n in ("orc_net_filter", "orc_net_bias", "orc_net_dst", "orc_net_grad"):
    _sig(_n, _f, C.c_void_p, C.c_int)
_sig("orc_net_input", _f, C.c_void_p)
_sig("orc_net_label", _f, C.c_void_p)
_sig("orc_net_set_labels", None, C.c_void_p, _i)
_sig("orc_net_forward", C.c_float, C.c_void_p)
_sig("orc_net_backward", None, C.c_void_p)


def shape(n, c, h, w, k=0, r=0, s=0, pad_h=0, pad_w=0, stride_h=1, stride_w=1):
    return Shape(n, c, h, w, k, r, s, pad_h, pad_w, stride_h, stride_w)


def out_dim(i, pad, win, stride):
    return lib.orc_out_dim(i, pad, win, stride)


def _p(a):
    return None if a is None else a.ctypes.data_as(_f)


def _pi(a):
    return a.ctypes.data_as(_i)


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def set_accumulate_double(on):
    lib.orc_set_accumulate_double(1 if on else 0)


def set_threads(n):
    lib.orc_set_threads(int(n))


def set_blocked_gemm(on):
    """Stride-1 convolutions through im2col + blocked SGEMM (the timed CPU baseline) instead of the direct loops."""
    lib.orc_set_blocked_gemm(int(bool(on)))


def get_threads():
    return lib.orc_get_threads()


def conv_out_shape(g):
    return (g.n, g.k, out_dim(g.h, g.pad_h, g.r, g.stride_h), out_dim(g.w, g.pad_w, g.s, g.stride_w))


def conv_fwd(g, x, w, bias=None, brute=False):
    x, w, bias = _f32(x), _f32(w), _f32(bias)
    y = np.empty(conv_out_shape(g), np.float32)
    (lib.orc_conv_fwd_brute if brute else lib.orc_conv_fwd)(C.byref(g), _p(x), _p(w), _p(bias), _p(y))
    return y


def conv_bwd_data(g, dy, w, brute=False):
    dy, w = _f32(dy), _f32(w)
    dx = np.empty((g.n, g.c, g.h, g.w), np.float32)
    (lib.orc_conv_bwd_data_brute if brute else lib.orc_conv_bwd_data)(C.byref(g), _p(dy), _p(w), _p(dx))
    return dx


def conv_bwd_filter_brute(g, x, dy):
    x, dy = _f32(x), _f32(dy)
    dw = np.empty((g.k, g.c, g.r, g.s), np.float32)
    lib.orc_conv_bwd_filter_brute(C.byref(g), _p(x), _p(dy), _p(dw))
    return dw


def conv_bwd_filter_sgd(g, x, dy, w, alpha):
    x, dy = _f32(x), _f32(dy)
    w = np.array(w, dtype=np.float32, order="C", copy=True)
    lib.orc_conv_bwd_filter_sgd(C.byref(g), _p(x), _p(dy), _p(w), alpha)
    return w


def conv_bwd_bias_sgd(g, dy, bias, alpha):
    dy = _f32(dy)
    bias = np.array(bias, dtype=np.float32, order="C", copy=True)
    lib.orc_conv_bwd_bias_sgd(C.byref(g), _p(dy), _p(bias), alpha)
    return bias


def fc_fwd(x, w, bias=None):
    x, w, bias = _f32(x), _f32(w), _f32(bias)
    n, cin = x.shape
    cout = w.shape[0]
    y = np.empty((n, cout), np.float32)
    lib.orc_fc_fwd(n, cin, cout, _p(x), _p(w), _p(bias), _p(y))
    return y


def fc_bwd_data(dy, w):
    dy, w = _f32(dy), _f32(w)
    n, cout = dy.shape
    cin = w.shape[1]
    dx = np.empty((n, cin), np.float32)
    lib.orc_fc_bwd_data(n, cin, cout, _p(dy), _p(w), _p(dx))
    return dx


def fc_bwd_weight_sgd(x, dy, w, alpha):
    x, dy = _f32(x), _f32(dy)
    w = np.array(w, dtype=np.float32, order="C", copy=True)
    lib.orc_fc_bwd_weight_sgd(x.shape[0], x.shape[1], dy.shape[1], _p(x), _p(dy), _p(w), alpha)
    return w


def fc_bwd_bias_sgd(dy, bias, alpha):
    dy = _f32(dy)
    bias = np.array(bias, dtype=np.float32, order="C", copy=True)
    lib.orc_fc_bwd_bias_sgd(dy.shape[0], dy.shape[1], _p(dy), _p(bias), alpha)
    return bias


def relu_fwd(x):
    x = _f32(x)
    y = np.empty_like(x)
    lib.orc_relu_fwd(x.size, _p(x), _p(y))
    return y


def relu_bwd(x, y, dy):
    x, y, dy = _f32(x), _f32(y), _f32(dy)
    dx = np.empty_like(dy)
    lib.orc_relu_bwd(dy.size, _p(x), _p(y), _p(dy), _p(dx))
    return dx


def _act_fwd(fn, x):
    x = _f32(x)
    y = np.empty_like(x)
    fn(x.size, _p(x), _p(y))
    return y


def _act_bwd(fn, y, dy):
    y, dy = _f32(y), _f32(dy)
    dx = np.empty_like(dy)
    fn(dy.size, _p(y), _p(dy), _p(dx))
    return dx


def round_bf16(x):
    """x rounded to the nearest bfloat16 (ties to even), as float32."""
    return _act_fwd(lib.orc_round_bf16, x)


def tanh_fwd(x):
    return _act_fwd(lib.orc_tanh_fwd, x)


def tanh_bwd(y, dy):
    return _act_bwd(lib.orc_tanh_bwd, y, dy)


def sigmoid_fwd(x):
    return _act_fwd(lib.orc_sigmoid_fwd, x)


def sigmoid_bwd(y, dy):
    return _act_bwd(lib.orc_sigmoid_bwd, y, dy)


def pool_out_shape(g):
    return (g.n, g.c, out_dim(g.h, g.pad_h, g.r, g.stride_h), out_dim(g.w, g.pad_w, g.s, g.stride_w))


def maxpool_fwd(g, x):
    x = _f32(x)
    y = np.empty(pool_out_shape(g), np.float32)
    lib.orc_maxpool_fwd(C.byref(g), _p(x), _p(y))
    return y


def maxpool_bwd(g, x, y, dy):
    x, y, dy = _f32(x), _f32(y), _f32(dy)
    dx = np.empty_like(x)
    lib.orc_maxpool_bwd(C.byref(g), _p(x), _p(y), _p(dy), _p(dx))
    return dx


def lrn_fwd(x):
    x = _f32(x)
    n, c = x.shape[:2]
    y = np.empty_like(x)
    lib.orc_lrn_fwd(n, c, x[0, 0].size, _p(x), _p(y))
    return y


def lrn_bwd(x, y, dy):
    x, y, dy = _f32(x), _f32(y), _f32(dy)
    n, c = x.shape[:2]
    dx = np.empty_like(x)
    lib.orc_lrn_bwd(n, c, x[0, 0].size, _p(x), _p(y), _p(dy), _p(dx))
    return dx


def softmax_fwd(x):
    x = _f32(x)
    y = np.empty_like(x)
    lib.orc_softmax_fwd(x.shape[0], x[0].size, _p(x), _p(y))
    return y


def softmax_bwd(y, dy):
    y, dy = _f32(y), _f32(dy)
    dx = np.empty_like(y)
    lib.orc_softmax_bwd(y.shape[0], y[0].size, _p(y), _p(dy), _p(dx))
    return dx


def softmax_ce_fwd(logits, labels):
    logits = _f32(logits)
    labels = np.ascontiguousarray(labels, np.int32)
    prob = np.empty_like(logits)
    loss = lib.orc_softmax_ce_fwd(logits.shape[0], logits.shape[1], _p(logits), _pi(labels), _p(prob))
    return prob, float(loss)


def softmax_ce_bwd(prob, labels):
    prob = _f32(prob)
    labels = np.ascontiguousarray(labels, np.int32)
    d = np.empty_like(prob)
    lib.orc_softmax_ce_bwd(prob.shape[0], prob.shape[1], _p(prob), _pi(labels), _p(d))
    return d


def cross_entropy_dense(prob, target):
    prob, target = _f32(prob), _f32(target)
    return float(lib.orc_cross_entropy_dense(prob.shape[0], prob[0].size, _p(prob), _p(target)))


def fill_normal(count, seed, stream, mean=0.0, std=1.0):
    a = np.empty(count, np.float32)
    lib.orc_fill_normal(_p(a), count, seed, stream, mean, std)
    return a


def fill_uniform(count, seed, stream, lo, hi):
    a = np.empty(count, np.float32)
    lib.orc_fill_uniform(_p(a), count, seed, stream, lo, hi)
    return a


def fill_labels(count, seed, stream, classes):
    a = np.empty(count, np.int32)
    lib.orc_fill_labels(_pi(a), count, seed, stream, classes)
    return a


class Net:
    """One of the reference's networks (or an explicit layer table) on the CPU checker."""

    def __init__(self, cnn=None, batch=0, layers=None):
        if layers is not None:
            arr = (LayerDesc * len(layers))(*layers)
            self._h = lib.orc_net_create_custom(arr, len(layers))
        else:
            self._h = lib.orc_net_create(int(cnn), int(batch))
        if not self._h:
            raise ValueError("unsupported network")
        self.num_layers = lib.orc_net_num_layers(self._h)
        self.desc = []
        for l in range(self.num_layers):
            d = LayerDesc()
            lib.orc_net_layer_desc(self._h, l, C.byref(d))
            self.desc.append(d)

    def close(self):
        if self._h:
            lib.orc_net_destroy(self._h)
            self._h = None

    def __del__(self):
        self.close()

    def _view(self, ptr, shape):
        n = int(np.prod(shape))
        if not ptr or n == 0:
            return None
        return np.ctypeslib.as_array(ptr, shape=(n,)).reshape(shape)

    def set_bf16(self, on=True):
        lib.orc_net_set_bf16(self._h, int(on))

    def init_seeded(self, seed):
        lib.orc_net_init_seeded(self._h, seed)

    def src_shape(self, l):
        g = self.desc[l].g
        return (g.n, g.c, g.h, g.w)

    def dst_shape(self, l):
        d = self.desc[l]
        return (d.n_out, d.c_out, d.h_out, d.w_out)

    def filter(self, l):
        g = self.desc[l].g
        if lib.orc_net_filter_count(self._h, l) == 0:
            return None
        return self._view(lib.orc_net_filter(self._h, l), (g.k, g.c, g.r, g.s))

    def bias(self, l):
        cnt = lib.orc_net_bias_count(self._h, l)
        return self._view(lib.orc_net_bias(self._h, l), (cnt,)) if cnt else None

    def input(self):
        return self._view(lib.orc_net_input(self._h), self.src_shape(0))

    def label(self):
        return self._view(lib.orc_net_label(self._h), self.dst_shape(self.num_layers - 1))

    def set_labels(self, labels):
        labels = np.ascontiguousarray(labels, np.int32)
        lib.orc_net_set_labels(self._h, _pi(labels))

    def forward(self):
        return float(lib.orc_net_forward(self._h))

    def backward(self):
        lib.orc_net_backward(self._h)

    def dst(self, l):
        return self._view(lib.orc_net_dst(self._h, l), self.dst_shape(l))

    def grad(self, l):
        return self._view(lib.orc_net_grad(self._h, l), self.src_shape(l))
