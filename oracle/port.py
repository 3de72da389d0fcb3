"""numpy front end of the plain-C restatement (excalibur_oracle.c). Test infrastructure only."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libexcalibur_oracle.so")

ACT_NONE, ACT_RELU, ACT_RELU6_ZEROING, ACT_SIGMOID, ACT_MISH = 0, 1, 3, 4, 5
POOL_MAX, POOL_AVE = 0, 1
ELT_PROD, ELT_SUM, ELT_MAX = 0, 1, 2


class Geom(ctypes.Structure):
    _fields_ = [(k, ctypes.c_int) for k in
                ("n", "c", "h", "w", "k", "kh", "kw", "sh", "sw", "pt", "pb", "pl", "pr", "groups")]


def build():
    subprocess.check_call(["make", "-s", "-C", _HERE, "oracle"])


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        L.exo_float32_to_int8.restype = ctypes.c_int8
        L.exo_float32_to_int8.argtypes = [ctypes.c_float]
        L.exo_dequant_scale.restype = ctypes.c_float
        L.exo_dequant_scale.argtypes = [ctypes.c_float, ctypes.c_float]
        L.exo_float32_to_float16.restype = ctypes.c_uint16
        L.exo_float32_to_float16.argtypes = [ctypes.c_float]
        L.exo_float16_to_float32.restype = ctypes.c_float
        L.exo_float16_to_float32.argtypes = [ctypes.c_uint16]
        L.exo_pool_out_dim.restype = ctypes.c_int
        L.exo_out_dim.restype = ctypes.c_int
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p) if a is not None else None


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def geom(x_shape, k, kh, kw=None, stride=1, pad=0, groups=1):
    kw = kh if kw is None else kw
    sh, sw = (stride, stride) if np.isscalar(stride) else stride
    pt, pb, pl, pr = (pad,) * 4 if np.isscalar(pad) else pad
    n, c, h, w = x_shape
    return Geom(n, c, h, w, k, kh, kw, sh, sw, pt, pb, pl, pr, groups)


def out_hw(g):
    L = lib()
    return (L.exo_out_dim(g.h, g.pt, g.pb, g.kh, g.sh), L.exo_out_dim(g.w, g.pl, g.pr, g.kw, g.sw))


def float32_to_int8(v):
    return int(lib().exo_float32_to_int8(float(np.float32(v))))


def quantize(x, fs):
    x = _f32(x)
    fs = _f32(np.atleast_1d(fs))
    n, c, h, w = x.shape
    q = np.empty(x.shape, np.int8)
    lib().exo_quantize_f32_i8(_p(x), _p(q), n, c, h * w, _p(fs), fs.size)
    return q


def conv2d_i8_acc(q, w, g):
    q = np.ascontiguousarray(q, np.int8)
    w = np.ascontiguousarray(w, np.int8)
    oh, ow = out_hw(g)
    acc = np.empty((g.n, g.k, oh, ow), np.int32)
    lib().exo_conv2d_i8_acc(_p(q), _p(w), _p(acc), ctypes.byref(g))
    return acc


def dequant_scale(ws, fs):
    return np.float32(lib().exo_dequant_scale(float(np.float32(ws)), float(np.float32(fs))))


def dequant_scales(ws, fs, k):
    ws = np.broadcast_to(_f32(np.atleast_1d(ws)), (k,)) if np.size(ws) == 1 else _f32(ws)
    fs = np.broadcast_to(_f32(np.atleast_1d(fs)), (k,)) if np.size(fs) == 1 else _f32(fs)
    return np.array([dequant_scale(ws[i], fs[i]) for i in range(k)], np.float32)


def dequant(acc, ws, fs, bias):
    """fmaf((float)acc, scale_k, bias_k) over an NCHW int32 accumulator tensor."""
    acc = np.ascontiguousarray(acc, np.int32)
    n, k, h, w = acc.shape
    ws = _f32(np.atleast_1d(ws))
    fs = _f32(np.atleast_1d(fs))
    bias = _f32(bias)
    y = np.empty(acc.shape, np.float32)
    lib().exo_dequant_i32_f32(_p(acc), _p(y), n, k, h * w, _p(ws), ws.size, _p(fs), fs.size, _p(bias))
    return y


def conv2d_i8(x, w, bias, ws, fs, act, g, want_acc=False):
    x = _f32(x)
    w = np.ascontiguousarray(w, np.int8)
    bias = _f32(bias)
    ws = _f32(np.atleast_1d(ws))
    fs = _f32(np.atleast_1d(fs))
    oh, ow = out_hw(g)
    y = np.empty((g.n, g.k, oh, ow), np.float32)
    acc = np.empty((g.n, g.k, oh, ow), np.int32) if want_acc else None
    lib().exo_conv2d_i8(_p(x), _p(w), _p(bias), _p(ws), ws.size, _p(fs), fs.size, int(act), _p(y), _p(acc),
                        ctypes.byref(g))
    return (y, acc) if want_acc else y


def conv2d_f32(x, w, bias, act, g):
    x, w, bias = _f32(x), _f32(w), _f32(bias)
    oh, ow = out_hw(g)
    y = np.empty((g.n, g.k, oh, ow), np.float32)
    lib().exo_conv2d_f32(_p(x), _p(w), _p(bias), int(act), _p(y), ctypes.byref(g))
    return y


def dw_dequant_weights(w, ws):
    w = np.ascontiguousarray(w, np.int8)
    ws = _f32(ws)
    k = w.shape[0]
    wf = np.empty(w.shape, np.float32)
    lib().exo_dw_dequant_weights(_p(w), _p(wf), k, w.size // k, _p(ws))
    return wf


def dwconv_f32(x, w, bias, act, g):
    x, w, bias = _f32(x), _f32(w), _f32(bias)
    oh, ow = out_hw(g)
    y = np.empty((g.n, g.k, oh, ow), np.float32)
    lib().exo_dwconv_f32(_p(x), _p(w), _p(bias), int(act), _p(y), ctypes.byref(g))
    return y


def pool_out_hw(h, w, kh, kw, sh, sw, pt, pb, pl, pr, pad_mode):
    L = lib()
    return (L.exo_pool_out_dim(h, pt, pb, kh, sh, pad_mode), L.exo_pool_out_dim(w, pl, pr, kw, sw, pad_mode))


def pool2d(x, ptype, kernel=0, stride=1, pad=0, global_pool=False, pad_mode=1, count_include_pad=0):
    x = _f32(x)
    n, c, h, w = x.shape
    kh, kw = (kernel, kernel) if np.isscalar(kernel) else kernel
    sh, sw = (stride, stride) if np.isscalar(stride) else stride
    pt, pb, pl, pr = (pad,) * 4 if np.isscalar(pad) else pad
    if global_pool:
        oh, ow = 1, 1
    else:
        oh, ow = pool_out_hw(h, w, kh, kw, sh, sw, pt, pb, pl, pr, pad_mode)
    y = np.empty((n, c, oh, ow), np.float32)
    lib().exo_pool2d_f32(_p(x), _p(y), n, c, h, w, int(ptype), kh, kw, sh, sw, pt, pb, pl, pr, int(global_pool),
                         int(pad_mode), int(count_include_pad))
    return y


def eltwise(inputs, etype, coeffs=None):
    arrs = [_f32(a) for a in inputs]
    ptrs = (ctypes.c_void_p * len(arrs))(*[a.ctypes.data for a in arrs])
    co = _f32(coeffs)
    y = np.empty(arrs[0].shape, np.float32)
    lib().exo_eltwise_f32(ptrs, len(arrs), _p(co), int(etype), _p(y), ctypes.c_long(y.size))
    return y


def binaryop_add(a, b):
    a, b = _f32(a), _f32(b)
    y = np.empty(a.shape, np.float32)
    lib().exo_binaryop_add_f32(_p(a), _p(b), _p(y), ctypes.c_long(y.size))
    return y


def relu(x):
    x = _f32(x)
    y = np.empty(x.shape, np.float32)
    lib().exo_relu_f32(_p(x), _p(y), ctypes.c_long(y.size))
    return y


def activation(x, act):
    y = _f32(x).copy()
    lib().exo_activation_f32(_p(y), ctypes.c_long(y.size), int(act))
    return y


def innerproduct(x, w, bias):
    x, w, bias = _f32(x), _f32(w), _f32(bias)
    m = x.shape[0]
    k_in = x.size // m
    n_out = w.size // k_in
    y = np.empty((m, n_out, 1, 1), np.float32)
    lib().exo_innerproduct_f32(_p(x), _p(w), _p(bias), _p(y), m, n_out, k_in)
    return y


def float2half(x):
    x = _f32(x)
    y = np.empty(x.shape, np.uint16)
    lib().exo_float2half(_p(x), _p(y), x.size)
    return y


def half2float(x):
    x = np.ascontiguousarray(x, np.uint16)
    y = np.empty(x.shape, np.float32)
    lib().exo_half2float(_p(x), _p(y), x.size)
    return y


# ---- activation / glue layers ----
def _unary(fn, x, *scalars):
    x = _f32(x)
    y = np.empty(x.shape, np.float32)
    fn(_p(x), _p(y), ctypes.c_long(y.size), *[ctypes.c_float(float(s)) for s in scalars])
    return y


def hardswish(x, alpha=1.0 / 6.0, beta=0.5):
    return _unary(lib().exo_hardswish_f32, x, alpha, beta)


def leakyrelu(x, alpha):
    return _unary(lib().exo_leakyrelu_f32, x, alpha)


def sigmoid(x):
    return _unary(lib().exo_sigmoid_f32, x)


def hardsigmoid(x, alpha=0.2, beta=0.5):
    return _unary(lib().exo_hardsigmoid_f32, x, alpha, beta)


def binaryop(a, b, op):
    """BinaryOp ADD / SUB / MUL / DIV (op 0..3) with the reference's broadcasting rules; the result has the shape of the
    operand the reference calls the larger one."""
    a, b = _f32(a), _f32(b)
    sa = (ctypes.c_int * 4)(*a.shape)
    sb = (ctypes.c_int * 4)(*b.shape)
    so = (ctypes.c_int * 4)()
    y = np.empty(max(a.size, b.size), np.float32)
    if lib().exo_binaryop_f32(int(op), _p(a), sa, _p(b), sb, _p(y), so) != 0:
        raise NotImplementedError(f"BinaryOp on shapes {a.shape} and {b.shape}")
    return y.reshape(tuple(so))


def clip(x, lo, hi):
    return _unary(lib().exo_clip_f32, x, lo, hi)


def softmax_channels(x):
    """Softmax over the channel axis of an NCHW tensor (the reference's only axis)."""
    x = _f32(x)
    n, c = x.shape[:2]
    y = np.empty(x.shape, np.float32)
    lib().exo_softmax_channels_f32(_p(x), _p(y), n, c, int(np.prod(x.shape[2:], dtype=np.int64)))
    return y


def transpose_hw(x):
    x = _f32(x)
    n, c, h, w = x.shape
    y = np.empty((n, c, w, h), np.float32)
    lib().exo_transpose_hw_f32(_p(x), _p(y), ctypes.c_long(n * c), h, w)
    return y


def prelu(x, slope):
    x, slope = _f32(x), _f32(slope)
    n, c, h, w = x.shape
    y = np.empty(x.shape, np.float32)
    lib().exo_prelu_f32(_p(x), _p(y), n, c, h * w, _p(slope), int(slope.size == 1))
    return y


def batchnorm(x, slope, mean, var, bias, eps=0.0):
    x = _f32(x)
    n, c, h, w = x.shape
    y = np.empty(x.shape, np.float32)
    lib().exo_batchnorm_f32(_p(x), _p(y), n, c, h * w, _p(_f32(slope)), _p(_f32(mean)), _p(_f32(var)), _p(_f32(bias)),
                            ctypes.c_float(float(eps)), None)
    return y


def input_layer(x, mean, scale):
    x = _f32(x)
    n, c, h, w = x.shape
    y = np.empty(x.shape, np.float32)
    lib().exo_input_f32(_p(x), _p(y), n, c, h * w, _p(_f32(mean)), _p(_f32(scale)))
    return y


def concat_channels(xs):
    arrs = [_f32(a) for a in xs]
    n, _, h, w = arrs[0].shape
    ptrs = (ctypes.c_void_p * len(arrs))(*[a.ctypes.data for a in arrs])
    ch = (ctypes.c_int * len(arrs))(*[a.shape[1] for a in arrs])
    y = np.empty((n, sum(a.shape[1] for a in arrs), h, w), np.float32)
    lib().exo_concat_channels_f32(ptrs, ch, len(arrs), n, h * w, _p(y))
    return y


def interp_nearest(x, height_scale, width_scale):
    x = _f32(x)
    n, c, h, w = x.shape
    oh, ow = int(np.float32(h) * np.float32(height_scale)), int(np.float32(w) * np.float32(width_scale))
    y = np.empty((n, c, oh, ow), np.float32)
    lib().exo_interp_nearest_f32(_p(x), _p(y), n, c, h, w, oh, ow)
    return y


def focus(x):
    x = _f32(x)
    n, c, h, w = x.shape
    y = np.empty((n, 4 * c, h // 2, w // 2), np.float32)
    lib().exo_focus_f32(_p(x), _p(y), n, c, h, w)
    return y


def deconv2d_f32(x, w, bias, stride, pad):
    """w: [C_in][K_out][kh][kw]; pad: one value or (top, bottom, left, right)."""
    x, w = _f32(x), _f32(w)
    n, c, h, wd = x.shape
    _, k, kh, kw = w.shape
    sh, sw = (stride, stride) if np.isscalar(stride) else stride
    pt, pb, pl, pr = (pad,) * 4 if np.isscalar(pad) else pad
    y = np.empty((n, k, (h - 1) * sh + kh - pt - pb, (wd - 1) * sw + kw - pl - pr), np.float32)
    lib().exo_deconv2d_f32(_p(x), _p(w), _p(_f32(bias)) if bias is not None else None, _p(y), n, c, h, wd, k, kh, kw, sh, sw, pt,
                           pb, pl, pr)
    return y
