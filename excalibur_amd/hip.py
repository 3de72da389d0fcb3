"""ctypes binding of the exhip C ABI (include/exhip.h) with numpy at the host boundary.

This is the Python face of the product library: it loads excalibur_amd/lib/libexhip.so and fails
loudly if that library or a gfx950 device is missing. There is no CPU fallback.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libexhip.so")

I8, F16, F32 = 0, 1, 2
_NP = {I8: np.int8, F16: np.uint16, F32: np.float32}


class ExhipError(RuntimeError):
    pass


class ConvDesc(ctypes.Structure):
    _fields_ = [(k, ctypes.c_int) for k in
                ("n", "c", "h", "w", "k", "kh", "kw", "sh", "sw", "pt", "pb", "pl", "pr", "act", "c_stride", "k_stride",
                 "post_relu")] + [("fs_out", ctypes.c_float), ("post_op", ctypes.c_int), ("post_alpha", ctypes.c_float),
                                  ("post_beta", ctypes.c_float), ("post_slope", ctypes.c_void_p),
                                  ("post_slope_shared", ctypes.c_int), ("residual_last", ctypes.c_int),
                                  ("post_bn_a", ctypes.c_void_p), ("post_bn_b", ctypes.c_void_p), ("exact_k", ctypes.c_int)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ExhipError(f"{LIB_PATH} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
                             "or `make -C excalibur_amd/csrc`")
        L = ctypes.CDLL(LIB_PATH)
        L.exhip_last_error.restype = ctypes.c_char_p
        L.exhip_conv_packed_bytes.restype = ctypes.c_size_t
        L.exhip_static_scratch_bytes.restype = ctypes.c_size_t
        _lib = L
    return _lib


def set_option(name, value):
    """Test / development switches of the library (exhip_set_option)."""
    _check(lib().exhip_set_option(name.encode(), int(value)))


def _check(rc):
    if rc != 0:
        raise ExhipError(f"exhip error {rc}: {lib().exhip_last_error().decode()}")


def pad_to(v, m):
    return (v + m - 1) // m * m


class DevArray:
    """A device allocation with a logical numpy shape/dtype."""

    def __init__(self, ctx, shape, dtype):
        self.ctx = ctx
        self.shape = tuple(int(s) for s in shape)
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        p = ctypes.c_void_p()
        _check(lib().exhip_malloc(ctx.h, ctypes.c_size_t(self.nbytes), ctypes.byref(p)))
        self.ptr = p

    @property
    def size(self):
        return self.nbytes // self.dtype.itemsize

    def upload(self, a):
        a = np.ascontiguousarray(a, self.dtype)
        assert a.nbytes == self.nbytes, (a.shape, self.shape)
        _check(lib().exhip_memcpy_h2d(self.ctx.h, self.ptr, a.ctypes.data_as(ctypes.c_void_p), ctypes.c_size_t(self.nbytes)))
        return self

    def download(self):
        out = np.empty(self.shape, self.dtype)
        _check(lib().exhip_memcpy_d2h(self.ctx.h, out.ctypes.data_as(ctypes.c_void_p), self.ptr, ctypes.c_size_t(self.nbytes)))
        return out

    def zero(self):
        _check(lib().exhip_memset(self.ctx.h, self.ptr, 0, ctypes.c_size_t(self.nbytes)))
        return self

    def free(self):
        if self.ptr:
            _check(lib().exhip_free(self.ctx.h, self.ptr))
            self.ptr = None

    def at(self, offset_bytes):
        """Something with a .ptr that many bytes into the allocation (an operand that starts inside a larger tensor)."""
        assert 0 <= offset_bytes < self.nbytes
        return _Inside(ctypes.c_void_p(self.ptr.value + int(offset_bytes)))


class _Inside:
    def __init__(self, ptr):
        self.ptr = ptr


class Event:
    def __init__(self):
        self.h = ctypes.c_void_p()
        _check(lib().exhip_event_create(ctypes.byref(self.h)))

    def record(self, ctx):
        _check(lib().exhip_event_record(ctx.h, self.h))

    def destroy(self):
        if self.h:
            _check(lib().exhip_event_destroy(self.h))
            self.h = None

    def elapsed_ms(self, stop):
        ms = ctypes.c_float()
        _check(lib().exhip_event_elapsed_ms(self.h, stop.h, ctypes.byref(ms)))
        return ms.value


def _ptr(a):
    return a.ptr if a is not None else None


class Ctx:
    def __init__(self, device=0):
        self.h = ctypes.c_void_p()
        _check(lib().exhip_init(int(device), ctypes.byref(self.h)))

    def close(self):
        if self.h:
            lib().exhip_destroy(self.h)
            self.h = None

    def device_name(self):
        buf = ctypes.create_string_buffer(256)
        _check(lib().exhip_device_name(self.h, buf, ctypes.c_size_t(256)))
        return buf.value.decode()

    def sync(self):
        _check(lib().exhip_sync(self.h))

    def empty(self, shape, dtype):
        return DevArray(self, shape, dtype)

    def array(self, a, dtype=None):
        a = np.ascontiguousarray(a, dtype if dtype is not None else a.dtype)
        return DevArray(self, a.shape, a.dtype).upload(a)

    # ---- layout / precision ----
    def quantize_nchw_to_nhwc_i8(self, x, fs, c_stride, fs_per_channel=None):
        n, c, h, w = x.shape
        y = self.empty((n, h, w, c_stride), np.int8)
        _check(lib().exhip_quantize_nchw_f32_to_nhwc_i8(self.h, x.ptr, n, c, h, w, ctypes.c_float(float(fs)),
                                                       _ptr(fs_per_channel), c_stride, y.ptr))
        return y

    def nchw_to_nhwc(self, x, c_stride, out="f32"):
        n, c, h, w = x.shape
        if x.dtype == np.float32 and out == "f32":
            y = self.empty((n, h, w, c_stride), np.float32)
            _check(lib().exhip_nchw_f32_to_nhwc_f32(self.h, x.ptr, n, c, h, w, c_stride, y.ptr))
        elif x.dtype == np.float32 and out == "f16":
            y = self.empty((n, h, w, c_stride), np.uint16)
            _check(lib().exhip_nchw_f32_to_nhwc_f16(self.h, x.ptr, n, c, h, w, c_stride, y.ptr))
        else:
            y = self.empty((n, h, w, c_stride), np.uint16)
            _check(lib().exhip_nchw_f16_to_nhwc_f16(self.h, x.ptr, n, c, h, w, c_stride, y.ptr))
        return y

    def nhwc_to_nchw(self, x, c, out="f32"):
        n, h, w, cs = x.shape
        if x.dtype == np.float32:
            y = self.empty((n, c, h, w), np.float32)
            _check(lib().exhip_nhwc_f32_to_nchw_f32(self.h, x.ptr, n, c, h, w, cs, y.ptr))
        elif out == "f32":
            y = self.empty((n, c, h, w), np.float32)
            _check(lib().exhip_nhwc_f16_to_nchw_f32(self.h, x.ptr, n, c, h, w, cs, y.ptr))
        else:
            y = self.empty((n, c, h, w), np.uint16)
            _check(lib().exhip_nhwc_f16_to_nchw_f16(self.h, x.ptr, n, c, h, w, cs, y.ptr))
        return y

    def f32_to_f16(self, x):
        y = self.empty(x.shape, np.uint16)
        _check(lib().exhip_f32_to_f16(self.h, x.ptr, y.ptr, ctypes.c_size_t(x.size)))
        return y

    def f16_to_f32(self, x):
        y = self.empty(x.shape, np.float32)
        _check(lib().exhip_f16_to_f32(self.h, x.ptr, y.ptr, ctypes.c_size_t(x.size)))
        return y

    # ---- convolution ----
    @staticmethod
    def conv_desc(n, c, h, w, k, kernel, stride=1, pad=0, act=0, c_stride=None, k_stride=None, post_relu=0, fs_out=0.0,
                  post_op=None, post_alpha=0.0, post_beta=0.0, residual_last=0, post_bn=None, exact_k=0):
        kh, kw = (kernel, kernel) if np.isscalar(kernel) else kernel
        sh, sw = (stride, stride) if np.isscalar(stride) else stride
        pt, pb, pl, pr = (pad,) * 4 if np.isscalar(pad) else pad
        return ConvDesc(n, c, h, w, k, kh, kw, sh, sw, pt, pb, pl, pr, act, c_stride if c_stride else c,
                        k_stride if k_stride else k, post_relu, fs_out, 0 if post_op is None else 1 + Ctx.UNARY[post_op],
                        post_alpha, post_beta, None, 0, residual_last, post_bn[0].ptr if post_bn else None,
                        post_bn[1].ptr if post_bn else None, int(exact_k))

    @staticmethod
    def conv_out_hw(d):
        oh, ow = ctypes.c_int(), ctypes.c_int()
        _check(lib().exhip_conv_out_hw(ctypes.byref(d), ctypes.byref(oh), ctypes.byref(ow)))
        return oh.value, ow.value

    def pack_conv_weights(self, d, dtype, w_oihw):
        nbytes = lib().exhip_conv_packed_bytes(ctypes.byref(d), dtype)
        if nbytes == 0:
            raise ExhipError(f"exhip_conv_packed_bytes: {lib().exhip_last_error().decode()}")
        w = np.ascontiguousarray(w_oihw, _NP[dtype])
        packed = np.empty(nbytes, np.uint8)
        _check(lib().exhip_conv_pack_weights(ctypes.byref(d), dtype, w.ctypes.data_as(ctypes.c_void_p),
                                             packed.ctypes.data_as(ctypes.c_void_p)))
        return self.array(packed)

    def conv2d_i8(self, d, x, wp, scale, bias=None, residual=None, y_i8=None, y_f32_nhwc=None, y_f32_nchw=None, acc=None):
        _check(lib().exhip_conv2d_i8(self.h, ctypes.byref(d), x.ptr, wp.ptr, scale.ptr, _ptr(bias), _ptr(residual),
                                     _ptr(y_i8), _ptr(y_f32_nhwc), _ptr(y_f32_nchw), _ptr(acc)))

    def conv2d_i8_maxpool3x3s2(self, d, pool_pad, pool_oh, pool_ow, x, wp, scale, bias=None, y_i8=None, y_f32_nhwc=None):
        _check(lib().exhip_conv2d_i8_maxpool3x3s2(self.h, ctypes.byref(d), pool_pad, pool_pad, pool_oh, pool_ow, x.ptr, wp.ptr,
                                                  scale.ptr, _ptr(bias), _ptr(y_i8), _ptr(y_f32_nhwc)))

    def stem_f32_conv_i8_maxpool3x3s2(self, d, pool_pad, pool_oh, pool_ow, x_nchw, fs_in, wp, scale, scales_nonnegative, bias=None,
                                      y_i8=None, y_f32_nhwc=None):
        """Returns False when the library leaves the shape to the quantizer + exhip_conv2d_i8_maxpool3x3s2."""
        rc = lib().exhip_stem_f32_conv_i8_maxpool3x3s2(self.h, ctypes.byref(d), pool_pad, pool_pad, pool_oh, pool_ow, x_nchw.ptr,
                                                       ctypes.c_float(fs_in), wp.ptr, scale.ptr, int(scales_nonnegative), _ptr(bias),
                                                       _ptr(y_i8), _ptr(y_f32_nhwc))
        if rc == 10002:
            return False
        _check(rc)
        return True

    def conv2d_i8_projection(self, d, x, wp, scale, bias, d_proj, x_proj, wp_proj, scale_proj, bias_proj, y_i8, y_f32_nhwc):
        """Returns False when the library leaves the pair to two exhip_conv2d_i8 calls."""
        rc = lib().exhip_conv2d_i8_projection(self.h, ctypes.byref(d), x.ptr, wp.ptr, scale.ptr, _ptr(bias), ctypes.byref(d_proj),
                                              x_proj.ptr, wp_proj.ptr, scale_proj.ptr, _ptr(bias_proj), y_i8.ptr, y_f32_nhwc.ptr)
        if rc == 10002:
            return False
        _check(rc)
        return True

    def conv2d_f16(self, d, x, wp, bias=None, residual=None, y_f16_nhwc=None, y_f16_nchw=None, y_f32_nchw=None):
        _check(lib().exhip_conv2d_f16(self.h, ctypes.byref(d), x.ptr, wp.ptr, _ptr(bias), _ptr(residual), _ptr(y_f16_nhwc),
                                      _ptr(y_f16_nchw), _ptr(y_f32_nchw)))

    def conv2d_f32(self, d, x, wp, bias=None, residual=None, y_f32_nhwc=None, y_f32_nchw=None):
        _check(lib().exhip_conv2d_f32(self.h, ctypes.byref(d), x.ptr, wp.ptr, _ptr(bias), _ptr(residual), _ptr(y_f32_nhwc),
                                      _ptr(y_f32_nchw)))

    def conv2d_direct(self, d, groups, x, y, w_f32=None, w_i8=None, fs=1.0, scale=None, bias=None):
        _check(lib().exhip_conv2d_direct_nchw(self.h, ctypes.byref(d), groups, x.ptr, _ptr(w_f32), _ptr(w_i8),
                                              ctypes.c_float(float(fs)), _ptr(scale), _ptr(bias), y.ptr))

    # ---- bandwidth-bound operators ----
    def dwconv3x3_nchw_f32(self, x, w9, bias, stride, pad, act):
        n, c, h, w = x.shape
        pt, pb, pl, pr = (pad,) * 4 if np.isscalar(pad) else pad
        oh, ow = (h + pt + pb - 3) // stride + 1, (w + pl + pr - 3) // stride + 1
        y = self.empty((n, c, oh, ow), np.float32)
        _check(lib().exhip_dwconv3x3_nchw_f32(self.h, x.ptr, w9.ptr, _ptr(bias), y.ptr, n, c, h, w, stride, pt, pb, pl, pr, act))
        return y

    def dwconv3x3_nhwc_f16(self, x, c, w9, bias, stride, pad, act):
        n, h, w, cs = x.shape
        pt, pb, pl, pr = (pad,) * 4 if np.isscalar(pad) else pad
        oh, ow = (h + pt + pb - 3) // stride + 1, (w + pl + pr - 3) // stride + 1
        y = self.empty((n, oh, ow, cs), np.uint16)
        _check(lib().exhip_dwconv3x3_nhwc_f16(self.h, x.ptr, w9.ptr, _ptr(bias), y.ptr, n, c, h, w, cs, stride, pt, pb, pl, pr,
                                              act))
        return y

    def dwconv3x3_nchw_f32_prelu(self, x, w9, bias, slope, shared, stride, pad):
        n, c, h, w = x.shape
        pt, pb, pl, pr = (pad,) * 4 if np.isscalar(pad) else pad
        oh, ow = (h + pt + pb - 3) // stride + 1, (w + pl + pr - 3) // stride + 1
        y = self.empty((n, c, oh, ow), np.float32)
        _check(lib().exhip_dwconv3x3_nchw_f32_prelu(self.h, x.ptr, w9.ptr, _ptr(bias), slope.ptr, int(shared), y.ptr, n, c, h, w,
                                                    stride, pt, pb, pl, pr))
        return y

    def dwconv3x3_nhwc_f16_prelu(self, x, c, w9, bias, slope, shared, stride, pad):
        n, h, w, cs = x.shape
        pt, pb, pl, pr = (pad,) * 4 if np.isscalar(pad) else pad
        oh, ow = (h + pt + pb - 3) // stride + 1, (w + pl + pr - 3) // stride + 1
        y = self.empty((n, oh, ow, cs), np.uint16)
        _check(lib().exhip_dwconv3x3_nhwc_f16_prelu(self.h, x.ptr, w9.ptr, _ptr(bias), slope.ptr, int(shared), y.ptr, n, c, h, w,
                                                    cs, stride, pt, pb, pl, pr))
        return y

    def dw_dequant_weights(self, w_i8, ws):
        k = w_i8.shape[0]
        wf = self.empty(w_i8.shape, np.float32)
        _check(lib().exhip_dw_dequant_weights(self.h, w_i8.ptr, ws.ptr, wf.ptr, k, w_i8.size // k))
        return wf

    @staticmethod
    def pool_out_hw(h, w, kh, kw, sh, sw, pt, pb, pl, pr, pad_mode):
        oh, ow = ctypes.c_int(), ctypes.c_int()
        _check(lib().exhip_pool_out_hw(h, w, kh, kw, sh, sw, pt, pb, pl, pr, pad_mode, ctypes.byref(oh), ctypes.byref(ow)))
        return oh.value, ow.value

    @staticmethod
    def _pool_args(h, w, kernel, stride, pad, global_pool, pad_mode):
        kh, kw = (kernel, kernel) if np.isscalar(kernel) else kernel
        sh, sw = (stride, stride) if np.isscalar(stride) else stride
        pt, pb, pl, pr = (pad,) * 4 if np.isscalar(pad) else pad
        if global_pool:  # src/Excalibur/operation_pooling.cpp:90-100
            kh, kw, sh, sw, pt, pb, pl, pr = h, w, 1, 1, 0, 0, 0, 0
        oh, ow = Ctx.pool_out_hw(h, w, kh, kw, sh, sw, pt, pb, pl, pr, pad_mode)
        return kh, kw, sh, sw, pt, pb, pl, pr, oh, ow

    def pool2d_nchw_f32(self, x, ptype, kernel=0, stride=1, pad=0, global_pool=False, pad_mode=1, count_include_pad=0):
        n, c, h, w = x.shape
        kh, kw, sh, sw, pt, pb, pl, pr, oh, ow = self._pool_args(h, w, kernel, stride, pad, global_pool, pad_mode)
        y = self.empty((n, c, oh, ow), np.float32)
        _check(lib().exhip_pool2d_nchw_f32(self.h, x.ptr, y.ptr, n, c, h, w, oh, ow, ptype, kh, kw, sh, sw, pt, pb, pl, pr,
                                           count_include_pad))
        return y

    def maxpool2d_nhwc_f32(self, x, c, kernel, stride, pad, fs_out=None, want_f32=True):
        n, h, w, cs = x.shape
        kh, kw, sh, sw, pt, pb, pl, pr, oh, ow = self._pool_args(h, w, kernel, stride, pad, False, 1)
        y = self.empty((n, oh, ow, cs), np.float32) if want_f32 else None
        yq = self.empty((n, oh, ow, cs), np.int8) if fs_out is not None else None
        _check(lib().exhip_maxpool2d_nhwc_f32(self.h, x.ptr, _ptr(y), _ptr(yq), ctypes.c_float(float(fs_out or 0.0)), n, c, h,
                                              w, cs, oh, ow, kh, kw, sh, sw, pt, pl))
        return y, yq

    def pool2d_nhwc_f16(self, x, c, ptype, kernel=0, stride=1, pad=0, global_pool=False, pad_mode=1, count_include_pad=0):
        n, h, w, cs = x.shape
        kh, kw, sh, sw, pt, pb, pl, pr, oh, ow = self._pool_args(h, w, kernel, stride, pad, global_pool, pad_mode)
        y = self.empty((n, oh, ow, cs), np.uint16)
        _check(lib().exhip_pool2d_nhwc_f16(self.h, x.ptr, y.ptr, n, c, h, w, cs, oh, ow, ptype, kh, kw, sh, sw, pt, pb, pl, pr,
                                           count_include_pad))
        return y

    def maxpool_same_nhwc_f16(self, x, k, y=None, tmp=None):
        """Stride-1 max pooling with window k and padding k // 2 on an NHWC half tensor; tmp is the caller's workspace."""
        n, h, w, c = x.shape
        y = y if y is not None else self.empty(x.shape, np.uint16)
        tmp = tmp if tmp is not None else self.empty(x.shape, np.uint16)
        _check(lib().exhip_maxpool_same_nhwc_f16(self.h, x.ptr, tmp.ptr, y.ptr, n, c, h, w, int(k)))
        return y

    def maxpool_same_nhwc_f16_static(self, x, k, y):
        """The same through the entry point that allocates nothing: y is preallocated by the caller."""
        n, h, w, c = x.shape
        _check(lib().exhip_maxpool_same_nhwc_f16_static(self.h, x.ptr, y.ptr, n, c, h, w, int(k)))
        return y

    def eltwise_f32(self, inputs, etype, coeffs=None):
        ptrs = (ctypes.c_void_p * len(inputs))(*[a.ptr.value for a in inputs])
        co = None
        if coeffs is not None:
            co = (ctypes.c_float * len(inputs))(*[float(v) for v in coeffs])
        y = self.empty(inputs[0].shape, np.float32)
        _check(lib().exhip_eltwise_f32(self.h, ptrs, len(inputs), co, etype, y.ptr, ctypes.c_size_t(y.size)))
        return y

    def add_f32(self, a, b, relu=False):
        y = self.empty(a.shape, np.float32)
        _check(lib().exhip_add_f32(self.h, a.ptr, b.ptr, y.ptr, ctypes.c_size_t(y.size), int(relu)))
        return y

    def relu_f32(self, x):
        y = self.empty(x.shape, np.float32)
        _check(lib().exhip_relu_f32(self.h, x.ptr, y.ptr, ctypes.c_size_t(y.size)))
        return y

    # ---- activation / glue layers ----
    UNARY = {"hardswish": 0, "leakyrelu": 1, "sigmoid": 2, "hardsigmoid": 3, "clip": 4}
    CHANNEL = {"prelu": 0, "batchnorm": 1, "input": 2}

    def unary_f32(self, op, x, alpha=0.0, beta=0.0):
        y = self.empty(x.shape, np.float32)
        _check(lib().exhip_unary_f32(self.h, self.UNARY[op], x.ptr, y.ptr, ctypes.c_size_t(y.size), ctypes.c_float(float(alpha)),
                                     ctypes.c_float(float(beta))))
        return y

    def channelwise_f32(self, op, x, p0, p1=None, shared=False):
        n, c, h, w = x.shape
        y = self.empty(x.shape, np.float32)
        _check(lib().exhip_channelwise_f32(self.h, self.CHANNEL[op], x.ptr, y.ptr, n, c, h * w, p0.ptr, _ptr(p1), int(shared)))
        return y

    def unary_f16(self, op, x, alpha=0.0, beta=0.0):
        y = self.empty(x.shape, np.uint16)
        _check(lib().exhip_unary_f16(self.h, self.UNARY[op], x.ptr, y.ptr, ctypes.c_size_t(y.size), ctypes.c_float(float(alpha)),
                                     ctypes.c_float(float(beta))))
        return y

    def channelwise_f16(self, op, x, p0, p1=None, shared=False):
        n, c, h, w = x.shape
        y = self.empty(x.shape, np.uint16)
        _check(lib().exhip_channelwise_f16(self.h, self.CHANNEL[op], x.ptr, y.ptr, n, c, h * w, p0.ptr, _ptr(p1), int(shared)))
        return y

    def channelwise_nhwc_f16(self, op, x, p0, p1=None, shared=False):
        n, h, w, c = x.shape
        y = self.empty(x.shape, np.uint16)
        _check(lib().exhip_channelwise_nhwc_f16(self.h, self.CHANNEL[op], x.ptr, y.ptr, ctypes.c_size_t(n * h * w), c, p0.ptr, _ptr(p1),
                                                int(shared)))
        return y

    def concat_nhwc_f32(self, inputs, channels, out_stride, bn=None, unary=None, alpha=0.0, beta=0.0, want_f32=True, fs_out=None):
        """Channel blocks of float32 NHWC blobs (inputs[i] has channels[i] channels at a stride of its last dimension) side by
        side, BatchNorm bn=(a, b) and the activation `unary` behind them, as float32 NHWC and / or int8 NHWC q8(v * fs_out)
        (exhip_concat_batchnorm_unary_nhwc_f32). Returns (float32 or None, int8 or None)."""
        n, h, w, _ = inputs[0].shape
        ptrs = (ctypes.c_void_p * len(inputs))(*[a.ptr.value for a in inputs])
        ch = (ctypes.c_int * len(inputs))(*channels)
        st = (ctypes.c_int * len(inputs))(*[a.shape[3] for a in inputs])
        y_f = self.empty((n, h, w, out_stride), np.float32) if want_f32 else None
        y_q = self.empty((n, h, w, out_stride), np.int8) if fs_out is not None else None
        _check(lib().exhip_concat_batchnorm_unary_nhwc_f32(self.h, ptrs, ch, st, len(inputs), ctypes.c_size_t(n * h * w),
                                                           _ptr(bn[0] if bn else None), _ptr(bn[1] if bn else None),
                                                           -1 if unary is None else self.UNARY[unary], ctypes.c_float(float(alpha)),
                                                           ctypes.c_float(float(beta)), int(out_stride), _ptr(y_f), _ptr(y_q),
                                                           ctypes.c_float(float(fs_out or 0.0))))
        return y_f, y_q

    def concat_nhwc_f16(self, inputs, bn=None, unary=None, alpha=0.0, beta=0.0):
        """Concat of NHWC half blobs along the channels; with bn=(a, b) and / or unary= the BatchNorm and activation layers
        behind it in the same kernel (exhip_concat_batchnorm_unary_nhwc_f16), else the plain exhip_concat_channels_nhwc_f16."""
        n, h, w, _ = inputs[0].shape
        ptrs = (ctypes.c_void_p * len(inputs))(*[a.ptr.value for a in inputs])
        ch = (ctypes.c_int * len(inputs))(*[a.shape[3] for a in inputs])
        y = self.empty((n, h, w, sum(a.shape[3] for a in inputs)), np.uint16)
        if bn is None and unary is None:
            _check(lib().exhip_concat_channels_nhwc_f16(self.h, ptrs, ch, len(inputs), ctypes.c_size_t(n * h * w), y.ptr))
        else:
            _check(lib().exhip_concat_batchnorm_unary_nhwc_f16(self.h, ptrs, ch, len(inputs), ctypes.c_size_t(n * h * w),
                                                               _ptr(bn[0] if bn else None), _ptr(bn[1] if bn else None),
                                                               -1 if unary is None else self.UNARY[unary], ctypes.c_float(float(alpha)),
                                                               ctypes.c_float(float(beta)), y.ptr))
        return y

    def concat_channels_f32(self, inputs):
        n, _, h, w = inputs[0].shape
        ptrs = (ctypes.c_void_p * len(inputs))(*[a.ptr.value for a in inputs])
        ch = (ctypes.c_int * len(inputs))(*[a.shape[1] for a in inputs])
        y = self.empty((n, sum(a.shape[1] for a in inputs), h, w), np.float32)
        _check(lib().exhip_concat_channels_f32(self.h, ptrs, ch, len(inputs), n, h * w, y.ptr))
        return y

    def interp_nearest_f32(self, x, oh, ow):
        n, c, h, w = x.shape
        y = self.empty((n, c, oh, ow), np.float32)
        _check(lib().exhip_interp_nearest_f32(self.h, x.ptr, y.ptr, n, c, h, w, oh, ow))
        return y

    def focus_f32(self, x):
        n, c, h, w = x.shape
        y = self.empty((n, 4 * c, h // 2, w // 2), np.float32)
        _check(lib().exhip_focus_f32(self.h, x.ptr, y.ptr, n, c, h, w))
        return y

    def focus_f16(self, x):
        n, c, h, w = x.shape
        y = self.empty((n, 4 * c, h // 2, w // 2), np.uint16)
        _check(lib().exhip_focus_f16(self.h, x.ptr, y.ptr, n, c, h, w))
        return y

    def maxpool2d_nhwc_i8(self, x, c, kernel, stride, pad, oh, ow):
        """MAX pooling on an int8 NHWC tensor [n, h, w, c_stride] (exhip_maxpool2d_nhwc_i8); pad = (top, left)."""
        n, h, w, cs = x.shape
        y = self.empty((n, oh, ow, cs), np.int8)
        _check(lib().exhip_maxpool2d_nhwc_i8(self.h, x.ptr, y.ptr, n, int(c), h, w, cs, int(oh), int(ow), int(kernel), int(kernel), int(stride),
                                             int(stride), int(pad[0]), int(pad[1])))
        return y


    def maxpool_same_pyramid_nhwc_i8(self, x, c, k, levels=3):
        """Stride-1 "same" max pools of window k applied `levels` times to an int8 NHWC tensor, every level's result returned
        (exhip_maxpool_same_pyramid_nhwc_i8)."""
        n, h, w, cs = x.shape
        ys = [self.empty((n, h, w, cs), np.int8) for _ in range(levels)]
        ptrs = [y.ptr for y in ys] + [None] * (3 - levels)
        _check(lib().exhip_maxpool_same_pyramid_nhwc_i8(self.h, x.ptr, ptrs[0], ptrs[1], ptrs[2], n, int(c), h, w, cs, int(k)))
        return ys
    def input_focus_quantize(self, x, means, scales, fs, c_stride=32):
        """Input layer, YoloV5Focus and the int8 quantizer in one pass (exhip_input_focus_quantize_nchw_f32_to_nhwc_i8): float32
        NCHW -> int8 NHWC [n, h / 2, w / 2, c_stride]. Returns None where the library leaves the shape to the three layers."""
        n, c, h, w = x.shape
        y = self.empty((n, h // 2, w // 2, c_stride), np.int8)
        m = (ctypes.c_float * len(means))(*[float(v) for v in means])
        sc = (ctypes.c_float * len(scales))(*[float(v) for v in scales])
        rc = lib().exhip_input_focus_quantize_nchw_f32_to_nhwc_i8(self.h, x.ptr, n, c, h, w, m, sc, ctypes.c_float(float(fs)), int(c_stride), y.ptr)
        if rc == 10002:
            return None
        _check(rc)
        return y

    def nhwc_to_grouped_f32(self, x, channels, groups):
        """[n, h, w, stride] float32 with `channels` = groups * per_group real channels -> [n, groups, h * w, per_group]
        (exhip_nhwc_f32_to_grouped_f32): a detection head's Reshape + Transpose on the NHWC result."""
        n, h, w, stride = x.shape
        per_group = channels // groups
        y = self.empty((n, groups, h * w, per_group), np.float32)
        _check(lib().exhip_nhwc_f32_to_grouped_f32(self.h, x.ptr, n, h * w, int(groups), int(per_group), int(stride), y.ptr))
        return y

    def binaryop_f32(self, op, mode, large, small):
        """op 0 ADD / 1 SUB / 2 MUL / 3 DIV; mode 0 equal shapes, 1 per image, 2 per (image, channel), 3 per (image, pixel)."""
        n, c, h, w = large.shape
        y = self.empty(large.shape, np.float32)
        _check(lib().exhip_binaryop_f32(self.h, int(op), int(mode), large.ptr, small.ptr, y.ptr, n, c, h * w, small.shape[0]))
        return y

    def softmax_channels_f32(self, x):
        n, c = x.shape[:2]
        y = self.empty(x.shape, np.float32)
        _check(lib().exhip_softmax_channels_f32(self.h, x.ptr, y.ptr, n, c, int(np.prod(x.shape[2:], dtype=np.int64))))
        return y

    def transpose_hw_f32(self, x):
        n, c, h, w = x.shape
        y = self.empty((n, c, w, h), np.float32)
        _check(lib().exhip_transpose_hw_f32(self.h, x.ptr, y.ptr, n * c, h, w))
        return y

    def transpose_hw_f16(self, x):
        n, c, h, w = x.shape
        y = self.empty((n, c, w, h), np.uint16)
        _check(lib().exhip_transpose_hw_f16(self.h, x.ptr, y.ptr, n * c, h, w))
        return y

    def deconv2d_f32(self, x, w, bias, stride, pad):
        n, c, h, wd = x.shape
        _, k, kh, kw = w.shape
        sh, sw = (stride, stride) if np.isscalar(stride) else stride
        pt, pb, pl, pr = (pad,) * 4 if np.isscalar(pad) else pad
        y = self.empty((n, k, (h - 1) * sh + kh - pt - pb, (wd - 1) * sw + kw - pl - pr), np.float32)
        _check(lib().exhip_deconv2d_f32(self.h, x.ptr, w.ptr, _ptr(bias), y.ptr, n, c, h, wd, k, kh, kw, sh, sw, pt, pb, pl, pr))
        return y

    def add_f16(self, a, b, relu=False):
        y = self.empty(a.shape, np.uint16)
        _check(lib().exhip_add_f16(self.h, a.ptr, b.ptr, y.ptr, ctypes.c_size_t(y.size), int(relu)))
        return y

    def relu_f16(self, x):
        y = self.empty(x.shape, np.uint16)
        _check(lib().exhip_relu_f16(self.h, x.ptr, y.ptr, ctypes.c_size_t(y.size)))
        return y

    def innerproduct_f32(self, x, w, bias=None):
        m = x.shape[0]
        k_in = x.size // m
        n_out = w.size // k_in
        y = self.empty((m, n_out, 1, 1), np.float32)
        _check(lib().exhip_innerproduct_f32(self.h, x.ptr, w.ptr, _ptr(bias), y.ptr, m, n_out, k_in))
        return y
