"""TEST INFRASTRUCTURE ONLY: numpy-facing wrappers over ``oracle/liboracle.so``.

``liboracle.so`` is this repo's CPU restatement (``oracle/oracle.cpp``) of the
TenniS reference hot path.  It is the parity checker for the HIP kernels; only
tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py``
may import this module.  The product path never does.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None

_vp = ctypes.c_void_p
_i = ctypes.c_int
_i64 = ctypes.c_int64
_f = ctypes.c_float


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_PATH):
            raise RuntimeError("oracle not built: run `make -C oracle oracle`")
        L = ctypes.CDLL(_PATH)
        L.orc_set_threads.argtypes = [_i]
        L.orc_get_max_threads.restype = _i
        L.orc_quantize_f32.argtypes = [_vp, _i64, _vp, _i, _vp]
        L.orc_im2col_i8.argtypes = [_vp] + [_i] * 13 + [_vp, ctypes.c_int8]
        L.orc_im2col_f32.argtypes = [_vp] + [_i] * 13 + [_vp, _f]
        L.orc_gemm_i8.argtypes = [_i, _i, _i, _vp, _vp, _vp, _i]
        L.orc_conv2d_quantized.argtypes = [_vp, _i, _i, _i, _i, _vp] + [_i] * 11 + [_f, _vp, _vp, _vp, _i]
        L.orc_add_bias_f32.argtypes = [_vp, _i64, _i, _i64, _vp, _vp]
        L.orc_relu_f32.argtypes = [_vp, _i64, _vp]
        L.orc_batch_norm_f32.argtypes = [_vp, _i64, _i, _i64, _vp, _vp, _f, _vp]
        L.orc_batch_scale_f32.argtypes = [_vp, _i64, _i, _i64, _vp, _vp, _vp]
        L.orc_fused_batch_norm_f32.argtypes = [_vp, _i64, _i, _i64, _vp, _vp, _vp, _vp, _f, _vp]
        L.orc_leaky_relu_f32.argtypes = [_vp, _i64, _f, _vp]
        L.orc_epilogue.argtypes = [_vp, _i64, _i, _i64, _vp, _vp, _vp, _i, _f, _vp, _vp, _i, _vp]
        L.orc_conv2d_i8_fused.argtypes = ([_vp, _i, _i, _i, _i, _vp] + [_i] * 11 +
                                          [_f, _vp, _vp, _i, _f, _vp, _vp, _i, _vp])
        L.orc_gemm_i8_dequant.argtypes = [_i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp]
        L.orc_gemm_f32.argtypes = [_i, _i, _i, _vp, _vp, _vp]
        L.orc_conv2d_f32.argtypes = [_vp, _i, _i, _i, _i, _vp] + [_i] * 11 + [_f, _vp]
        L.orc_inner_prod_f32.argtypes = [_vp, _i, _i, _vp, _i, _i, _vp]
        L.orc_winograd_f63.argtypes = [_vp, _i, _i, _i, _i, _vp, _i, _i, _i, _i, _i, _f, _vp]
        L.orc_depthwise_conv2d_f32.argtypes = [_vp, _i, _i, _i, _i, _vp] + [_i] * 10 + [_f, _vp]
        L.orc_resize_nearest_f32.argtypes = [_vp, ctypes.c_int64, _i, _i, _vp, _i, _i]
        for _n in ('orc_softplus_f32', 'orc_tanh_f32', 'orc_mish_f32'):
            getattr(L, _n).argtypes = [_vp, ctypes.c_int64, _vp]
        L.orc_add_f32.argtypes = [_vp, _vp, ctypes.c_int64, _vp]
        L.orc_pooling2d_f32.argtypes = [_vp, ctypes.c_int64] + [_i] * 10 + [_vp, _i, _i]
        L.orc_winograd_f23.argtypes = [_vp, _i, _i, _i, _i, _vp, _i, _i, _i, _i, _i, _f, _vp]
        _lib = L
    return _lib


def set_threads(n):
    lib().orc_set_threads(int(n))


def max_threads():
    return lib().orc_get_max_threads()


def _p(a):
    return None if a is None else a.ctypes.data_as(_vp)


def _c(a, dt):
    return None if a is None else np.ascontiguousarray(a, dt)


def out_hw(h, w, kh, kw, pads, strides, dilations):
    """include/backend/common_function.h:30-40."""
    ho = (h + pads[0] + pads[1] - (dilations[0] * (kh - 1) + 1)) // strides[0] + 1
    wo = (w + pads[2] + pads[3] - (dilations[1] * (kw - 1) + 1)) // strides[1] + 1
    return ho, wo


def quantize(x, scales):
    x = _c(x, np.float32)
    s = _c(np.atleast_1d(scales), np.float32)
    out = np.empty(x.shape, np.int8)
    lib().orc_quantize_f32(_p(x), x.size, _p(s), s.size, _p(out))
    return out


def im2col(x, kh, kw, pads, strides, dilations, padding_value=0):
    c, h, w = x.shape
    ho, wo = out_hw(h, w, kh, kw, pads, strides, dilations)
    out = np.empty((c * kh * kw, ho * wo), x.dtype)
    x = np.ascontiguousarray(x)
    fn = lib().orc_im2col_i8 if x.dtype == np.int8 else lib().orc_im2col_f32
    fn(_p(x), c, h, w, kh, kw, *pads, *strides, *dilations, _p(out), padding_value)
    return out


def gemm_i8(a, b, faithful=False):
    a = _c(a, np.int8)
    b = _c(b, np.int8)
    m, k = a.shape
    n = b.shape[1]
    c = np.empty((m, n), np.int32)
    lib().orc_gemm_i8(m, n, k, _p(a), _p(b), _p(c), int(faithful))
    return c


def conv2d_quantized(x, w, dq, pads=(0, 0, 0, 0), strides=(1, 1), dilations=(1, 1), padding_value=0.0,
                     return_acc=False, faithful=False):
    x = _c(x, np.int8)
    w = _c(w, np.int8)
    dq = _c(dq, np.float32)
    n, c, h, wd = x.shape
    cout, _, kh, kw = w.shape
    ho, wo = out_hw(h, wd, kh, kw, pads, strides, dilations)
    out = np.empty((n, cout, ho, wo), np.float32)
    acc = np.empty((n, cout, ho, wo), np.int32) if return_acc else None
    lib().orc_conv2d_quantized(_p(x), n, c, h, wd, _p(w), cout, kh, kw, *pads, *strides, *dilations,
                               padding_value, _p(dq), _p(out), _p(acc), int(faithful))
    return (out, acc) if return_acc else out


def add_bias(x, bias, dim=1):
    x = _c(x, np.float32)
    bias = _c(bias, np.float32)
    pre = int(np.prod(x.shape[:dim], dtype=np.int64))
    inner = int(np.prod(x.shape[dim + 1:], dtype=np.int64))
    out = np.empty_like(x)
    lib().orc_add_bias_f32(_p(x), pre, x.shape[dim], inner, _p(bias), _p(out))
    return out


def _channel_args(x, dim):
    pre = int(np.prod(x.shape[:dim], dtype=np.int64))
    inner = int(np.prod(x.shape[dim + 1:], dtype=np.int64))
    return pre, x.shape[dim], inner


def batch_norm(x, mean, variance, epsilon=1e-5, dim=1):
    """cpu::BatchNorm (src/kernels/cpu/batch_norm.cpp:61-105): (x - mean[c]) / sqrt(variance[c] + epsilon)."""
    x = _c(x, np.float32)
    out = np.empty_like(x)
    pre, ch, inner = _channel_args(x, dim)
    lib().orc_batch_norm_f32(_p(x), pre, ch, inner, _p(_c(mean, np.float32)), _p(_c(variance, np.float32)),
                             float(epsilon), _p(out))
    return out


def batch_scale(x, scale, bias, dim=1):
    """cpu::BatchScale (src/kernels/cpu/batch_scale.cpp:57-97): x * scale[c] + bias[c]."""
    x = _c(x, np.float32)
    out = np.empty_like(x)
    pre, ch, inner = _channel_args(x, dim)
    lib().orc_batch_scale_f32(_p(x), pre, ch, inner, _p(_c(scale, np.float32)), _p(_c(bias, np.float32)), _p(out))
    return out


def fused_batch_norm(x, mean, variance, scale, bias, epsilon=1e-5, dim=1):
    """cpu::FusedBatchNorm (src/kernels/cpu/fused_batch_norm.cpp:70-125): batch_norm followed by batch_scale."""
    x = _c(x, np.float32)
    out = np.empty_like(x)
    pre, ch, inner = _channel_args(x, dim)
    lib().orc_fused_batch_norm_f32(_p(x), pre, ch, inner, _p(_c(mean, np.float32)), _p(_c(variance, np.float32)),
                                   _p(_c(scale, np.float32)), _p(_c(bias, np.float32)), float(epsilon), _p(out))
    return out


def relu(x):
    x = _c(x, np.float32)
    out = np.empty_like(x)
    lib().orc_relu_f32(_p(x), x.size, _p(out))
    return out


def leaky_relu(x, scale):
    x = _c(x, np.float32)
    out = np.empty_like(x)
    lib().orc_leaky_relu_f32(_p(x), x.size, scale, _p(out))
    return out


ACT = {None: 0, "none": 0, "relu": 1, "leaky_relu": 2}


def epilogue(acc, dq, bias=None, act=None, slope=0.0, q_scales=None, row_scale=None, want_f32=True):
    """acc is [pre, channels, *inner] int32."""
    acc = _c(acc, np.int32)
    pre, ch = acc.shape[0], acc.shape[1]
    inner = int(np.prod(acc.shape[2:], dtype=np.int64))
    dq = _c(dq, np.float32)
    bias = _c(bias, np.float32)
    row_scale = _c(row_scale, np.float32)
    out = np.empty(acc.shape, np.float32) if want_f32 else None
    qs = _c(None if q_scales is None else np.atleast_1d(q_scales), np.float32)
    q = np.empty(acc.shape, np.int8) if qs is not None else None
    lib().orc_epilogue(_p(acc), pre, ch, inner, _p(dq), _p(row_scale), _p(bias), ACT[act], slope, _p(out),
                       _p(qs), 0 if qs is None else qs.size, _p(q))
    return out, q


def conv2d_i8_fused(x, w, dq, bias=None, act=None, slope=0.0, q_scales=None, pads=(0, 0, 0, 0), strides=(1, 1),
                    dilations=(1, 1), padding_value=0.0):
    x = _c(x, np.int8)
    w = _c(w, np.int8)
    dq = _c(dq, np.float32)
    bias = _c(bias, np.float32)
    n, c, h, wd = x.shape
    cout, _, kh, kw = w.shape
    ho, wo = out_hw(h, wd, kh, kw, pads, strides, dilations)
    out = np.empty((n, cout, ho, wo), np.float32)
    qs = _c(None if q_scales is None else np.atleast_1d(q_scales), np.float32)
    q = np.empty((n, cout, ho, wo), np.int8) if qs is not None else None
    lib().orc_conv2d_i8_fused(_p(x), n, c, h, wd, _p(w), cout, kh, kw, *pads, *strides, *dilations, padding_value,
                              _p(dq), _p(bias), ACT[act], slope, _p(out), _p(qs), 0 if qs is None else qs.size,
                              _p(q))
    return out, q


def gemm_i8_dequant(a, b, dq_w, dq_a=None, bias=None, return_acc=False):
    a = _c(a, np.int8)
    b = _c(b, np.int8)
    m, k = a.shape
    n = b.shape[1]
    dq_w = _c(dq_w, np.float32)
    dq_a = _c(dq_a, np.float32)
    bias = _c(bias, np.float32)
    out = np.empty((m, n), np.float32)
    acc = np.empty((m, n), np.int32) if return_acc else None
    lib().orc_gemm_i8_dequant(m, n, k, _p(a), _p(b), _p(dq_w), _p(dq_a), _p(bias), _p(out), _p(acc))
    return (out, acc) if return_acc else out


def gemm_f32(a, b):
    a = _c(a, np.float32)
    b = _c(b, np.float32)
    m, k = a.shape
    n = b.shape[1]
    c = np.empty((m, n), np.float32)
    lib().orc_gemm_f32(m, n, k, _p(a), _p(b), _p(c))
    return c


def conv2d_f32(x, w, pads=(0, 0, 0, 0), strides=(1, 1), dilations=(1, 1), padding_value=0.0):
    x = _c(x, np.float32)
    w = _c(w, np.float32)
    n, c, h, wd = x.shape
    cout, _, kh, kw = w.shape
    ho, wo = out_hw(h, wd, kh, kw, pads, strides, dilations)
    out = np.empty((n, cout, ho, wo), np.float32)
    lib().orc_conv2d_f32(_p(x), n, c, h, wd, _p(w), cout, kh, kw, *pads, *strides, *dilations, padding_value,
                         _p(out))
    return out


def inner_prod_f32(lhs, rhs, transpose=False):
    lhs = _c(lhs, np.float32)
    rhs = _c(rhs, np.float32)
    m, k = lhs.shape
    n = rhs.shape[0] if transpose else rhs.shape[1]
    out = np.empty((m, n), np.float32)
    lib().orc_inner_prod_f32(_p(lhs), m, k, _p(rhs), n, int(transpose), _p(out))
    return out


def winograd_f63(x, w, pads, padding_value=0.0):
    x = _c(x, np.float32)
    w = _c(w, np.float32)
    n, c, h, wd = x.shape
    cout = w.shape[0]
    ho, wo = out_hw(h, wd, 3, 3, pads, (1, 1), (1, 1))
    out = np.empty((n, cout, ho, wo), np.float32)
    lib().orc_winograd_f63(_p(x), n, c, h, wd, _p(w), cout, *pads, padding_value, _p(out))
    return out


def winograd_f23(x, w, pads, padding_value=0.0):
    """Conv2dWinogradAlgorithm<float>::winograd_f23 (winograd_algorithm.cpp:347-459): 3x3, stride 1."""
    x = _c(x, np.float32)
    w = _c(w, np.float32)
    n, c, h, wd = x.shape
    cout = w.shape[0]
    ho, wo = out_hw(h, wd, 3, 3, pads, (1, 1), (1, 1))
    out = np.empty((n, cout, ho, wo), np.float32)
    lib().orc_winograd_f23(_p(x), n, c, h, wd, _p(w), cout, *pads, padding_value, _p(out))
    return out


def add(a, b):
    """cpu::Add on equal shapes (src/kernels/cpu/add.cpp)."""
    a = _c(a, np.float32)
    b = _c(b, np.float32)
    assert a.shape == b.shape
    out = np.empty_like(a)
    lib().orc_add_f32(_p(a), _p(b), a.size, _p(out))
    return out


def pool_out_hw(h, w, ksize, pads, strides):
    """pooling2d_forward (include/backend/common_function.h:14-20): ceil, evaluated in fp32 like the reference."""
    ho = int(np.ceil(np.float32(h + pads[0] + pads[1] - ksize[0]) / np.float32(strides[0]) + np.float32(1)))
    wo = int(np.ceil(np.float32(w + pads[2] + pads[3] - ksize[1]) / np.float32(strides[1]) + np.float32(1)))
    return ho, wo


def pooling2d(x, kind, ksize, strides, pads=(0, 0, 0, 0), white=False):
    """cpu::Pooling2D (pooling2d_core.cpp:48-186): kind "max" or "avg"; pads = (top, bottom, left, right)."""
    x = _c(x, np.float32)
    n, c, h, w = x.shape
    ho, wo = pool_out_hw(h, w, ksize, pads, strides)
    out = np.empty((n, c, ho, wo), np.float32)
    lib().orc_pooling2d_f32(_p(x), n * c, h, w, {"max": 0, "avg": 1}[kind], pads[0], pads[2], ksize[0], ksize[1],
                            strides[0], strides[1], int(white), _p(out), ho, wo)
    return out


def global_pooling2d(x, kind):
    """base::GlobalPooling2D (base_global_pooling2d.cpp:58-79) = pooling2d over the whole map, BLACK padding."""
    return pooling2d(x, kind, x.shape[2:], (1, 1))


def depthwise_conv2d(x, w, pads=(0, 0, 0, 0), strides=(1, 1), dilations=(1, 1), padding_value=0.0):
    """cpu::DepthwiseConv2D, general form (depthwise_conv2d_algorithm.cpp:44-85); w is [1, C, KH, KW]."""
    x = _c(x, np.float32)
    w = _c(w, np.float32)
    n, c, h, wd = x.shape
    assert w.shape[0] == 1 and w.shape[1] == c
    kh, kw = w.shape[2], w.shape[3]
    ho, wo = out_hw(h, wd, kh, kw, pads, strides, dilations)
    out = np.empty((n, c, ho, wo), np.float32)
    lib().orc_depthwise_conv2d_f32(_p(x), n, c, h, wd, _p(w), kh, kw, *pads, *strides, *dilations, padding_value, _p(out))
    return out


def resize_nearest(x, ho, wo):
    """cpu::Resize2D, NEAREST, on the two last axes of NCHW (resize2d.cpp:186-215)."""
    x = _c(x, np.float32)
    n, c, h, w = x.shape
    out = np.empty((n, c, ho, wo), np.float32)
    lib().orc_resize_nearest_f32(_p(x), n * c, h, w, _p(out), ho, wo)
    return out


def _unary(name, x):
    x = _c(x, np.float32)
    out = np.empty_like(x)
    getattr(lib(), name)(_p(x), x.size, _p(out))
    return out


def softplus(x):
    return _unary("orc_softplus_f32", x)


def tanh(x):
    return _unary("orc_tanh_f32", x)


def mish(x):
    """x * tanh(softplus(x)) with TenniS's softplus and tanh (softplus.cpp:30-39, tanh.cpp:14-23)."""
    return _unary("orc_mish_f32", x)


def concat(tensors, dim=1):
    """cpu::Concat (src/kernels/cpu/concat.cpp): a copy."""
    return np.concatenate([np.asarray(t) for t in tensors], axis=dim)
