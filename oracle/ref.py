"""TEST INFRASTRUCTURE ONLY: ctypes access to the compiled TenniS reference.

``oracle/_ref/libref_driver.so`` is this repo's thin ``extern "C"`` driver
(``oracle/ref_driver.cpp``) linked against the reference CPU library built by
``oracle/ref.mk`` from the reference's own sources.  It exists only where the
reference tree was present at build time; ``available()`` says whether it is.
Only tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_PATH = os.path.join(_HERE, "_ref", "libref_driver.so")

# Reference DTYPE codes (include/core/dtype.h:11-47).
INT8, INT32, FLOAT32, CHAR8, BOOLEAN = 1, 5, 10, 13, 21
_NP2TS = {np.dtype(np.int8): INT8, np.dtype(np.int32): INT32, np.dtype(np.float32): FLOAT32,
          np.dtype(np.uint8): 2, np.dtype(np.float64): 11, np.dtype(np.bool_): BOOLEAN}
_TS2NP = {INT8: np.int8, INT32: np.int32, FLOAT32: np.float32, 2: np.uint8, 11: np.float64}


class _Tensor(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char_p), ("dtype", ctypes.c_int32), ("ndim", ctypes.c_int32),
                ("shape", ctypes.POINTER(ctypes.c_int32)), ("data", ctypes.c_void_p)]


class _Output(ctypes.Structure):
    _fields_ = [("dtype", ctypes.c_int32), ("ndim", ctypes.c_int32), ("shape", ctypes.c_int32 * 8),
                ("data", ctypes.c_void_p), ("capacity", ctypes.c_int64), ("bytes", ctypes.c_int64)]


_lib = None


def available():
    return os.path.exists(_PATH)


def lib():
    global _lib
    if _lib is None:
        if not available():
            raise RuntimeError("reference driver not built: run `make -f oracle/ref.mk` where /root/reference exists")
        _lib = ctypes.CDLL(_PATH)
        _lib.ref_last_error.restype = ctypes.c_char_p
    return _lib


def _check(rc):
    if rc != 0:
        raise RuntimeError("reference raised: " + lib().ref_last_error().decode(errors="replace"))


def _pack(name, value, keep):
    """Turn a python value into a _Tensor; ``keep`` holds the buffers alive."""
    if isinstance(value, str):
        arr = np.frombuffer(value.encode(), dtype=np.uint8).copy()
        code = CHAR8
    else:
        arr = np.ascontiguousarray(value)
        if arr.dtype == np.int64:
            arr = arr.astype(np.int32)
        code = _NP2TS[arr.dtype]
    shape = (ctypes.c_int32 * max(arr.ndim, 1))(*arr.shape)
    keep.extend([arr, shape])
    return _Tensor(name.encode() if name else None, code, arr.ndim, shape, arr.ctypes.data)


def run_op(op, params, inputs, out_bytes, threads=1):
    """Run reference operator ``op`` (CPU device) and return its single output as numpy."""
    keep = []
    p = (_Tensor * max(len(params), 1))(*[_pack(k, v, keep) for k, v in params.items()])
    i = (_Tensor * max(len(inputs), 1))(*[_pack("", v, keep) for v in inputs])
    buf = np.empty(out_bytes, dtype=np.uint8)
    out = _Output()
    out.data = buf.ctypes.data
    out.capacity = out_bytes
    _check(lib().ref_run_op(op.encode(), len(params), p, len(inputs), i, int(threads), ctypes.byref(out)))
    shape = tuple(out.shape[k] for k in range(out.ndim))
    return buf[:out.bytes].view(_TS2NP[out.dtype]).reshape(shape).copy()


def save_tensor(path, value):
    """Write ``value`` (numpy array or str) as a TenniS `.t` file with the reference's own serializer."""
    keep = []
    t = _pack("", value, keep)
    _check(lib().ref_save_tensor(str(path).encode(), ctypes.byref(t)))


def load_tensor(path, max_bytes=1 << 24):
    """Read a `.t` file with the reference's own reader; returns (dtype code, numpy array of raw dtype)."""
    buf = np.empty(max_bytes, dtype=np.uint8)
    out = _Output()
    out.data = buf.ctypes.data
    out.capacity = max_bytes
    _check(lib().ref_load_tensor(str(path).encode(), ctypes.byref(out)))
    shape = tuple(out.shape[k] for k in range(out.ndim))
    np_type = _TS2NP.get(out.dtype, np.uint8)
    return out.dtype, buf[:out.bytes].view(np_type).reshape(shape).copy()


def run_module(path, inputs, out_bytes=1 << 24, device="cpu", threads=1):
    """Load a `.tsm` file with the reference's own Module::Load, run it in a Workbench; returns output 0."""
    keep = []
    i = (_Tensor * max(len(inputs), 1))(*[_pack("", v, keep) for v in inputs])
    buf = np.empty(out_bytes, dtype=np.uint8)
    out = _Output()
    out.data = buf.ctypes.data
    out.capacity = out_bytes
    _check(lib().ref_run_module(str(path).encode(), device.encode(), len(inputs), i, int(threads), ctypes.byref(out)))
    shape = tuple(out.shape[k] for k in range(out.ndim))
    return buf[:out.bytes].view(_TS2NP[out.dtype]).reshape(shape).copy()


def _conv_params(pads, strides, dilations, padding_value=0.0):
    return {
        "format": "NCHW",
        "padding": np.array([[0, 0], [0, 0], [pads[0], pads[1]], [pads[2], pads[3]]], np.int32),
        "padding_value": np.array([padding_value], np.float32),
        "stride": np.array([1, 1, strides[0], strides[1]], np.int32),
        "dilation": np.array([1, 1, dilations[0], dilations[1]], np.int32),
    }


def _out_hw(h, w, kh, kw, pads, strides, dilations):
    ho = (h + pads[0] + pads[1] - (dilations[0] * (kh - 1) + 1)) // strides[0] + 1
    wo = (w + pads[2] + pads[3] - (dilations[1] * (kw - 1) + 1)) // strides[1] + 1
    return ho, wo


def quantize(x, scales, threads=1):
    x = np.ascontiguousarray(x, np.float32)
    return run_op("quantize", {"quantize_scale": np.asarray(scales, np.float32)}, [x], x.size, threads)


def conv2d_quantized(x, w, dq, pads=(0, 0, 0, 0), strides=(1, 1), dilations=(1, 1), padding_value=0.0, threads=1):
    p = _conv_params(pads, strides, dilations, padding_value)
    p["dequantize_scales"] = np.asarray(dq, np.float32)
    ho, wo = _out_hw(x.shape[2], x.shape[3], w.shape[2], w.shape[3], pads, strides, dilations)
    return run_op("conv2d_quantized", p, [x, w], 4 * x.shape[0] * w.shape[0] * ho * wo, threads)


def conv2d(x, w, pads=(0, 0, 0, 0), strides=(1, 1), dilations=(1, 1), padding_value=0.0, threads=1):
    p = _conv_params(pads, strides, dilations, padding_value)
    ho, wo = _out_hw(x.shape[2], x.shape[3], w.shape[2], w.shape[3], pads, strides, dilations)
    return run_op("conv2d", p, [x, w], 4 * x.shape[0] * w.shape[0] * ho * wo, threads)


def depthwise_conv2d(x, w, pads=(0, 0, 0, 0), strides=(1, 1), dilations=(1, 1), padding_value=0.0, threads=1):
    p = _conv_params(pads, strides, dilations, padding_value)
    ho, wo = _out_hw(x.shape[2], x.shape[3], w.shape[2], w.shape[3], pads, strides, dilations)
    return run_op("depthwise_conv2d", p, [x, w], 4 * x.shape[0] * x.shape[1] * w.shape[0] * ho * wo, threads)


def add_bias(x, b, dim=1, threads=1):
    return run_op("add_bias", {"dim": np.array([dim], np.int32)}, [x, b], x.nbytes, threads)


def relu(x, threads=1):
    return run_op("relu", {}, [x], x.nbytes, threads)


def leaky_relu(x, scale, threads=1):
    return run_op("leaky_relu", {"scale": np.array([scale], np.float32)}, [x], x.nbytes, threads)


def add(a, b, threads=1):
    return run_op("add", {}, [a, b], max(a.nbytes, b.nbytes), threads)


def pooling2d(x, kind, ksize, strides, pads=(0, 0, 0, 0), white=False, threads=1):
    p = {"format": "NCHW", "type": np.array([{"max": 0, "avg": 1}[kind]], np.int32),
         "padding": np.array([[0, 0], [0, 0], [pads[0], pads[1]], [pads[2], pads[3]]], np.int32),
         "padding_type": np.array([3 if white else 0], np.int32),
         "ksize": np.array([1, 1, ksize[0], ksize[1]], np.int32),
         "stride": np.array([1, 1, strides[0], strides[1]], np.int32)}
    return run_op("pooling2d", p, [x], 4 * x.size + 4096, threads)


def global_pooling2d(x, kind, threads=1):
    p = {"format": "NCHW", "type": np.array([{"max": 0, "avg": 1}[kind]], np.int32)}
    return run_op("global_pooling2d", p, [x], 4 * x.shape[0] * x.shape[1], threads)


def unary(op, x, threads=1):
    return run_op(op, {}, [x], x.nbytes, threads)


def mul(a, b, threads=1):
    return run_op("mul", {}, [a, b], max(a.nbytes, b.nbytes), threads)


def concat(tensors, dim=1, threads=1):
    return run_op("concat", {"dim": np.array([dim], np.int32)}, list(tensors), sum(t.nbytes for t in tensors), threads)


def resize_nearest(x, ho, wo, threads=1):
    size = np.array([-1, -1, ho, wo], np.int32)
    return run_op("_resize2d", {"type": np.array([2], np.int32)}, [x, size], 4 * x.shape[0] * x.shape[1] * ho * wo, threads)


def inner_prod(lhs, rhs, transpose=False, threads=1):
    n = rhs.shape[0] if transpose else rhs.shape[1]
    return run_op("inner_prod", {"transpose": np.array([transpose], np.bool_)}, [lhs, rhs],
                  4 * lhs.shape[0] * n, threads)


def winograd(x, k, pads, f63=True, padding_value=0.0, threads=1):
    x = np.ascontiguousarray(x, np.float32)
    k = np.ascontiguousarray(k, np.float32)
    n, c, h, w = x.shape
    ho, wo = _out_hw(h, w, 3, 3, pads, (1, 1), (1, 1))
    out = np.empty((n, k.shape[0], ho, wo), np.float32)
    pad = (ctypes.c_int * 4)(*pads)
    _check(lib().ref_winograd(int(f63), x.ctypes.data_as(ctypes.c_void_p), n, c, h, w,
                              k.ctypes.data_as(ctypes.c_void_p), k.shape[0], pad,
                              ctypes.c_float(padding_value), out.ctypes.data_as(ctypes.c_void_p), ho, wo,
                              int(threads)))
    return out


def gemm_i8(a, b):
    a = np.ascontiguousarray(a, np.int8)
    b = np.ascontiguousarray(b, np.int8)
    m, k = a.shape
    n = b.shape[1]
    c = np.empty((m, n), np.int32)
    _check(lib().ref_gemm_i8(m, n, k, a.ctypes.data_as(ctypes.c_void_p), b.ctypes.data_as(ctypes.c_void_p),
                             c.ctypes.data_as(ctypes.c_void_p)))
    return c


def gemm_f32(a, b, threads=1):
    a = np.ascontiguousarray(a, np.float32)
    b = np.ascontiguousarray(b, np.float32)
    m, k = a.shape
    n = b.shape[1]
    c = np.empty((m, n), np.float32)
    _check(lib().ref_gemm_f32(m, n, k, a.ctypes.data_as(ctypes.c_void_p), b.ctypes.data_as(ctypes.c_void_p),
                              c.ctypes.data_as(ctypes.c_void_p), int(threads)))
    return c
