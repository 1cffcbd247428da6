"""Python access to the C++ operator layer (libtsx_backend.so): run a TenniS operator by name on
device "hip" with numpy inputs, the way TenniS's operator test runner drives an operator
(tools/run_test/test_case.hpp:424-522).  The operator classes, parameter parsing, shape
inference and device plumbing all live in C++ (tennis_amd/backend); this module only marshals."""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libtsx_backend.so")

# TenniS DTYPE codes (include/core/dtype.h:11-47)
INT8, UINT8, INT32, INT64, FLOAT32, FLOAT64, CHAR8, BOOLEAN = 1, 2, 5, 7, 10, 11, 13, 21
_NP2TS = {np.dtype(np.int8): INT8, np.dtype(np.uint8): UINT8, np.dtype(np.int32): INT32, np.dtype(np.int64): INT64,
          np.dtype(np.float32): FLOAT32, np.dtype(np.float64): FLOAT64, np.dtype(np.bool_): BOOLEAN}
_TS2NP = {INT8: np.int8, UINT8: np.uint8, INT32: np.int32, INT64: np.int64, FLOAT32: np.float32, FLOAT64: np.float64}


class _Tensor(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char_p), ("dtype", ctypes.c_int32), ("ndim", ctypes.c_int32),
                ("shape", ctypes.POINTER(ctypes.c_int32)), ("data", ctypes.c_void_p)]


class _Output(ctypes.Structure):
    _fields_ = [("dtype", ctypes.c_int32), ("ndim", ctypes.c_int32), ("shape", ctypes.c_int32 * 8),
                ("data", ctypes.c_void_p), ("capacity", ctypes.c_int64), ("bytes", ctypes.c_int64)]


class OperatorError(RuntimeError):
    """The operator raised (TenniS: EjectionException)."""


class OperatorNotFound(OperatorError):
    pass


SYMBOLS = ("tsxop_last_error", "tsxop_is_registered", "tsxop_check_params", "tsxop_run_op")
_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise OperatorError("libtsx_backend.so is not built: run `python -m tennis_amd.build`")
        try:
            # torch ships a HIP runtime of its own: where it is used in the same process it has to come up before
            # the library's (loaded from /opt/rocm), or torch no longer finds the device afterwards
            import torch
            torch.cuda.is_available()
        except ImportError:
            pass
        L = ctypes.CDLL(LIB_PATH)
        L.tsxop_last_error.restype = ctypes.c_char_p
        _lib = L
    return _lib


def _pack(name, value, keep):
    if isinstance(value, str):
        arr = np.frombuffer(value.encode(), dtype=np.uint8).copy()
        code = CHAR8
    else:
        arr = np.ascontiguousarray(value)
        code = _NP2TS[arr.dtype]
    shape = (ctypes.c_int32 * max(arr.ndim, 1))(*arr.shape)
    keep.extend([arr, shape])
    return _Tensor(name.encode() if name else None, code, arr.ndim, shape, arr.ctypes.data)


def _raise(rc):
    msg = lib().tsxop_last_error().decode(errors="replace")
    raise (OperatorNotFound if rc == 2 else OperatorError)(msg)


def is_registered(device, op):
    return bool(lib().tsxop_is_registered(device.encode(), op.encode()))


def check_params(op, params, device="hip", strict=True):
    """Create the operator, set the parameters and run init() (host only, no device needed)."""
    keep = []
    p = (_Tensor * max(len(params), 1))(*[_pack(k, v, keep) for k, v in params.items()])
    rc = lib().tsxop_check_params(device.encode(), op.encode(), int(strict), len(params), p)
    if rc:
        _raise(rc)


def run_op(op, params, inputs, device="hip", device_id=0, strict=True, infer_only=False, out_bytes=None):
    """Run operator `op` on `device`; returns its single output (or (dtype, shape) when infer_only)."""
    keep = []
    p = (_Tensor * max(len(params), 1))(*[_pack(k, v, keep) for k, v in params.items()])
    i = (_Tensor * max(len(inputs), 1))(*[_pack("", v, keep) for v in inputs])
    if out_bytes is None:
        out_bytes = 0 if infer_only else 1 << 28
    buf = np.empty(out_bytes, dtype=np.uint8)
    out = _Output()
    out.data = buf.ctypes.data
    out.capacity = out_bytes
    rc = lib().tsxop_run_op(device.encode(), int(device_id), op.encode(), int(strict), len(params), p, len(inputs), i,
                            int(infer_only), ctypes.byref(out))
    if rc:
        _raise(rc)
    shape = tuple(out.shape[k] for k in range(out.ndim))
    if infer_only:
        return out.dtype, shape
    return buf[:out.bytes].view(_TS2NP[out.dtype]).reshape(shape).copy()


def conv_params(pads=(0, 0, 0, 0), strides=(1, 1), dilations=(1, 1), padding_value=0.0):
    """The parameter block of conv2d / conv2d_quantized as a graph carries it (NCHW)."""
    return {
        "format": "NCHW",
        "padding": np.array([[0, 0], [0, 0], [pads[0], pads[1]], [pads[2], pads[3]]], np.int32),
        "padding_value": np.array([padding_value], np.float32),
        "stride": np.array([1, 1, strides[0], strides[1]], np.int32),
        "dilation": np.array([1, 1, dilations[0], dilations[1]], np.int32),
    }
