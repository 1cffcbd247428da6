"""TenniS's own runtime with this repository's "hip" device backend built into it, from Python.

`tennis_amd/lib/intree/libtennis_hip.so` is TenniS compiled from its sources with `tennis_amd/backend/hip/*.cpp`
inside (recipe: `tennis_amd/backend/intree/intree.mk`, run by `__graft_entry__.build()` where the TenniS source
tree is present); `libtennis_hip_driver.so` beside it is a C driver over that library's Workbench.  An application
would link libtennis_hip.so and use TenniS's C++ / C API as before, naming device "hip"; this module does the same
through ctypes: operators and `.tsm` modules in a Workbench on "hip" (or on "cpu", the same library's host
operators, to compare with).  `available()` says whether the library was built.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
DRIVER_PATH = os.path.join(_HERE, "lib", "intree", "libtennis_hip_driver.so")

# TenniS DTYPE codes (include/core/dtype.h:11-47)
INT8, INT32, FLOAT32, CHAR8, BOOLEAN = 1, 5, 10, 13, 21
_NP2TS = {np.dtype(np.int8): INT8, np.dtype(np.int32): INT32, np.dtype(np.float32): FLOAT32,
          np.dtype(np.uint8): 2, np.dtype(np.float64): 11, np.dtype(np.bool_): BOOLEAN}
_TS2NP = {INT8: np.int8, INT32: np.int32, FLOAT32: np.float32, 2: np.uint8, 11: np.float64}


class IntreeError(RuntimeError):
    pass


class _Tensor(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char_p), ("dtype", ctypes.c_int32), ("ndim", ctypes.c_int32),
                ("shape", ctypes.POINTER(ctypes.c_int32)), ("data", ctypes.c_void_p)]


class _Output(ctypes.Structure):
    _fields_ = [("dtype", ctypes.c_int32), ("ndim", ctypes.c_int32), ("shape", ctypes.c_int32 * 8),
                ("data", ctypes.c_void_p), ("capacity", ctypes.c_int64), ("bytes", ctypes.c_int64)]


_lib = None


def available():
    return os.path.exists(DRIVER_PATH)


def lib():
    global _lib
    if _lib is None:
        if not available():
            raise IntreeError("%s is not built: run `make -f tennis_amd/backend/intree/intree.mk` where the TenniS "
                              "sources are present" % DRIVER_PATH)
        L = ctypes.CDLL(DRIVER_PATH)
        L.intree_last_error.restype = ctypes.c_char_p
        for name in ("intree_fused_chain_count", "intree_handover_count", "intree_dual_output_count",
                     "intree_host_delegate_count"):
            getattr(L, name).restype = ctypes.c_long
        _lib = L
    return _lib


def _check(rc):
    if rc != 0:
        raise IntreeError("TenniS raised: " + lib().intree_last_error().decode(errors="replace"))


def _pack(name, value, keep):
    """A python value as a _Tensor; `keep` holds the buffers alive."""
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


def _new_output(out_bytes):
    buf = np.empty(out_bytes, dtype=np.uint8)
    out = _Output()
    out.data = buf.ctypes.data
    out.capacity = out_bytes
    return buf, out


def _take(buf, out):
    shape = tuple(out.shape[k] for k in range(out.ndim))
    return buf[:out.bytes].view(_TS2NP[out.dtype]).reshape(shape).copy()


def run_op(device, op, params, inputs, out_bytes, threads=1, strict=True):
    """Operator `op` in a Workbench on `device` ("cpu" or "hip").  strict: the class registered for that device
    only (no factory fallback to the host operator)."""
    keep = []
    p = (_Tensor * max(len(params), 1))(*[_pack(k, v, keep) for k, v in params.items()])
    i = (_Tensor * max(len(inputs), 1))(*[_pack("", v, keep) for v in inputs])
    buf, out = _new_output(out_bytes)
    _check(lib().intree_run_op(device.encode(), int(strict), op.encode(), len(params), p, len(inputs), i, int(threads),
                               ctypes.byref(out)))
    return _take(buf, out)


def run_module(device, path, inputs, out_bytes=1 << 24, threads=1):
    """A `.tsm` file in a Workbench on `device`: TenniS's module loader, graph compiler and runtime; output 0."""
    keep = []
    i = (_Tensor * max(len(inputs), 1))(*[_pack("", v, keep) for v in inputs])
    buf, out = _new_output(out_bytes)
    _check(lib().intree_run_module(str(path).encode(), device.encode(), len(inputs), i, int(threads), ctypes.byref(out)))
    return _take(buf, out)


def time_module(device, path, inputs, warmup=2, reps=10, out_bytes=1 << 24, threads=1, resident=False):
    """ms per run of a `.tsm` module on `device` (loaded and compiled once; each run ends with output 0 read back),
    and that output.  resident: the inputs are moved to the device before the timed loop instead of being uploaded
    by every run."""
    keep = []
    i = (_Tensor * max(len(inputs), 1))(*[_pack("", v, keep) for v in inputs])
    buf, out = _new_output(out_bytes)
    ms = ctypes.c_double(0.0)
    _check(lib().intree_time_module(str(path).encode(), device.encode(), len(inputs), i, int(threads), int(warmup),
                                    int(reps), int(bool(resident)), ctypes.byref(ms), ctypes.byref(out)))
    return ms.value, _take(buf, out)


def run_module_cloned(device, path, input_sets, runs=3, out_bytes=1 << 24):
    """The module loaded once on `device`, its Workbench cloned for every further input set (Workbench::clone), and
    each Workbench run `runs` times by a host thread of its own, all at once: output 0 of every thread's last run."""
    keep = []
    nthreads, ninputs = len(input_sets), len(input_sets[0])
    flat = [_pack("", v, keep) for s in input_sets for v in s]
    i = (_Tensor * len(flat))(*flat)
    bufs, outs = zip(*[_new_output(out_bytes) for _ in range(nthreads)])
    o = (_Output * nthreads)(*outs)
    _check(lib().intree_run_module_cloned(str(path).encode(), device.encode(), nthreads, int(runs), ninputs, i, o))
    return [_take(b, o[t]) for t, b in enumerate(bufs)]


def fused_chain_count():
    """Chains the "hip" device's zipper option has replaced so far in this process."""
    return int(lib().intree_fused_chain_count())


def handover_counts():
    """(fused nodes that write a staged int8 output for the convolutions behind them, those of them that return the
    fp32 form as well) so far in this process."""
    return int(lib().intree_handover_count()), int(lib().intree_dual_output_count())


def host_delegate_count():
    """Operator runs on "hip" that were handed to the host operator so far in this process (inputs a "hip" class
    does not cover)."""
    return int(lib().intree_host_delegate_count())
