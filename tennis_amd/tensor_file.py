"""TenniS tensor files (`.t`): reader and writer of the format Tensor::serialize / Tensor::externalize
define (src/core/tensor.cpp:314-389), which tensor::save / tensor::load (include/core/tensor_builder.h:153-159)
and the operator test cases of tools/run_test (test_case.hpp:218-246) use.

Layout, all little-endian:
    uint32  fields                       (1 for an ordinary tensor, n for a packed one)
    per field:
        uint8   dtype                    (DTYPE code, include/core/dtype.h:11-47)
        uint32  ndims
        uint32  sizes[ndims]
        bytes   count * type_bytes       (row-major)
"""
import struct

import numpy as np

# DTYPE code -> numpy type (include/core/dtype.h:11-47); CHAR8 strings are returned as python str
VOID, INT8, UINT8, INT16, UINT16, INT32, UINT32, INT64, UINT64 = 0, 1, 2, 3, 4, 5, 6, 7, 8
FLOAT16, FLOAT32, FLOAT64, PTR, CHAR8, CHAR16, CHAR32 = 9, 10, 11, 12, 13, 14, 15
BOOLEAN = 21
_TS2NP = {INT8: np.int8, UINT8: np.uint8, INT16: np.int16, UINT16: np.uint16, INT32: np.int32, UINT32: np.uint32,
          INT64: np.int64, UINT64: np.uint64, FLOAT16: np.float16, FLOAT32: np.float32, FLOAT64: np.float64,
          CHAR8: np.uint8, CHAR16: np.uint16, CHAR32: np.uint32, BOOLEAN: np.uint8}
_NP2TS = {np.dtype(np.int8): INT8, np.dtype(np.uint8): UINT8, np.dtype(np.int16): INT16, np.dtype(np.uint16): UINT16,
          np.dtype(np.int32): INT32, np.dtype(np.uint32): UINT32, np.dtype(np.int64): INT64,
          np.dtype(np.uint64): UINT64, np.dtype(np.float16): FLOAT16, np.dtype(np.float32): FLOAT32,
          np.dtype(np.float64): FLOAT64, np.dtype(np.bool_): BOOLEAN}


class TensorFileError(ValueError):
    pass


def _take(buf, pos, n, what):
    if pos + n > len(buf):
        raise TensorFileError("truncated tensor file: %s needs %d bytes at offset %d of %d" % (what, n, pos, len(buf)))
    return buf[pos:pos + n], pos + n


def parse_fields(buf):
    """[(dtype code, numpy array)] for every field of a serialized tensor."""
    raw, pos = _take(buf, 0, 4, "field count")
    (fields,) = struct.unpack("<I", raw)
    out = []
    for f in range(fields):
        raw, pos = _take(buf, pos, 5, "prototype of field %d" % f)
        code, ndims = struct.unpack("<BI", raw)
        if code not in _TS2NP:
            raise TensorFileError("field %d: dtype code %d has no fixed-size element" % (f, code))
        raw, pos = _take(buf, pos, 4 * ndims, "sizes of field %d" % f)
        shape = struct.unpack("<%dI" % ndims, raw)
        np_type = np.dtype(_TS2NP[code]).newbyteorder("<")
        count = int(np.prod(shape, dtype=np.int64)) if ndims else 1
        raw, pos = _take(buf, pos, count * np_type.itemsize, "data of field %d" % f)
        arr = np.frombuffer(raw, dtype=np_type).reshape(shape).astype(_TS2NP[code])
        if code == BOOLEAN:
            arr = arr.astype(np.bool_)
        out.append((code, arr))
    if pos != len(buf):
        raise TensorFileError("%d bytes behind the last field" % (len(buf) - pos))
    return out


def _value(code, arr):
    if code == CHAR8:
        return arr.tobytes().decode()
    return arr


def read_tensor(path, with_dtype=False):
    """The tensor in file ``path``: a numpy array (a str for CHAR8), or a list of them for a packed tensor.
    with_dtype=True returns (DTYPE code, value) pairs instead."""
    with open(path, "rb") as fh:
        fields = parse_fields(fh.read())
    vals = [(c, _value(c, a)) if with_dtype else _value(c, a) for c, a in fields]
    return vals[0] if len(vals) == 1 else vals


def serialize(value):
    """Bytes of ``value`` (numpy array, python str, or a list of those for a packed tensor)."""
    fields = value if isinstance(value, (list, tuple)) else [value]
    out = [struct.pack("<I", len(fields))]
    for v in fields:
        if isinstance(v, str):
            arr, code = np.frombuffer(v.encode(), dtype=np.uint8), CHAR8
        else:
            arr = np.asarray(v)
            if not arr.flags.c_contiguous:
                arr = arr.copy(order="C")
            if arr.dtype not in _NP2TS:
                raise TensorFileError("numpy type %s has no TenniS DTYPE" % arr.dtype)
            code = _NP2TS[arr.dtype]
        out.append(struct.pack("<BI", code, arr.ndim))
        out.append(struct.pack("<%dI" % arr.ndim, *arr.shape))
        data = arr.astype(np.uint8) if code == BOOLEAN else arr.astype(arr.dtype.newbyteorder("<"))
        out.append(data.tobytes())
    return b"".join(out)


def write_tensor(path, value):
    with open(path, "wb") as fh:
        fh.write(serialize(value))
