"""Data types of the array library: NumPy dtype objects, numbered as the C ABI numbers them."""
import numpy as np

from .. import _lib

bool = np.dtype("?")  # noqa: A001  (array-API name)
int8 = np.dtype("i1")
uint8 = np.dtype("u1")
int16 = np.dtype("i2")
uint16 = np.dtype("u2")
int32 = np.dtype("i4")
uint32 = np.dtype("u4")
int64 = np.dtype("i8")
uint64 = np.dtype("u8")
float16 = np.dtype("f2")
float32 = np.dtype("f4")
float64 = np.dtype("f8")
complex64 = np.dtype("c8")
complex128 = np.dtype("c16")

ALL_DTYPES = [bool, int8, uint8, int16, uint16, int32, uint32, int64, uint64,
              float16, float32, float64, complex64, complex128]

_TO_ID = {dt: i for i, dt in enumerate(ALL_DTYPES)}
assert _TO_ID[float32] == _lib.FLOAT and _TO_ID[complex128] == _lib.CDOUBLE


class UnsupportedDtypeError(TypeError, ValueError):
    """A valid NumPy dtype that device arrays do not have (object, strings, datetimes...).  The
    reference raises TypeError from its array constructor and ValueError from finfo / iinfo."""


def dtype(obj):
    """Normalise `obj` to one of the 14 supported dtype objects."""
    dt = np.dtype(obj)
    if dt not in _TO_ID:
        raise UnsupportedDtypeError(f"Data type '{dt}' is not supported")
    return ALL_DTYPES[_TO_ID[dt]]


def dtype_id(dt):
    return _TO_ID[np.dtype(dt)]


def dtype_from_id(i):
    return ALL_DTYPES[i] if 0 <= i < len(ALL_DTYPES) else None


def finfo(dt):
    return np.finfo(dtype(dt))


def iinfo(dt):
    return np.iinfo(dtype(dt))


def isdtype(dt, kind):
    """Array-API isdtype."""
    dt = np.dtype(dt)
    if isinstance(kind, tuple):
        return any(isdtype(dt, k) for k in kind)
    if isinstance(kind, np.dtype):
        return dt == kind
    kinds = {
        "bool": "b", "signed integer": "i", "unsigned integer": "u",
        "integral": "iu", "real floating": "f", "complex floating": "c",
        "numeric": "iufc",
    }
    if kind not in kinds:
        raise ValueError(f"Unrecognized data type kind: {kind}")
    return dt.kind in kinds[kind]
