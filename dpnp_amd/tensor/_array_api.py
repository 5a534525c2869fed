"""Array-API inspection namespace: `__array_namespace_info__()` and `__array_api_version__`
(dpnp/tensor/_array_api.py:80-260), for the one device kind this library drives."""
from . import _dtypes as dt_
from . import _tensor_impl as ti
from ._device import Device
from ._dtypes import isdtype

__array_api_version__ = "2025.12"


class Info:
    """Namespace returned by `__array_namespace_info__()`."""

    def __init__(self):
        self._capabilities = {"boolean indexing": False, "data-dependent shapes": False, "max dimensions": None}
        self._all_dtypes = {
            "bool": dt_.bool, "float32": dt_.float32, "float64": dt_.float64, "complex64": dt_.complex64,
            "complex128": dt_.complex128, "int8": dt_.int8, "int16": dt_.int16, "int32": dt_.int32,
            "int64": dt_.int64, "uint8": dt_.uint8, "uint16": dt_.uint16, "uint32": dt_.uint32,
            "uint64": dt_.uint64,
        }

    def capabilities(self):
        """What the namespace supports (boolean-mask indexing and data-dependent shapes are not
        part of this library)."""
        return self._capabilities.copy()

    def default_device(self):
        return Device()

    def default_dtypes(self, *, device=None):
        """Default data types: float64, complex128, int64, and int64 for indices."""
        return {
            "real floating": dt_.dtype(ti.default_device_fp_type(device)),
            "complex floating": dt_.dtype(ti.default_device_complex_type(device)),
            "integral": dt_.dtype(ti.default_device_int_type(device)),
            "indexing": dt_.dtype(ti.default_device_index_type(device)),
        }

    def dtypes(self, *, device=None, kind=None):
        """Array-API data types of a `kind` ("bool", "signed integer", "unsigned integer",
        "integral", "real floating", "complex floating", "numeric", or a tuple of those)."""
        if kind is None:
            return dict(self._all_dtypes)
        return {k: v for k, v in self._all_dtypes.items() if isdtype(v, kind)}

    def devices(self):
        return (Device(),)


def __array_namespace_info__():
    """Inspection namespace of the array API."""
    return Info()
