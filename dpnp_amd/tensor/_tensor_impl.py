"""Drop-in for the reference's `_tensor_impl` extension module, hot-path part only:
where, cast-copy, fill, overlap predicates and the default-dtype queries
(libtensor/source/tensor_ctors.cpp:191,360-448).  Same function names and keyword
arguments; `sycl_queue` selects nothing (there is one stream) and `depends` is
ignored because the stream is in-order.  Each call returns a pair of events like
the reference does.
"""
from .. import _lib
from ._device import Event

lib = _lib.lib


def _events(q):
    e = Event(q)
    return e, e


from ._device import current_stream_ptr as _current_stream_ptr


def _stream(q):
    return _current_stream_ptr(0) if q is None else q.stream_ptr


_where = _lib.ext._where  # (condition, x1, x2, dst, sycl_queue=None, depends=()) -> (event, event)


def _clip(src, min, max, dst, sycl_queue=None, depends=()):  # noqa: A002
    """ti._clip (libtensor/source/clip.cpp:69-263): dst = min(max(src, min), max), operands of dst's
    dtype and shape."""
    views = [a._as_view() for a in (src, min, max, dst)]
    _lib.check(lib.dpx_clip(*views, _stream(sycl_queue)))
    return _events(sycl_queue)


def _where_compare(cmp_name, lhs, rhs, x1, x2, dst, sycl_queue=None, depends=()):
    """dst = (lhs CMP rhs) ? x1 : x2 in one pass (no counterpart in the reference)."""
    return _lib.ext._where_compare(_lib.BINARY_ID[cmp_name], lhs, rhs, x1, x2, dst, sycl_queue, depends)


_copy_usm_ndarray_into_usm_ndarray = _lib.ext._copy_usm_ndarray_into_usm_ndarray  # (src, dst, sycl_queue=None, depends=())


def _full_usm_ndarray(fill_value, dst, sycl_queue=None, depends=()):
    vd = dst._as_view()
    if isinstance(fill_value, (bool, int)) or (hasattr(fill_value, "dtype") and fill_value.dtype.kind in "biu"):
        iv = int(fill_value)
        if dst.dtype.kind == "u" or iv >= 2 ** 63:
            iv = iv & (2 ** 64 - 1)
            iv = iv - 2 ** 64 if iv >= 2 ** 63 else iv
        _lib.check(lib.dpx_fill(vd, 0.0, 0.0, iv, 1, _stream(sycl_queue)))
    else:
        c = complex(fill_value)
        _lib.check(lib.dpx_fill(vd, c.real, c.imag, 0, 0, _stream(sycl_queue)))
    return _events(sycl_queue)


_array_overlap = _lib.ext._array_overlap
_same_logical_tensors = _lib.ext._same_logical_tensors


# device_support_queries.cpp: MI355X has fp16 and fp64, so the defaults are NumPy's
def default_device_fp_type(q=None):
    return "f8"


def default_device_int_type(q=None):
    return "i8"


def default_device_uint_type(q=None):
    return "u8"


def default_device_bool_type(q=None):
    return "b1"


def default_device_complex_type(q=None):
    return "c16"


def default_device_index_type(q=None):
    return "i8"
