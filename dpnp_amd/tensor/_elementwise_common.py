"""Callables for unary and binary elementwise functions: type resolution, broadcasting,
`out=` and `order=` handling around one kernel call.

Observable behaviour follows UnaryElementwiseFunc / BinaryElementwiseFunc of
dpnp/tensor/_elementwise_common.py:182-289,475-988: result dtype, layout of a freshly
allocated result (order "K" keeps the operands' layout), the exception raised for each
misuse, aliasing rules for `out` (same view: computed in place; partial overlap: computed
into a temporary then copied).
"""
from collections import OrderedDict

import numpy as np

from .. import _lib
from . import _tensor_impl as ti
from ._copy_utils import _empty_like_orderK, _empty_like_pair_orderK
from ._ctors import empty, empty_like, full
from ._device import ExecutionPlacementError  # noqa: F401  (re-exported)
from ._device import current_stream_ptr
from ._dtypes import dtype as _as_dtype
from ._dtypes import ALL_DTYPES, dtype_id
from ._manipulation_functions import _broadcast_shape_impl, broadcast_to
from ._type_utils import (
    WeakBooleanType,
    WeakComplexType,
    WeakFloatingType,
    WeakIntegralType,
    _acceptance_fn_default_binary,
    _acceptance_fn_default_unary,
    _find_buf_dtype,
    _find_buf_dtype2,
    _find_buf_dtype_in_place_op,
    _resolve_weak_types,
    _resolve_weak_types_all_py_ints,
)
from ._usmarray import usm_ndarray


_ext_unary_call = _lib.ext.unary_call
_ext_binary_call = _lib.ext.binary_call


def _operand_dtype(o):
    """Concrete dtype of an array operand, weak type of a Python scalar."""
    if isinstance(o, usm_ndarray):
        return o.dtype
    if isinstance(o, np.ndarray):
        return _as_dtype(o.dtype)
    if isinstance(o, np.generic):
        return _as_dtype(o.dtype)
    if isinstance(o, bool):
        return WeakBooleanType(o)
    if isinstance(o, int):
        return WeakIntegralType(o)
    if isinstance(o, float):
        return WeakFloatingType(o)
    if isinstance(o, complex):
        return WeakComplexType(o)
    a = _foreign_as_numpy(o)
    return None if a is None else _as_dtype(a.dtype)


def _foreign_as_numpy(o):
    """NumPy form of an operand that is neither an array of this package nor a Python/NumPy
    scalar (ctypes scalars, objects with the buffer protocol, nested sequences); None if it has
    no numeric interpretation."""
    if isinstance(o, (usm_ndarray, np.ndarray, np.generic, bool, int, float, complex)) or o is None:
        return None
    try:
        a = np.asarray(o)
    except Exception:
        return None
    if a.dtype.kind not in "biufc" or a.dtype.itemsize > 16:
        return None
    return a


def _operand_shape(o):
    if isinstance(o, (usm_ndarray, np.ndarray)):
        return tuple(o.shape)
    if isinstance(o, (bool, int, float, complex, np.generic)):
        return ()
    a = _foreign_as_numpy(o)
    if a is not None:
        return tuple(a.shape)
    # anything else counts as a scalar here and is rejected by the dtype check that follows
    # (`_get_shape`, dpnp/tensor/_scalar_utils.py:108-115)
    return getattr(o, "shape", ())


def _as_device_array(o, dt):
    """Array form of a non-array operand, already of dtype `dt`."""
    if isinstance(o, usm_ndarray):
        return o
    if isinstance(o, np.ndarray):
        from ._copy_utils import from_numpy

        return from_numpy(o, dtype=dt)
    if not isinstance(o, (bool, int, float, complex, np.generic)):
        from ._copy_utils import from_numpy

        return from_numpy(_foreign_as_numpy(o), dtype=dt)
    v = o.item() if isinstance(o, np.generic) else o
    if dt.kind in "iu" and isinstance(v, int):
        info = np.iinfo(dt)
        if not (info.min <= v <= info.max):
            raise OverflowError(f"Python integer {v} out of bounds for {dt}")
    # 0-d constants recur (x * 2, x > 0, ...): keep the most recent ones on the device instead of
    # launching a fill kernel per call.  Keyed by the bit pattern (so -0.0 and 0.0, and NaN
    # payloads, stay apart) and by the stream the fill was queued on.
    try:
        key = (dt.char, np.asarray(v, dtype=dt).tobytes(), current_stream_ptr())
    except (OverflowError, TypeError, ValueError):
        return full((), v, dtype=dt)
    hit = _SCALAR_CACHE.get(key)
    if hit is not None:
        _SCALAR_CACHE.move_to_end(key)
        return hit
    arr = full((), v, dtype=dt)
    arr.flags.writable = False
    _SCALAR_CACHE[key] = arr
    if len(_SCALAR_CACHE) > _SCALAR_CACHE_MAX:
        _SCALAR_CACHE.popitem(last=False)
    return arr


_SCALAR_CACHE = OrderedDict()
_SCALAR_CACHE_MAX = 128


def _norm_order(order):
    return order if order in ("K", "C", "F", "A") else "K"


def _check_out(out, shape, res_dt):
    if not isinstance(out, usm_ndarray):
        raise TypeError(f"output array must be of usm_ndarray type, got {type(out)}")
    if not out.flags.writable:
        raise ValueError("provided `out` array is read-only")
    if out.shape != tuple(shape):
        raise ValueError("The shape of input and output arrays are inconsistent. "
                         f"Expected output shape is {tuple(shape)}, got {out.shape}")
    if res_dt != out.dtype:
        raise ValueError(f"Output array of type {res_dt} is needed, got {out.dtype}")


def _fast_out_ok(out, shape, dt):
    """`out` can be written directly by a kernel that produces a C-contiguous `shape` of `dt`."""
    return type(out) is usm_ndarray and out._dtype == dt and out._shape == shape and out._writable \
        and out._is_c_contiguous()


def _spans_meet(x, y):
    """Two C-contiguous arrays share at least one byte."""
    x0, x1 = x._contiguous_span()
    y0, y1 = y._contiguous_span()
    return x0 < y1 and y0 < x1


def _scalar_operand(v, dt, shape):
    """The cached 0-d device array for Python scalar `v` as dtype `dt`, seen with `shape`
    (all strides zero).  The last few shapes asked for are kept with the 0-d array."""
    s = _as_device_array(v, dt)
    if not shape:
        return s
    views = s.__dict__.get("_bviews")
    if views is None:
        views = s._bviews = {}
    r = views.get(shape)
    if r is None:
        if len(views) >= 8:
            views.clear()
        r = views[shape] = s._view(shape, (0,) * len(shape), s._offset)
        r._writable = False
    return r


class UnaryElementwiseFunc:
    """Elementwise function of one array.

    name: function name; result_type_resolver_fn(dtype) -> result dtype or None;
    unary_dp_impl_fn(src, dst, sycl_queue=, depends=): the kernel entry point;
    acceptance_fn: veto hook of the cast search.
    """

    def __init__(self, name, result_type_resolver_fn, unary_dp_impl_fn, docs="",
                 acceptance_fn=_acceptance_fn_default_unary):
        self.__name__ = "UnaryElementwiseFunc"
        self.name_ = name
        self.result_type_resolver_fn_ = result_type_resolver_fn
        self.unary_fn_ = unary_dp_impl_fn
        self._op_id = _lib.UNARY_ID.get(name, -1)  # the extension module's plain-call path is keyed by it
        self._ext_types_known = False
        self._fast_cache = {}
        self.__doc__ = docs
        self.acceptance_fn_ = acceptance_fn

    def __str__(self):
        return f"<{self.__name__} '{self.name_}'>"

    __repr__ = __str__

    def get_implementation_function(self):
        return self.unary_fn_

    def get_type_result_resolver_function(self):
        return self.result_type_resolver_fn_

    def get_type_promotion_path_acceptance_function(self):
        return self.acceptance_fn_

    @property
    def nin(self):
        return 1

    @property
    def nout(self):
        return 1

    @property
    def types(self):
        out = []
        for dt in ("?", "b", "B", "h", "H", "i", "I", "l", "L", "e", "f", "d", "F", "D"):
            r = self.result_type_resolver_fn_(_as_dtype(dt))
            if r is not None:
                out.append(f"{dt}->{r.char}")
        return out

    types_ = types

    def _tell_ext_types(self):
        """Enter this function's result dtype for every input dtype it takes without a cast into the extension
        module's table (the type search stays here; the module's plain-call path only looks the answer up)."""
        self._ext_types_known = True
        if self._op_id < 0:
            return
        for dt in ALL_DTYPES:
            try:
                buf_dt, r = _find_buf_dtype(dt, self.result_type_resolver_fn_, None, acceptance_fn=self.acceptance_fn_)
                ok = r is not None and buf_dt is None
            except Exception:  # a type the function refuses with an error of its own: the general path raises it
                ok = False
            _lib.ext.set_unary_type(self._op_id, dtype_id(dt), dtype_id(r) if ok else -1)

    def _fast(self, x, out=None):
        """The result for a C-contiguous array whose dtype the kernel takes as it is, else None:
        the common call without the general path's checks (nothing to cast, order "K" of a
        C-contiguous input is C; an `out` must be a writable C-contiguous array of the result's
        shape and dtype in an allocation of its own)."""
        if not self._ext_types_known:
            self._tell_ext_types()
        r = _ext_unary_call(self._op_id, x, out)  # the same checks, on the descriptors
        if r is not NotImplemented:
            return r
        if type(x) is not usm_ndarray or not x._is_c_contiguous():
            return None
        dt = x._dtype
        res_dt = self._fast_cache.get(dt)
        if res_dt is None:
            buf_dt, r = _find_buf_dtype(dt, self.result_type_resolver_fn_, None, acceptance_fn=self.acceptance_fn_)
            res_dt = self._fast_cache[dt] = r if (r is not None and buf_dt is None) else False
        if res_dt is False:
            return None
        if out is None:
            out = usm_ndarray._new_contiguous(x._shape, res_dt)
        elif not _fast_out_ok(out, x._shape, res_dt) or _spans_meet(out, x):
            return None
        self.unary_fn_(x, out)
        return out

    def __call__(self, x, /, *, out=None, order="K"):
        if order == "K":
            r = self._fast(x, out)
            if r is not None:
                return r
        if not isinstance(x, usm_ndarray):
            raise TypeError(f"Expected dpnp_amd.tensor.usm_ndarray, got {type(x)}")
        order = _norm_order(order)
        buf_dt, res_dt = _find_buf_dtype(x.dtype, self.result_type_resolver_fn_, None,
                                         acceptance_fn=self.acceptance_fn_)
        if res_dt is None:
            raise ValueError(
                f"function '{self.name_}' does not support input type ({x.dtype}), "
                "and the input could not be safely coerced to any supported types according to "
                "the casting rule ''safe''.")
        orig_out = out
        if out is not None:
            _check_out(out, x.shape, res_dt)
            if buf_dt is None and ti._array_overlap(x, out) and not ti._same_logical_tensors(x, out):
                out = empty_like(out)
        if order == "A":
            order = "F" if x.flags.f_contiguous else "C"
        src = x
        if buf_dt is not None:
            src = _empty_like_orderK(x, buf_dt) if order == "K" else empty_like(x, dtype=buf_dt, order=order)
            ti._copy_usm_ndarray_into_usm_ndarray(src=x, dst=src)
        if out is None:
            out = _empty_like_orderK(src, res_dt) if order == "K" else empty_like(src, dtype=res_dt, order=order)
        self.unary_fn_(src, out)
        if orig_out is not None and orig_out is not out:
            ti._copy_usm_ndarray_into_usm_ndarray(src=out, dst=orig_out)
            out = orig_out
        return out


class BinaryElementwiseFunc:
    """Elementwise function of two operands (arrays or Python scalars, at least one array).

    binary_dp_impl_fn(src1, src2, dst, ...) and optional binary_inplace_fn(lhs, rhs, ...)
    are the kernel entry points; weak_type_resolver maps Python-scalar operand types to
    concrete dtypes.
    """

    def __init__(self, name, result_type_resolver_fn, binary_dp_impl_fn, docs="",
                 binary_inplace_fn=None, acceptance_fn=_acceptance_fn_default_binary,
                 weak_type_resolver=_resolve_weak_types):
        self.__name__ = "BinaryElementwiseFunc"
        self.name_ = name
        self.result_type_resolver_fn_ = result_type_resolver_fn
        self.binary_fn_ = binary_dp_impl_fn
        self.binary_inplace_fn_ = binary_inplace_fn
        self.__doc__ = docs
        self.acceptance_fn_ = acceptance_fn
        self.weak_type_resolver_ = weak_type_resolver
        self._op_id = _lib.BINARY_ID.get(name, -1)
        self._ext_types_known = False
        self._fused_cache = {}
        self._fast_cache = {}

    def __str__(self):
        return f"<{self.__name__} '{self.name_}'>"

    __repr__ = __str__

    def get_implementation_function(self):
        return self.binary_fn_

    def get_implementation_inplace_function(self):
        return self.binary_inplace_fn_

    def get_type_result_resolver_function(self):
        return self.result_type_resolver_fn_

    def get_type_promotion_path_acceptance_function(self):
        return self.acceptance_fn_

    def get_array_dtype_scalar_type_resolver_function(self):
        return self.weak_type_resolver_

    @property
    def nin(self):
        return 2

    @property
    def nout(self):
        return 1

    @property
    def types(self):
        out = []
        for dt in ("?", "b", "B", "h", "H", "i", "I", "l", "L", "e", "f", "d", "F", "D"):
            r = self.result_type_resolver_fn_(_as_dtype(dt), _as_dtype(dt))
            if r is not None:
                out.append(f"{dt}{dt}->{r.char}")
        return out

    types_ = types

    def _resolve(self, o1, o2):
        is_arr1, is_arr2 = isinstance(o1, usm_ndarray), isinstance(o2, usm_ndarray)
        if not (is_arr1 or is_arr2):
            raise ExecutionPlacementError(
                "Execution placement can not be unambiguously inferred from input arguments. "
                "One of the arguments must represent USM allocation and expose "
                "`__sycl_usm_array_interface__` property")
        s1, s2 = _operand_shape(o1), _operand_shape(o2)
        if s1 is None or s2 is None:
            raise TypeError("Shape of arguments can not be inferred. Arguments are expected to be "
                            "lists, tuples, or both")
        try:
            res_shape = _broadcast_shape_impl([s1, s2])
        except ValueError:
            raise ValueError(f"operands could not be broadcast together with shapes {s1} and {s2}")
        d1, d2 = _operand_dtype(o1), _operand_dtype(o2)
        if d1 is None or d2 is None:
            raise ValueError("Operands have unsupported data types")
        d1, d2 = self.weak_type_resolver_(d1, d2, None)
        return res_shape, d1, d2

    def _fused_cast(self, d1, d2):
        """dtype the kernel gives for operands of dtypes d1 != d2 when it converts one of them
        while reading (a few arithmetic pairs), else None.  Only consulted after the promotion
        search has settled on casting that operand, so result dtypes stay the reference's."""
        key = (d1, d2)
        hit = self._fused_cache.get(key, False)
        if hit is False:
            from . import _tensor_elementwise_impl as tei

            hit = self._fused_cache[key] = tei._fused_cast_result_type(self.name_, d1, d2)
        return hit

    def _tell_ext_types(self):
        """See UnaryElementwiseFunc._tell_ext_types."""
        self._ext_types_known = True
        if self._op_id < 0:
            return
        for dt in ALL_DTYPES:
            try:
                b1, b2, r = _find_buf_dtype2(dt, dt, self.result_type_resolver_fn_, None, acceptance_fn=self.acceptance_fn_)
                ok = r is not None and b1 is None and b2 is None
            except Exception:  # e.g. subtract of bool: the general path raises the function's own error
                ok = False
            _lib.ext.set_binary_type(self._op_id, dtype_id(dt), dtype_id(r) if ok else -1)

    def _fast(self, o1, o2, out=None):
        """The result for two C-contiguous arrays of one shape and one dtype that the kernel
        takes as it is, or for such an array of a floating or complex dtype and a Python float
        or int (which then takes the array's dtype whatever its value); else None.  See
        UnaryElementwiseFunc._fast."""
        if not self._ext_types_known:
            self._tell_ext_types()
        r = _ext_binary_call(self._op_id, o1, o2, out)  # two arrays: the same checks, on the descriptors
        if r is not NotImplemented:
            return r
        t1, t2 = type(o1), type(o2)
        scalar = None
        if t1 is usm_ndarray:
            arr = o1
            if t2 is usm_ndarray:
                if o2._dtype != o1._dtype or o1._shape != o2._shape or not o2._is_c_contiguous():
                    return None
            elif (t2 is float or t2 is int) and o1._dtype.kind in "fc":
                scalar = o2
            else:
                return None
        elif t2 is usm_ndarray and (t1 is float or t1 is int) and o2._dtype.kind in "fc":
            arr, scalar = o2, o1
        else:
            return None
        if not arr._is_c_contiguous():
            return None
        dt = arr._dtype
        res_dt = self._fast_cache.get(dt)
        if res_dt is None:
            b1, b2, r = _find_buf_dtype2(dt, dt, self.result_type_resolver_fn_, None, acceptance_fn=self.acceptance_fn_)
            res_dt = self._fast_cache[dt] = r if (r is not None and b1 is None and b2 is None) else False
        if res_dt is False:
            return None
        if scalar is not None:
            if self.weak_type_resolver_ is not _resolve_weak_types \
                    and self.weak_type_resolver_ is not _resolve_weak_types_all_py_ints:
                return None
            sv = _scalar_operand(scalar, dt, arr._shape)
            if arr is o1:
                o2 = sv
            else:
                o1 = sv
        if out is None:
            out = usm_ndarray._new_contiguous(arr._shape, res_dt)
        elif not _fast_out_ok(out, arr._shape, res_dt) or _spans_meet(out, arr) \
                or (scalar is None and _spans_meet(out, o2)):
            return None
        self.binary_fn_(src1=o1, src2=o2, dst=out)
        return out

    def __call__(self, o1, o2, /, *, out=None, order="K"):
        if order == "K":
            r = self._fast(o1, o2, out)
            if r is not None:
                return r
        order = _norm_order(order)
        res_shape, d1, d2 = self._resolve(o1, o2)
        buf1_dt, buf2_dt, res_dt = _find_buf_dtype2(d1, d2, self.result_type_resolver_fn_, None,
                                                    acceptance_fn=self.acceptance_fn_)
        if res_dt is None:
            raise ValueError(
                f"function '{self.name_}' does not support input types ({d1}, {d2}), "
                "and the inputs could not be safely coerced to any supported types according to "
                "the casting rule ''safe''.")
        if buf1_dt is not None or buf2_dt is not None:
            # "cast one operand (or both) to the result type, then compute": one kernel does it all for some pairs
            # (a dtype compares equal to None when it is float64, hence the explicit tests)
            fused = self._fused_cast(d1, d2)
            if fused is not None and fused == res_dt and (
                    (buf1_dt is not None and buf1_dt == res_dt and buf2_dt is None and d2 == res_dt)
                    or (buf2_dt is not None and buf2_dt == res_dt and buf1_dt is None and d1 == res_dt)
                    or (buf1_dt is not None and buf2_dt is not None and buf1_dt == res_dt and buf2_dt == res_dt)):
                buf1_dt = buf2_dt = None
        orig_out = out
        if out is not None:
            _check_out(out, res_shape, res_dt)
            if isinstance(o1, usm_ndarray) and buf1_dt is None and ti._array_overlap(o1, out):
                if not ti._same_logical_tensors(o1, out):
                    out = empty_like(out)
                elif self.binary_inplace_fn_ is not None:
                    # out is o1 itself: lhs op= rhs
                    rhs = _as_device_array(o2, d2)
                    if buf2_dt is None and isinstance(o2, usm_ndarray) and ti._array_overlap(o2, out) \
                            and not ti._same_logical_tensors(o2, out):
                        buf2_dt = d2
                    if buf2_dt is not None:
                        tmp = empty_like(rhs, dtype=buf2_dt)
                        ti._copy_usm_ndarray_into_usm_ndarray(src=rhs, dst=tmp)
                        rhs = tmp
                    if rhs.shape != res_shape:
                        rhs = broadcast_to(rhs, res_shape)
                    self.binary_inplace_fn_(lhs=o1, rhs=rhs)
                    return out
            if isinstance(o2, usm_ndarray) and buf2_dt is None and out is orig_out \
                    and ti._array_overlap(o2, out) and not ti._same_logical_tensors(o2, out):
                out = empty_like(out)

        src1 = _as_device_array(o1, d1)
        src2 = _as_device_array(o2, d2)
        if order == "A":
            order = "F" if (src1.flags.f_contiguous and src2.flags.f_contiguous) else "C"
        if buf1_dt is not None and buf2_dt is not None and order == "K":
            if src1.flags.c_contiguous and src2.flags.c_contiguous:
                order = "C"
            elif src1.flags.f_contiguous and src2.flags.f_contiguous:
                order = "F"

        def cast(src, bdt):
            if bdt is None:
                return src
            b = _empty_like_orderK(src, bdt) if order == "K" else empty_like(src, dtype=bdt, order=order)
            ti._copy_usm_ndarray_into_usm_ndarray(src=src, dst=b)
            return b

        src1 = cast(src1, buf1_dt)
        src2 = cast(src2, buf2_dt)
        if out is None:
            if order == "K":
                out = _empty_like_pair_orderK(src1, src2, res_dt, res_shape)
            else:
                out = empty(res_shape, dtype=res_dt, order=order)
        if src1.shape != res_shape:
            src1 = broadcast_to(src1, res_shape)
        if src2.shape != res_shape:
            src2 = broadcast_to(src2, res_shape)
        self.binary_fn_(src1=src1, src2=src2, dst=out)
        if orig_out is not None and orig_out is not out:
            ti._copy_usm_ndarray_into_usm_ndarray(src=out, dst=orig_out)
            out = orig_out
        return out

    def _inplace_op(self, o1, o2):
        """o1 op= o2 with the dedicated in-place kernel; o1 is never cast or reallocated."""
        if self.binary_inplace_fn_ is None:
            raise ValueError("binary function does not have a dedicated in-place implementation")
        if not isinstance(o1, usm_ndarray):
            raise TypeError(f"Expected first argument to be dpnp_amd.tensor.usm_ndarray, got {type(o1)}")
        if not o1.flags.writable:
            raise ValueError("provided left-hand side array is read-only")
        s2 = _operand_shape(o2)
        if s2 is None:
            raise TypeError("Shape of second argument can not be inferred. Expected list or tuple.")
        try:
            res_shape = _broadcast_shape_impl([o1.shape, s2])
        except ValueError:
            raise ValueError(f"operands could not be broadcast together with shapes {o1.shape} and {s2}")
        if res_shape != o1.shape:
            raise ValueError(f"The shape of the non-broadcastable left-hand side {o1.shape} is "
                             f"inconsistent with the broadcast shape {res_shape}.")
        d2 = _operand_dtype(o2)
        if d2 is None:
            raise ValueError("Operand has an unsupported data type")
        d1, d2 = self.weak_type_resolver_(o1.dtype, d2, None)
        buf_dt, res_dt = _find_buf_dtype_in_place_op(d1, d2, self.result_type_resolver_fn_, None)
        if res_dt is None:
            raise ValueError(
                f"function '{self.name_}' does not support input types ({d1}, {d2}), "
                "and the inputs could not be safely coerced to any supported types according to "
                "the casting rule ''same_kind''.")
        if res_dt != d1:
            raise ValueError(f"Output array of type {res_dt} is needed, got {d1}")
        if buf_dt is not None and buf_dt == d1:
            fused = self._fused_cast(d1, d2)
            if fused is not None and fused == d1:
                buf_dt = None  # the kernel converts the right operand while reading it
        rhs = _as_device_array(o2, d2)
        if buf_dt is None and isinstance(o2, usm_ndarray) and ti._array_overlap(o2, o1) \
                and not ti._same_logical_tensors(o2, o1):
            buf_dt = d2
        if buf_dt is not None:
            tmp = empty_like(rhs, dtype=buf_dt)
            ti._copy_usm_ndarray_into_usm_ndarray(src=rhs, dst=tmp)
            rhs = tmp
        if rhs.shape != res_shape:
            rhs = broadcast_to(rhs, res_shape)
        self.binary_inplace_fn_(lhs=o1, rhs=rhs)
        return o1
