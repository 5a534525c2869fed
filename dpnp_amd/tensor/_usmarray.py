"""usm_ndarray: a strided N-d view of device memory.

Plays the role of dpnp.tensor.usm_ndarray (dpnp/tensor/_usmarray.pyx): shape, element
strides, dtype, contiguity/writable flags and a base allocation.  Basic indexing makes
views (NumPy rules, as dpnp/tensor/_slicing.pyx); arithmetic operators forward to the
elementwise functions of this package.
"""
import operator

import numpy as np

from .. import _lib
from . import _device
from ._dtypes import dtype as _as_dtype
from ._dtypes import dtype_id


def _contig_strides(shape, order="C"):
    st = [0] * len(shape)
    acc = 1
    rng = range(len(shape) - 1, -1, -1) if order == "C" else range(len(shape))
    for d in rng:
        st[d] = acc
        acc *= max(int(shape[d]), 1)
    return tuple(st)


def _contig_flags(shape, strides):
    """(c_contiguous, f_contiguous) by NumPy's rules: extent-1 dims do not matter."""
    if any(s == 0 for s in shape):
        return True, True
    c = f = True
    acc = 1
    for d in range(len(shape) - 1, -1, -1):
        if shape[d] != 1:
            if strides[d] != acc:
                c = False
            acc *= shape[d]
    acc = 1
    for d in range(len(shape)):
        if shape[d] != 1:
            if strides[d] != acc:
                f = False
            acc *= shape[d]
    return c, f


class Flags:
    """The flags of an array: contiguity and writability."""

    def __init__(self, arr):
        self._arr = arr

    @property
    def c_contiguous(self):
        return _contig_flags(self._arr.shape, self._arr.strides)[0]

    @property
    def f_contiguous(self):
        return _contig_flags(self._arr.shape, self._arr.strides)[1]

    @property
    def contiguous(self):
        return self.forc

    @property
    def forc(self):
        c, f = _contig_flags(self._arr.shape, self._arr.strides)
        return c or f

    @property
    def fnc(self):
        c, f = _contig_flags(self._arr.shape, self._arr.strides)
        return f and not c

    @property
    def writable(self):
        return self._arr._writable

    @writable.setter
    def writable(self, value):
        if not isinstance(value, bool):
            raise TypeError("Expecting type bool")
        self._arr._writable = value

    def __getitem__(self, name):
        table = {"C": "c_contiguous", "C_CONTIGUOUS": "c_contiguous", "F": "f_contiguous",
                 "F_CONTIGUOUS": "f_contiguous", "W": "writable", "WRITABLE": "writable",
                 "FNC": "fnc", "FORC": "forc", "CONTIGUOUS": "forc"}
        if name not in table:
            raise KeyError(f"Unknown flag name: {name}")
        return getattr(self, table[name])

    def __setitem__(self, name, value):
        # only the writable flag can be changed (dpnp/tensor/_flags.pyx: "W" / "WRITABLE")
        if name not in ("W", "WRITABLE"):
            raise ValueError("Only writable ('W' or 'WRITABLE') flag can be set")
        self.writable = value

    def __repr__(self):
        return (f"  C_CONTIGUOUS : {self.c_contiguous}\n  F_CONTIGUOUS : {self.f_contiguous}\n"
                f"  WRITABLE : {self.writable}")


class usm_ndarray:
    """usm_ndarray(shape, dtype="f8", strides=None, buffer=None, offset=0, order="C")

    `buffer` is None (allocate), another usm_ndarray (share its allocation) or a
    uint8 device allocation made by this package; `offset` and `strides` count
    elements.
    """

    __array_priority__ = 100.0

    def __init__(self, shape, dtype="f8", strides=None, buffer=None, offset=0, order="C",
                 writable=True):
        if isinstance(shape, (int, np.integer)):
            shape = (int(shape),)
        shape = tuple(operator.index(s) for s in shape)
        if any(s < 0 for s in shape):
            raise ValueError("negative dimensions are not allowed")
        if len(shape) > _lib.MAX_ND:
            raise ValueError(f"arrays of more than {_lib.MAX_ND} dimensions are not supported")
        dt = _as_dtype(dtype)
        if order not in ("C", "F"):
            raise ValueError("order must be 'C' or 'F'")
        if strides is None:
            strides = _contig_strides(shape, order)
        else:
            strides = tuple(operator.index(s) for s in strides)
            if len(strides) != len(shape):
                raise ValueError("strides and shape must have the same length")
        self._shape = shape
        self._strides = strides
        self._dtype = dt
        self._offset = int(offset)
        self._writable = bool(writable)
        size = 1
        for s in shape:
            size *= s
        lo = hi = 0
        if size:
            for s, st in zip(shape, strides):
                if st < 0:
                    lo += (s - 1) * st
                else:
                    hi += (s - 1) * st
        if buffer is None:
            if self._offset + lo < 0:
                raise ValueError("offset and strides address memory before the allocation")
            self._buf = _device.alloc((self._offset + hi + 1) * dt.itemsize if size else 0)
            self._base = None
        else:
            if isinstance(buffer, usm_ndarray):
                self._buf = buffer._buf
                self._base = buffer._base if buffer._base is not None else buffer
            else:
                self._buf = buffer
                self._base = None
            if size and ((self._offset + lo) < 0 or
                         (self._offset + hi + 1) * dt.itemsize > self._buf.numel()):
                raise ValueError("shape, strides and offset address memory outside the allocation")

    @staticmethod
    def _new_contiguous(shape, dt, order="C"):
        """Freshly allocated C- or F-contiguous array (arguments already normalised)."""
        r = usm_ndarray.__new__(usm_ndarray)
        size = 1
        for s in shape:
            size *= s
        r._shape = shape
        r._strides = _contig_strides(shape, order)
        r._dtype = dt
        r._offset = 0
        r._writable = True
        r._buf = _device.alloc(size * dt.itemsize)
        r._base = None
        return r

    # -- construction of views -------------------------------------------------------------
    def _view(self, shape, strides, offset, dtype=None):
        r = usm_ndarray.__new__(usm_ndarray)
        r._shape = tuple(shape)
        r._strides = tuple(strides)
        r._dtype = self._dtype if dtype is None else dtype
        r._offset = offset
        r._writable = self._writable
        r._buf = self._buf
        r._base = self._base if self._base is not None else self
        return r

    # -- basic properties --------------------------------------------------------------------
    @property
    def shape(self):
        return self._shape

    @shape.setter
    def shape(self, new_shape):
        from ._manipulation_functions import reshape

        r = reshape(self, new_shape, copy=False)
        self._shape, self._strides = r._shape, r._strides
        self.__dict__.pop("_cview", None)
        self.__dict__.pop("_perm_views", None)

    @property
    def strides(self):
        return self._strides

    @property
    def dtype(self):
        return self._dtype

    @property
    def ndim(self):
        return len(self._shape)

    @property
    def size(self):
        n = 1
        for s in self._shape:
            n *= s
        return n

    @property
    def itemsize(self):
        return self._dtype.itemsize

    @property
    def nbytes(self):
        return self.size * self._dtype.itemsize

    @property
    def flags(self):
        return Flags(self)

    @property
    def base(self):
        return self._base

    @property
    def usm_type(self):
        return "device"

    @property
    def sycl_queue(self):
        return _device.default_queue()

    @property
    def sycl_device(self):
        return _device.default_queue().sycl_device

    @property
    def device(self):
        return _device.default_queue().sycl_device

    @property
    def usm_data(self):
        """The allocation this array lives in (one object for an array and all of its views)."""
        return self._buf

    @property
    def _pointer(self):
        return self._buf.data_ptr() + self._offset * self._dtype.itemsize

    @property
    def _element_offset(self):
        return self._offset

    def _as_view(self):
        """The C descriptor of this array (borrowed; valid while `self` is alive).  Built once:
        shape, strides, offset and allocation of an array object never change; only the
        writable bit may."""
        try:
            v = self._cview
        except AttributeError:
            c, f = _contig_flags(self._shape, self._strides)
            flags = (_lib.C_CONTIGUOUS if c else 0) | (_lib.F_CONTIGUOUS if f else 0)
            ptr = self._pointer
            v = self._cview = _lib.make_view(ptr, self._shape, self._strides, dtype_id(self._dtype), flags)
            self._cview_c = c
            self._cview_w = None
            n = 1
            for d in self._shape:
                n *= d
            self._cview_span = (ptr, ptr + n * self._dtype.itemsize)  # the bytes of a contiguous array
        if self._cview_w is not self._writable:
            w = self._cview_w = bool(self._writable)
            self._writable = w
            v.flags = (v.flags & ~_lib.WRITABLE) | (_lib.WRITABLE if w else 0)
        return v

    def _contiguous_span(self):
        """(first byte, one past the last byte) of a C- or F-contiguous array."""
        try:
            return self._cview_span
        except AttributeError:
            self._as_view()
            return self._cview_span

    def _is_c_contiguous(self):
        """C-contiguity by NumPy's rules, computed once per array object."""
        try:
            return self._cview_c
        except AttributeError:
            self._as_view()
            return self._cview_c

    @property
    def T(self):
        if self.ndim < 2:
            return self
        return self._view(self._shape[::-1], self._strides[::-1], self._offset)

    @property
    def mT(self):
        if self.ndim < 2:
            raise ValueError("array.mT requires array to have at least 2 dimensions.")
        sh, st = list(self._shape), list(self._strides)
        sh[-1], sh[-2] = sh[-2], sh[-1]
        st[-1], st[-2] = st[-2], st[-1]
        return self._view(sh, st, self._offset)

    @property
    def real(self):
        if self._dtype.kind != "c":
            return self
        half = np.dtype("f4") if self._dtype.itemsize == 8 else np.dtype("f8")
        return self._view(self._shape, tuple(2 * s for s in self._strides), 2 * self._offset, dtype=half)

    @property
    def imag(self):
        if self._dtype.kind != "c":
            from ._ctors import zeros_like

            r = zeros_like(self)
            r._writable = False
            return r
        half = np.dtype("f4") if self._dtype.itemsize == 8 else np.dtype("f8")
        return self._view(self._shape, tuple(2 * s for s in self._strides), 2 * self._offset + 1, dtype=half)

    # -- indexing -------------------------------------------------------------------------------
    def _basic_index(self, key):
        if not isinstance(key, tuple):
            key = (key,)
        for k in key:
            if not (k is None or k is Ellipsis or isinstance(k, (slice, int, np.integer))):
                if isinstance(k, (usm_ndarray, np.ndarray, list)):
                    raise NotImplementedError(
                        "advanced (integer or boolean array) indexing is outside this library's scope; "
                        "use basic slices, integers, None and Ellipsis")
                raise IndexError("only integers, slices (`:`), ellipsis (`...`) and None are valid indices")
        n_ell = sum(1 for k in key if k is Ellipsis)
        if n_ell > 1:
            raise IndexError("an index can only have a single ellipsis ('...')")
        n_idx = sum(1 for k in key if k is not None and k is not Ellipsis)
        if n_idx > self.ndim:
            raise IndexError(f"too many indices for array: array is {self.ndim}-dimensional, "
                             f"but {n_idx} were indexed")
        if n_ell == 0:
            key = key + (Ellipsis,)
        shape, strides, offset = [], [], self._offset
        d = 0
        for k in key:
            if k is None:
                shape.append(1)
                strides.append(0)
            elif k is Ellipsis:
                for _ in range(self.ndim - n_idx):
                    shape.append(self._shape[d])
                    strides.append(self._strides[d])
                    d += 1
            elif isinstance(k, slice):
                start, stop, step = k.indices(self._shape[d])
                n = len(range(start, stop, step))
                shape.append(n)
                strides.append(self._strides[d] * step if n > 0 else 1)
                offset += start * self._strides[d] if n > 0 else 0
                d += 1
            else:
                i = operator.index(k)
                ext = self._shape[d]
                if i < -ext or i >= ext:
                    raise IndexError(f"index {i} is out of bounds for axis {d} with size {ext}")
                offset += (i + ext if i < 0 else i) * self._strides[d]
                d += 1
        return self._view(shape, strides, offset)

    def __getitem__(self, key):
        return self._basic_index(key)

    def __setitem__(self, key, value):
        if not self._writable:
            raise ValueError("Can not modify read-only array.")
        from . import _copy_utils as cu

        cu._assign(self._basic_index(key), value)

    # -- conversions ------------------------------------------------------------------------------
    def _scalar(self):
        if self.size != 1:
            raise ValueError("only size-1 arrays can be converted to Python scalars")
        from ._copy_utils import asnumpy

        return asnumpy(self).reshape(()).item()

    def __bool__(self):
        if self.size == 0:
            raise ValueError("The truth value of an empty array is ambiguous")
        if self.size != 1:
            raise ValueError("The truth value of an array with more than one element is ambiguous. "
                             "Use dpnp_amd.tensor.any() or dpnp_amd.tensor.all()")
        return bool(self._scalar())

    def __float__(self):
        return float(self._scalar())

    def __int__(self):
        return int(self._scalar())

    def __complex__(self):
        return complex(self._scalar())

    def __index__(self):
        if self._dtype.kind not in "iu":
            raise IndexError("only integer arrays are valid indices")
        return int(self._scalar())

    def __len__(self):
        if self.ndim == 0:
            raise TypeError("len() of unsized object")
        return self._shape[0]

    def __iter__(self):
        if self.ndim == 0:
            raise TypeError("iteration over a 0-d array")
        return (self[i] for i in range(self._shape[0]))

    def __repr__(self):
        from ._copy_utils import asnumpy

        if not _device.gpu_available():
            return f"usm_ndarray(shape={self._shape}, dtype={self._dtype})"
        body = repr(asnumpy(self))
        return "usm_ndarray" + body[body.index("("):] if body.startswith("array") else body

    def __str__(self):
        from ._copy_utils import asnumpy

        return str(asnumpy(self))

    def __array_namespace__(self, api_version=None):
        import dpnp_amd.tensor as dpt

        return dpt

    def to_device(self, target_device, /, *, stream=None):
        return self

    def __dlpack_device__(self):
        return (10, 0)  # kDLROCM, device 0

    # -- operators ------------------------------------------------------------------------------------
    def _fn(self, name):
        from . import _elementwise_funcs as ef

        return getattr(ef, name)

    def __add__(self, o): return self._fn("add")(self, o)
    def __radd__(self, o): return self._fn("add")(o, self)
    def __sub__(self, o): return self._fn("subtract")(self, o)
    def __rsub__(self, o): return self._fn("subtract")(o, self)
    def __mul__(self, o): return self._fn("multiply")(self, o)
    def __rmul__(self, o): return self._fn("multiply")(o, self)
    def __truediv__(self, o): return self._fn("divide")(self, o)
    def __rtruediv__(self, o): return self._fn("divide")(o, self)
    def __floordiv__(self, o): return self._fn("floor_divide")(self, o)
    def __rfloordiv__(self, o): return self._fn("floor_divide")(o, self)
    def __mod__(self, o): return self._fn("remainder")(self, o)
    def __rmod__(self, o): return self._fn("remainder")(o, self)
    def __pow__(self, o): return self._fn("pow")(self, o)
    def __rpow__(self, o): return self._fn("pow")(o, self)
    def __and__(self, o): return self._fn("bitwise_and")(self, o)
    def __rand__(self, o): return self._fn("bitwise_and")(o, self)
    def __or__(self, o): return self._fn("bitwise_or")(self, o)
    def __ror__(self, o): return self._fn("bitwise_or")(o, self)
    def __xor__(self, o): return self._fn("bitwise_xor")(self, o)
    def __rxor__(self, o): return self._fn("bitwise_xor")(o, self)
    def __lshift__(self, o): return self._fn("bitwise_left_shift")(self, o)
    def __rlshift__(self, o): return self._fn("bitwise_left_shift")(o, self)
    def __rshift__(self, o): return self._fn("bitwise_right_shift")(self, o)
    def __rrshift__(self, o): return self._fn("bitwise_right_shift")(o, self)
    def __neg__(self): return self._fn("negative")(self)
    def __pos__(self): return self._fn("positive")(self)
    def __abs__(self): return self._fn("abs")(self)
    def __invert__(self): return self._fn("bitwise_invert")(self)
    def __eq__(self, o): return self._fn("equal")(self, o)
    def __ne__(self, o): return self._fn("not_equal")(self, o)
    def __lt__(self, o): return self._fn("less")(self, o)
    def __le__(self, o): return self._fn("less_equal")(self, o)
    def __gt__(self, o): return self._fn("greater")(self, o)
    def __ge__(self, o): return self._fn("greater_equal")(self, o)
    __hash__ = None

    def __iadd__(self, o): return self._fn("add")._inplace_op(self, o)
    def __isub__(self, o): return self._fn("subtract")._inplace_op(self, o)
    def __imul__(self, o): return self._fn("multiply")._inplace_op(self, o)
    def __itruediv__(self, o): return self._fn("divide")._inplace_op(self, o)
    def __ifloordiv__(self, o): return self._fn("floor_divide")._inplace_op(self, o)
    def __imod__(self, o): return self._fn("remainder")._inplace_op(self, o)
    def __ipow__(self, o): return self._fn("pow")._inplace_op(self, o)
    def __iand__(self, o): return self._fn("bitwise_and")._inplace_op(self, o)
    def __ior__(self, o): return self._fn("bitwise_or")._inplace_op(self, o)
    def __ixor__(self, o): return self._fn("bitwise_xor")._inplace_op(self, o)
    def __ilshift__(self, o): return self._fn("bitwise_left_shift")._inplace_op(self, o)
    def __irshift__(self, o): return self._fn("bitwise_right_shift")._inplace_op(self, o)


def _ext_alloc(shape, dt_id):
    """Fresh C-contiguous array for the extension module's calls that make their own result."""
    from ._dtypes import ALL_DTYPES

    return usm_ndarray._new_contiguous(shape, ALL_DTYPES[dt_id])


def _init_ext():
    from ._tensor_impl import _events

    # the stream: the library's own is one per process (asked for once, at the first call that needs it);
    # PyTorch's current stream is asked for at every call
    _lib.ext.init(usm_ndarray, _device.current_stream_ptr, _lib.MEMORY == "native", _events, _ext_alloc)


_init_ext()
