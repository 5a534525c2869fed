"""dpnp_array: the NumPy-flavoured ndarray of the package, a thin wrapper over a
usm_ndarray (role of dpnp/dpnp_array.py: construction, views, operators and the
sum/max/argmax/mean/var methods that sit on the elementwise + reduction path)."""
import numpy as np

from . import tensor as dpt
from .tensor._usmarray import usm_ndarray


class dpnp_array:
    """ndarray(shape, dtype=None, buffer=None, offset=0, strides=None, order="C")"""

    __array_priority__ = 200.0

    def __init__(self, shape, dtype=None, buffer=None, offset=0, strides=None, order="C",
                 device=None, usm_type="device", sycl_queue=None):
        if order is None:
            order = "C"
        if buffer is not None:
            buffer = buffer.get_array() if isinstance(buffer, dpnp_array) else buffer
        self._array_obj = usm_ndarray(shape, dtype="f8" if dtype is None else dtype, strides=strides,
                                      buffer=buffer, offset=offset, order=order.upper())

    @staticmethod
    def _create_from_usm_ndarray(usm_ary):
        if not isinstance(usm_ary, usm_ndarray):
            raise TypeError(f"Expected dpnp_amd.tensor.usm_ndarray, got {type(usm_ary)}")
        r = dpnp_array.__new__(dpnp_array)
        r._array_obj = usm_ary
        return r

    def get_array(self):
        """The underlying usm_ndarray."""
        return self._array_obj

    # -- attributes ---------------------------------------------------------------------------
    shape = property(lambda s: s._array_obj.shape)
    strides = property(lambda s: tuple(st * s._array_obj.itemsize for st in s._array_obj.strides))
    dtype = property(lambda s: s._array_obj.dtype)
    ndim = property(lambda s: s._array_obj.ndim)
    size = property(lambda s: s._array_obj.size)
    itemsize = property(lambda s: s._array_obj.itemsize)
    nbytes = property(lambda s: s._array_obj.nbytes)
    flags = property(lambda s: s._array_obj.flags)
    sycl_queue = property(lambda s: s._array_obj.sycl_queue)
    sycl_device = property(lambda s: s._array_obj.sycl_device)
    usm_type = property(lambda s: s._array_obj.usm_type)
    device = property(lambda s: s._array_obj.device)
    T = property(lambda s: dpnp_array._create_from_usm_ndarray(s._array_obj.T))
    mT = property(lambda s: dpnp_array._create_from_usm_ndarray(s._array_obj.mT))
    real = property(lambda s: dpnp_array._create_from_usm_ndarray(s._array_obj.real))
    imag = property(lambda s: dpnp_array._create_from_usm_ndarray(s._array_obj.imag))

    def __getitem__(self, key):
        key = key.get_array() if isinstance(key, dpnp_array) else key
        return dpnp_array._create_from_usm_ndarray(self._array_obj[key])

    def __setitem__(self, key, val):
        val = val.get_array() if isinstance(val, dpnp_array) else val
        self._array_obj[key] = val

    def __len__(self):
        return len(self._array_obj)

    def __iter__(self):
        return (self[i] for i in range(len(self)))

    def __bool__(self):
        return bool(self._array_obj)

    def __float__(self):
        return float(self._array_obj)

    def __int__(self):
        return int(self._array_obj)

    def __complex__(self):
        return complex(self._array_obj)

    def __index__(self):
        return self._array_obj.__index__()

    def __repr__(self):
        r = repr(self._array_obj)
        return "array" + r[len("usm_ndarray"):] if r.startswith("usm_ndarray") else r

    def __str__(self):
        return str(self._array_obj)

    def asnumpy(self):
        return dpt.asnumpy(self._array_obj)

    def item(self):
        return self._array_obj._scalar()

    def astype(self, dtype, order="K", casting="unsafe", subok=True, copy=True, device=None):
        return dpnp_array._create_from_usm_ndarray(
            dpt.astype(self._array_obj, dtype, order=order, casting=casting, copy=copy))

    def clip(self, /, min=None, max=None, out=None, **kwargs):  # noqa: A002
        from . import dpnp_iface

        return dpnp_iface.clip(self, min, max, out=out, **kwargs)

    def copy(self, order="C"):
        return dpnp_array._create_from_usm_ndarray(dpt.copy(self._array_obj, order=order))

    def reshape(self, *shape, order="C", copy=None):
        if len(shape) == 1 and isinstance(shape[0], (tuple, list)):
            shape = shape[0]
        return dpnp_array._create_from_usm_ndarray(dpt.reshape(self._array_obj, shape, order=order, copy=copy))

    def transpose(self, *axes):
        if not axes or axes == (None,):
            return self.T
        if len(axes) == 1 and isinstance(axes[0], (tuple, list)):
            axes = axes[0]
        return dpnp_array._create_from_usm_ndarray(dpt.permute_dims(self._array_obj, axes))

    def squeeze(self, axis=None):
        return dpnp_array._create_from_usm_ndarray(dpt.squeeze(self._array_obj, axis))

    def fill(self, value):
        self._array_obj[...] = value

    # -- reductions as methods ---------------------------------------------------------------------
    def sum(self, axis=None, dtype=None, out=None, keepdims=False, initial=None, where=True):
        from . import dpnp_iface as dpnp

        return dpnp.sum(self, axis=axis, dtype=dtype, out=out, keepdims=keepdims, initial=initial, where=where)

    def prod(self, axis=None, dtype=None, out=None, keepdims=False, initial=None, where=True):
        from . import dpnp_iface as dpnp

        return dpnp.prod(self, axis=axis, dtype=dtype, out=out, keepdims=keepdims, initial=initial, where=where)

    def max(self, axis=None, out=None, keepdims=False, initial=None, where=True):
        from . import dpnp_iface as dpnp

        return dpnp.max(self, axis=axis, out=out, keepdims=keepdims, initial=initial, where=where)

    def min(self, axis=None, out=None, keepdims=False, initial=None, where=True):
        from . import dpnp_iface as dpnp

        return dpnp.min(self, axis=axis, out=out, keepdims=keepdims, initial=initial, where=where)

    def argmax(self, axis=None, out=None, *, keepdims=False):
        from . import dpnp_iface as dpnp

        return dpnp.argmax(self, axis=axis, out=out, keepdims=keepdims)

    def argmin(self, axis=None, out=None, *, keepdims=False):
        from . import dpnp_iface as dpnp

        return dpnp.argmin(self, axis=axis, out=out, keepdims=keepdims)

    def mean(self, axis=None, dtype=None, out=None, keepdims=False, *, where=True):
        from . import dpnp_iface as dpnp

        return dpnp.mean(self, axis=axis, dtype=dtype, out=out, keepdims=keepdims, where=where)

    def var(self, axis=None, dtype=None, out=None, ddof=0, keepdims=False, *, where=True, mean=None,
            correction=None):
        from . import dpnp_iface as dpnp

        return dpnp.var(self, axis=axis, dtype=dtype, out=out, ddof=ddof, keepdims=keepdims, where=where,
                        mean=mean, correction=correction)

    def std(self, axis=None, dtype=None, out=None, ddof=0, keepdims=False, *, where=True, mean=None,
            correction=None):
        from . import dpnp_iface as dpnp

        return dpnp.std(self, axis=axis, dtype=dtype, out=out, ddof=ddof, keepdims=keepdims, where=where,
                        mean=mean, correction=correction)

    def all(self, axis=None, out=None, keepdims=False, *, where=True):
        from . import dpnp_iface as dpnp

        return dpnp.all(self, axis=axis, out=out, keepdims=keepdims, where=where)

    def any(self, axis=None, out=None, keepdims=False, *, where=True):
        from . import dpnp_iface as dpnp

        return dpnp.any(self, axis=axis, out=out, keepdims=keepdims, where=where)

    def round(self, decimals=0, out=None):
        from . import dpnp_iface_compositions as comp

        return comp.round(self, decimals, out)

    def conj(self):
        """Complex conjugate; an array of a real dtype comes back as it is (dpnp_array.conj)."""
        from . import dpnp_iface as dpnp

        return dpnp.conj(self) if self.dtype.kind == "c" else self

    conjugate = conj

    def __copy__(self):
        return self.copy(order="K")

    def __array_namespace__(self, /, *, api_version=None):
        return self._array_obj.__array_namespace__(api_version=api_version)

    def swapaxes(self, axis1, axis2):
        return dpnp_array._create_from_usm_ndarray(dpt.swapaxes(self._array_obj, axis1, axis2))

    def ravel(self, order="C"):
        from . import dpnp_iface_manipulation as manip

        return manip.ravel(self, order=order)

    def flatten(self, order="C"):
        """A 1-D copy of the elements in the given order."""
        return self.reshape(-1, order=order, copy=True)

    def tolist(self):
        return self.asnumpy().tolist()

    # -- operators ------------------------------------------------------------------------------------
    def _b(self, name, other, reflected=False):
        from . import dpnp_iface as dpnp

        f = getattr(dpnp, name)
        return f(other, self) if reflected else f(self, other)

    def _ib(self, name, other):
        from . import dpnp_iface as dpnp

        getattr(dpnp, name)(self, other, out=self)
        return self

    def __add__(self, o): return self._b("add", o)
    def __radd__(self, o): return self._b("add", o, True)
    def __iadd__(self, o): return self._ib("add", o)
    def __sub__(self, o): return self._b("subtract", o)
    def __rsub__(self, o): return self._b("subtract", o, True)
    def __isub__(self, o): return self._ib("subtract", o)
    def __mul__(self, o): return self._b("multiply", o)
    def __rmul__(self, o): return self._b("multiply", o, True)
    def __imul__(self, o): return self._ib("multiply", o)
    def __truediv__(self, o): return self._b("divide", o)
    def __rtruediv__(self, o): return self._b("divide", o, True)
    def __itruediv__(self, o): return self._ib("divide", o)
    def __floordiv__(self, o): return self._b("floor_divide", o)
    def __rfloordiv__(self, o): return self._b("floor_divide", o, True)
    def __mod__(self, o): return self._b("remainder", o)
    def __rmod__(self, o): return self._b("remainder", o, True)
    def __pow__(self, o): return self._b("power", o)
    def __rpow__(self, o): return self._b("power", o, True)
    def __and__(self, o): return self._b("bitwise_and", o)
    def __rand__(self, o): return self._b("bitwise_and", o, True)
    def __iand__(self, o): return self._ib("bitwise_and", o)
    def __or__(self, o): return self._b("bitwise_or", o)
    def __ror__(self, o): return self._b("bitwise_or", o, True)
    def __ior__(self, o): return self._ib("bitwise_or", o)
    def __xor__(self, o): return self._b("bitwise_xor", o)
    def __rxor__(self, o): return self._b("bitwise_xor", o, True)
    def __ixor__(self, o): return self._ib("bitwise_xor", o)
    def __lshift__(self, o): return self._b("left_shift", o)
    def __rlshift__(self, o): return self._b("left_shift", o, True)
    def __ilshift__(self, o): return self._ib("left_shift", o)
    def __rshift__(self, o): return self._b("right_shift", o)
    def __rrshift__(self, o): return self._b("right_shift", o, True)
    def __irshift__(self, o): return self._ib("right_shift", o)
    def __ifloordiv__(self, o): return self._ib("floor_divide", o)
    def __imod__(self, o): return self._ib("remainder", o)
    def __ipow__(self, o): return self._ib("power", o)
    def __divmod__(self, o): return self._b("divmod", o)
    def __rdivmod__(self, o): return self._b("divmod", o, True)
    def __eq__(self, o): return self._b("equal", o)
    def __ne__(self, o): return self._b("not_equal", o)
    def __lt__(self, o): return self._b("less", o)
    def __le__(self, o): return self._b("less_equal", o)
    def __gt__(self, o): return self._b("greater", o)
    def __ge__(self, o): return self._b("greater_equal", o)
    __hash__ = None

    def __neg__(self):
        from . import dpnp_iface as dpnp

        return dpnp.negative(self)

    def __pos__(self):
        from . import dpnp_iface as dpnp

        return dpnp.positive(self)

    def __abs__(self):
        from . import dpnp_iface as dpnp

        return dpnp.abs(self)

    def __invert__(self):
        from . import dpnp_iface as dpnp

        return dpnp.invert(self)


def _register_with_ext():
    from . import _lib

    _lib.ext.set_array_class(dpnp_array, dpnp_array._create_from_usm_ndarray)


_register_with_ext()


def _np_scalar_or(x):
    return x.item() if isinstance(x, np.generic) else x
