"""dpnp_amd: the elementwise + axis-reduction core of dpnp on AMD MI355X.

`dpnp_amd.tensor` is the array-API layer (usm_ndarray and functions); this top-level
namespace is the NumPy-flavoured surface (`ndarray`, add, multiply, exp, where, sum, max,
argmax, mean, var ...).  All arithmetic runs in hand-written HIP kernels reached through
the C ABI of libdpnp_amd.so; importing fails if that library is not built.
"""
from . import _lib  # noqa: F401  (loads libdpnp_amd.so or raises)
from . import tensor  # noqa: F401
from .dpnp_iface import *  # noqa: F401,F403
from .dpnp_iface import __all__ as _iface_all
from .dpnp_iface_nanfunctions import *  # noqa: F401,F403
from .dpnp_iface_nanfunctions import __all__ as _nan_all
from .dpnp_iface_compositions import *  # noqa: F401,F403
from .dpnp_iface_compositions import __all__ as _comp_all
from .dpnp_iface_types import *  # noqa: F401,F403
from .dpnp_iface_types import __all__ as _types_all
from .dpnp_iface_manipulation import *  # noqa: F401,F403
from .dpnp_iface_manipulation import __all__ as _manip_all
from .dpnp_array import dpnp_array as ndarray

__all__ = list(_iface_all) + list(_nan_all) + list(_comp_all) + list(_types_all) + list(_manip_all) + ["ndarray", "tensor"]
__version__ = "0.1.0"
