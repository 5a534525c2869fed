"""dpnp_amd.tensor: the array-API layer over the HIP kernels (counterpart of dpnp.tensor
for elementwise functions, `where` and axis reductions)."""
from ._copy_utils import asnumpy, astype, copy, from_numpy, to_numpy
from ._ctors import (
    arange,
    asarray,
    empty,
    empty_like,
    full,
    full_like,
    linspace,
    ones,
    ones_like,
    zeros,
    zeros_like,
)
from ._device import Device, ExecutionPlacementError, Queue, get_execution_queue
from ._dtypes import (
    bool,
    complex64,
    complex128,
    dtype,
    finfo,
    float16,
    float32,
    float64,
    iinfo,
    int8,
    int16,
    int32,
    int64,
    isdtype,
    uint8,
    uint16,
    uint32,
    uint64,
)
from ._elementwise_funcs import *  # noqa: F401,F403
from ._elementwise_funcs import abs, pow, round  # noqa: A004
from ._manipulation_functions import (
    concat,
    diff,
    stack,
    broadcast_arrays,
    broadcast_to,
    expand_dims,
    flip,
    matrix_transpose,
    moveaxis,
    permute_dims,
    reshape,
    squeeze,
    swapaxes,
)
from ._reduction import (  # noqa: A004
    all,
    any,
    argmax,
    argmin,
    count_nonzero,
    logsumexp,
    max,
    min,
    prod,
    reduce_hypot,
    sum,
)
from ._search_functions import where
from ._clip import clip
from ._statistical_functions import mean, std, var
from ._type_utils import can_cast, result_type
from ._usmarray import usm_ndarray
from ._array_api import __array_api_version__, __array_namespace_info__  # noqa: E402
from ._testing import allclose  # noqa: E402

e = 2.718281828459045
pi = 3.141592653589793
nan = float("nan")
inf = float("inf")
newaxis = None
