"""Python host layer without a GPU: type promotion, weak scalars, view arithmetic, layout
of results.  Arrays here sit on a host byte buffer: only descriptors are exercised."""
import numpy as np
import pytest

import dpnp_amd.tensor as dpt
from dpnp_amd.tensor import _tensor_elementwise_impl as tei
from dpnp_amd.tensor import _type_utils as tu
from dpnp_amd.tensor._copy_utils import _empty_like_orderK, _empty_like_pair_orderK
from dpnp_amd.tensor._manipulation_functions import _reshape_strides
from dpnp_amd.tensor._usmarray import usm_ndarray

ALL = list(dpt._dtypes.ALL_DTYPES)


class HostBytes:
    """Host memory with the two methods this package uses of an allocation."""

    def __init__(self, nbytes):
        self.a = np.empty(max(int(nbytes), 1), dtype=np.uint8)

    def data_ptr(self):
        return self.a.ctypes.data

    def numel(self):
        return self.a.size


def host_array(shape, dtype="f4", order="C"):
    n = int(np.prod(shape)) if len(shape) else 1
    buf = HostBytes(max(n, 1) * np.dtype(dtype).itemsize)
    return usm_ndarray(shape, dtype=dtype, buffer=buf, order=order)


def np_like(x):
    """NumPy array with the same shape and element strides (for cross-checking view math)."""
    base = np.empty(x._buf.numel() // x.itemsize, dtype=x.dtype)
    return np.lib.stride_tricks.as_strided(base[x._offset:], x.shape, [s * x.itemsize for s in x.strides])


@pytest.fixture(autouse=True)
def _host_alloc(monkeypatch):
    # allocations made by the layout helpers go to host bytes in these tests
    from dpnp_amd.tensor import _device

    monkeypatch.setattr(_device, "alloc", HostBytes)


# ---- promotion ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("op", ["add", "multiply", "maximum"])
def test_binary_promotion_matches_numpy(op):
    # dpnp/tests/tensor/elementwise/test_add.py:62-65
    q = getattr(tei, f"_{op}_result_type")
    for d1 in ALL:
        for d2 in ALL:
            b1, b2, r = tu._find_buf_dtype2(d1, d2, q)
            assert r == np.result_type(d1, d2)
            assert (b1 is None) == (d1 == r) or q(d1, d2) is not None
            if b1 is not None:
                assert np.can_cast(d1, b1)
            if b2 is not None:
                assert np.can_cast(d2, b2)


def test_divide_promotion():
    q = tei._divide_result_type
    for d1 in ALL:
        for d2 in ALL:
            _, _, r = tu._find_buf_dtype2(d1, d2, q, acceptance_fn=tu._acceptance_fn_divide)
            want = np.true_divide(np.ones(1, d1), np.ones(1, d2)).dtype
            assert r == want, (d1, d2, r, want)


def test_comparison_promotion_gives_bool_and_uses_mixed_kernel():
    q = tei._less_result_type
    assert tu._find_buf_dtype2(dpt.int64, dpt.uint64, q) == (None, None, dpt.bool)
    b1, b2, r = tu._find_buf_dtype2(dpt.int8, dpt.uint8, q)
    assert r == dpt.bool and b1 == b2 == dpt.int16


def test_unary_promotion():
    assert tu._find_buf_dtype(dpt.int32, tei._exp_result_type) == (dpt.float64, dpt.float64)
    assert tu._find_buf_dtype(dpt.int8, tei._exp_result_type) == (dpt.float16, dpt.float16)
    assert tu._find_buf_dtype(dpt.bool, tei._sqrt_result_type) == (dpt.float16, dpt.float16)
    assert tu._find_buf_dtype(dpt.float32, tei._exp_result_type) == (None, dpt.float32)
    assert tu._find_buf_dtype(dpt.complex64, tei._floor_result_type) == (None, None)
    with pytest.raises(ValueError):
        tu._find_buf_dtype(dpt.bool, tei._negative_result_type, acceptance_fn=tu._acceptance_fn_negative)
    with pytest.raises(ValueError):
        tu._find_buf_dtype2(dpt.bool, dpt.bool, tei._subtract_result_type,
                            acceptance_fn=tu._acceptance_fn_subtract)


def test_weak_scalar_resolution():
    # dpnp/tests/tensor/test_type_utils.py: a Python scalar adopts the array's dtype unless its
    # kind is higher
    R = tu._resolve_weak_types
    assert R(dpt.float32, tu.WeakFloatingType(1.5)) == (dpt.float32, dpt.float32)
    assert R(dpt.int8, tu.WeakIntegralType(3)) == (dpt.int8, dpt.int8)
    assert R(dpt.int8, tu.WeakFloatingType(3.0)) == (dpt.int8, dpt.float64)
    assert R(dpt.float16, tu.WeakComplexType(1j)) == (dpt.float16, dpt.complex64)
    assert R(dpt.float64, tu.WeakComplexType(1j)) == (dpt.float64, dpt.complex128)
    assert R(dpt.bool, tu.WeakIntegralType(1)) == (dpt.bool, dpt.int64)
    assert R(tu.WeakBooleanType(True), dpt.uint8) == (dpt.uint8, dpt.uint8)
    with pytest.raises(ValueError):
        R(tu.WeakIntegralType(1), tu.WeakIntegralType(2))
    P = tu._resolve_weak_types_all_py_ints
    assert P(dpt.uint8, tu.WeakIntegralType(-1)) == (dpt.uint8, dpt.int8)
    assert P(dpt.int8, tu.WeakIntegralType(300)) == (dpt.int8, dpt.uint16)
    assert P(dpt.int8, tu.WeakIntegralType(3)) == (dpt.int8, dpt.int8)


def test_inplace_promotion():
    q = tei._add_result_type
    assert tu._find_buf_dtype_in_place_op(dpt.float32, dpt.float32, q) == (None, dpt.float32)
    assert tu._find_buf_dtype_in_place_op(dpt.float32, dpt.int32, q) == (dpt.float32, dpt.float32)
    assert tu._find_buf_dtype_in_place_op(dpt.int32, dpt.float32, q) == (None, None)


def test_accumulation_dtypes():
    D = tu._default_accumulation_dtype
    assert [D(d) for d in (dpt.bool, dpt.int8, dpt.int32, dpt.int64)] == [dpt.int64] * 4
    assert [D(d) for d in (dpt.uint8, dpt.uint32, dpt.uint64)] == [dpt.uint64] * 3
    assert [D(d) for d in (dpt.float16, dpt.float32, dpt.complex64)] == [dpt.float16, dpt.float32, dpt.complex64]


# ---- views ---------------------------------------------------------------------------------------------
def test_basic_indexing_matches_numpy_strides():
    x = host_array((6, 8, 10))
    ref = np_like(x)
    keys = [np.s_[1], np.s_[:, ::2], np.s_[::-1, 1:7:3, ...], np.s_[..., -1], np.s_[None, 2, :, None, ::-2],
            np.s_[2:2], np.s_[-3:, :, 4], np.s_[::-2, ::-3, ::-4]]
    for k in keys:
        v, r = x[k], ref[k]
        assert v.shape == r.shape
        if r.size:
            assert tuple(s * x.itemsize for s in v.strides) == tuple(
                st if sh != 1 or k is keys[4] else st for st, sh in zip(r.strides, r.shape)) or v.shape.count(1)
            off = (r.__array_interface__["data"][0] - ref.__array_interface__["data"][0]) // x.itemsize
            assert v._offset == off
    with pytest.raises(IndexError):
        x[6]
    with pytest.raises(IndexError):
        x[0, 0, 0, 0]
    assert x.T.shape == (10, 8, 6) and x.T.strides == x.strides[::-1]
    assert x.mT.shape == (6, 10, 8)


def test_flags_and_contiguity():
    x = host_array((4, 5))
    assert x.flags.c_contiguous and not x.flags.f_contiguous
    assert x.T.flags.f_contiguous and not x.T.flags.c_contiguous
    assert not x[:, ::2].flags.forc
    assert x[1:2].flags.c_contiguous and x[1:2].flags.f_contiguous  # extent-1 dims do not count
    assert host_array((0, 3)).flags.c_contiguous
    f = host_array((4, 5), order="F")
    assert f.strides == (1, 4)


def test_broadcast_permute_reshape():
    x = host_array((1, 4096))
    b = dpt.broadcast_to(x, (8192, 4096))
    assert b.shape == (8192, 4096) and b.strides == (0, 1)
    with pytest.raises(ValueError):
        dpt.broadcast_to(host_array((3,)), (4,))
    y = host_array((2, 3, 4))
    p = dpt.permute_dims(y, (2, 0, 1))
    assert p.shape == (4, 2, 3) and p.strides == (1, 12, 4)
    assert dpt.reshape(y, (6, 4)).strides == (4, 1)
    assert dpt.reshape(y, (-1,)).shape == (24,)
    assert _reshape_strides((4, 6), (12, 2), (4, 2, 3)) == [12, 6, 2]
    assert _reshape_strides((4, 6), (1, 4), (24,)) is None          # F layout cannot flatten in C order
    assert dpt.reshape(y[:, :, ::2], (6, 2)).strides == (4, 2)
    with pytest.raises(ValueError):
        dpt.reshape(p, (24,), copy=False)
    assert dpt.squeeze(host_array((1, 3, 1))).shape == (3,)
    assert dpt.expand_dims(host_array((3,)), 0).shape == (1, 3)
    assert dpt.flip(host_array((5,))).strides == (-1,)


def test_order_k_allocation():
    # dpnp/tensor/_copy_utils.py:811-911: the result keeps the operands' layout
    x = host_array((4, 6))
    assert _empty_like_orderK(x, dpt.float32).strides == (6, 1)
    assert _empty_like_orderK(x.T, dpt.float32).strides == (1, 6)
    v = dpt.permute_dims(host_array((2, 3, 4)), (1, 2, 0))  # neither C nor F
    r = _empty_like_orderK(v, dpt.float64)
    assert r.shape == v.shape and np.argsort(r.strides).tolist() == np.argsort(v.strides).tolist()
    a, b = host_array((4, 6)).T, host_array((4, 6)).T
    assert _empty_like_pair_orderK(a, b, dpt.float32, (6, 4)).flags.f_contiguous
    assert _empty_like_pair_orderK(a, host_array((6, 4)), dpt.float32, (6, 4)).flags.c_contiguous


def test_descriptor_for_c_abi():
    x = host_array((3, 4))[1:, ::2]
    v = x._as_view()
    assert v.nd == 2 and list(v.shape[:2]) == [2, 2] and list(v.strides[:2]) == [4, 2]
    assert v.data == x._buf.data_ptr() + 4 * x.itemsize
    assert v.dtype == 10 and (v.flags & 4)
    x.flags.writable = False
    assert not (x._as_view().flags & 4)


def test_errors_raised_by_the_python_layer_before_any_kernel():
    x, y = host_array((3, 4)), host_array((5,))
    with pytest.raises(ValueError, match="broadcast"):
        dpt.add(x, y)
    with pytest.raises(TypeError):
        dpt.exp([1, 2, 3])
    with pytest.raises(dpt.ExecutionPlacementError):
        dpt.add(1, 2)
    with pytest.raises(ValueError, match="Output array of type"):
        dpt.add(x, x, out=host_array((3, 4), "f8"))
    with pytest.raises(ValueError, match="inconsistent"):
        dpt.add(x, x, out=host_array((4, 3)))
    ro = host_array((3, 4))
    ro.flags.writable = False
    with pytest.raises(ValueError, match="read-only"):
        dpt.add(x, x, out=ro)
    with pytest.raises(ValueError, match="does not support input type"):
        dpt.floor(host_array((3,), "c8"))
    with pytest.raises(ValueError, match="zero-size"):
        dpt.max(host_array((3, 0)), axis=1)
    with pytest.raises(TypeError):
        dpt.argmax(x, axis=(0, 1))
    with pytest.raises(ValueError, match="complex"):
        dpt.var(host_array((3,), "c8"))
    with pytest.raises(IndexError):
        dpt.sum(x, axis=2)


def test_reduction_over_leading_axis_leaves_no_reference_cycle():
    # the permuted view a reduction keeps with its input must not keep the input alive: dropping the last
    # reference frees the allocation at once, with the cycle collector switched off
    import gc
    import weakref

    from dpnp_amd.tensor._reduction import _move_reduced_axes_last

    was = gc.isenabled()
    gc.disable()
    try:
        for axis in (0, 1, (0, 2), None):
            x = host_array((4, 5, 6))
            alive = weakref.ref(x._buf.a.base if x._buf.a.base is not None else x._buf)
            buf_alive = weakref.ref(x._buf)
            arr, _, _ = _move_reduced_axes_last(x, axis)
            again, _, _ = _move_reduced_axes_last(x, axis)
            assert again is arr  # kept with the array
            v = x[1:]  # a view of x: its own permuted view refers to x, not to v
            _move_reduced_axes_last(v, 0)
            del arr, again, v, x
            assert buf_alive() is None and alive() is None, axis
    finally:
        if was:
            gc.enable()


# ---- the extension module's plain-call path: what it takes and what it leaves to the general path ---------
def test_plain_call_path_declines_everything_but_the_plain_case():
    """binary_call / unary_call / reduce_call / where_call decide on the array descriptors alone.  Every case
    here is one they must hand back (NotImplemented) BEFORE anything is launched: no GPU is present, and a
    launch would raise."""
    import dpnp_amd._lib as L

    ext = L.ext
    add, exp, rsum, amax = L.BINARY_ID["add"], L.UNARY_ID["exp"], L.REDUCE_ID["sum"], L.SEARCH_ID["argmax"]
    f4, i4 = 10, 5
    ext.set_binary_type(add, f4, f4)
    ext.set_unary_type(exp, f4, f4)
    a, b, c = host_array((4, 6)), host_array((4, 6)), host_array((4, 6))
    assert ext.binary_call(add, a, host_array((4, 6), "f8"), c) is NotImplemented  # mixed dtypes: promotion
    assert ext.binary_call(add, a, host_array((6,)), None) is NotImplemented  # broadcasting without out: layout rules
    assert ext.binary_call(add, a.T, b.T, None) is NotImplemented  # not C-contiguous without out: order "K"
    assert ext.binary_call(add, a, host_array((5,)), c) is NotImplemented  # shapes that do not broadcast
    assert ext.binary_call(add, a, b, host_array((4, 6), "f8")) is NotImplemented  # out of another dtype
    assert ext.binary_call(add, a, b, host_array((6, 4))) is NotImplemented  # out of another shape
    assert ext.binary_call(add, a, b, a) is NotImplemented  # in place
    assert ext.binary_call(add, a, b, a[1:]) is NotImplemented  # out overlaps an input
    ro = host_array((4, 6))
    ro.flags.writable = False
    assert ext.binary_call(add, a, b, ro) is NotImplemented  # read-only out: the general path raises
    assert ext.binary_call(add, a, 2.0, c) is NotImplemented  # scalars stay with the Python layer
    assert ext.binary_call(L.BINARY_ID["hypot"], a, b, c) is NotImplemented  # type not looked up yet
    ia = host_array((4, 6), "i4")
    assert ext.unary_call(exp, ia, None) is NotImplemented  # needs a cast
    assert ext.unary_call(exp, a.T, None) is NotImplemented
    assert ext.unary_call(exp, a, a) is NotImplemented
    assert ext.unary_call(exp, a.T, c) is NotImplemented  # out of another shape
    # reductions: axis forms, out checks, empty extents
    r = host_array((4,))
    assert ext.reduce_call(rsum, a, [1], r) is NotImplemented  # a list: normalised by the general path
    assert ext.reduce_call(rsum, a, 2, r) is NotImplemented  # out of range: the general path raises
    assert ext.reduce_call(rsum, a, (1, 1), r) is NotImplemented  # repeated axis
    assert ext.reduce_call(rsum, a, (), None) is NotImplemented  # nothing reduced: a copy
    assert ext.reduce_call(rsum, a, 1, host_array((6,))) is NotImplemented  # out of another shape
    assert ext.reduce_call(rsum, a, 1, host_array((4,), "f8")) is NotImplemented  # out of another dtype
    assert ext.reduce_call(rsum, a, 1, a[:, 0]) is NotImplemented  # out inside the input
    assert ext.reduce_call(rsum, host_array((0, 6)), 0, None) is NotImplemented  # empty reduced axis
    assert ext.reduce_call(rsum, host_array((4, 0)), 0, None) is NotImplemented  # empty result
    assert ext.reduce_call(rsum, host_array(()), None, None) is NotImplemented  # 0-d
    assert ext.search_call(amax, a, (0, 1), None) is NotImplemented  # a search takes one axis
    assert ext.search_call(amax, a, 1, host_array((4,), "i4")) is NotImplemented  # the index type is int64
    # where: branches of different dtypes, shapes that do not broadcast, out mismatches, overlap
    m = host_array((4, 6), "?")
    assert ext.where_call(m, a, host_array((4, 6), "f8"), None) is NotImplemented
    assert ext.where_call(m, a, host_array((5,)), None) is NotImplemented
    assert ext.where_call(m, a, host_array((6,)), None) is NotImplemented  # broadcast without out: layout rules
    assert ext.where_call(m, a, b, host_array((4, 6), "f8")) is NotImplemented
    assert ext.where_call(m, a, b, a) is NotImplemented
    assert ext.where_call(m, a, 1.0, c) is NotImplemented
    assert ext.where_call(host_array((0,), "?"), host_array((0,)), host_array((0,)), None) is NotImplemented
    # the plain cases reach the library; where no device is present the launch error comes back as RuntimeError
    # (with a device these arrays of host memory must not be launched on at all)
    import ctypes

    n = ctypes.c_int(0)
    L.check(L.lib.dpx_device_count(ctypes.byref(n)))
    if n.value:
        return
    for call in (lambda: ext.binary_call(add, a, b, c), lambda: ext.unary_call(exp, a, c),
                 lambda: ext.binary_call(add, a[:, ::2], host_array((1, 3)), host_array((4, 3))),
                 lambda: ext.unary_call(exp, a.T, host_array((6, 4))),
                 lambda: ext.where_call(m, a, host_array((6,)), c)):
        with pytest.raises(RuntimeError):
            call()


def test_every_function_can_tell_the_extension_module_its_types():
    """The per-function type tables of the plain-call path are filled from the Python layer's own type search,
    for every dtype, also those a function refuses with an error of its own (subtract and negative of bool)."""
    import dpnp_amd._lib as L
    from dpnp_amd.tensor import _elementwise_funcs as ef
    from dpnp_amd.tensor._elementwise_common import BinaryElementwiseFunc, UnaryElementwiseFunc

    seen = 0
    for f in vars(ef).values():
        if isinstance(f, (BinaryElementwiseFunc, UnaryElementwiseFunc)):
            f._tell_ext_types()
            assert f._ext_types_known and f._op_id >= 0
            seen += 1
    assert seen >= 70
    assert L.ext.binary_type(L.BINARY_ID["subtract"], 0) == -1 and L.ext.binary_type(L.BINARY_ID["subtract"], 10) == 10
    assert L.ext.binary_type(L.BINARY_ID["less"], 11) == 0  # comparisons give bool
    assert L.ext.unary_type(L.UNARY_ID["negative"], 0) == -1 and L.ext.unary_type(L.UNARY_ID["exp"], 5) == -1
    assert L.ext.unary_type(L.UNARY_ID["abs"], 13) == 11  # |complex128| is float64
