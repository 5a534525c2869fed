"""Differential tests over seeded random cases: dtype, function, shape, memory layout of every operand (permuted
axes, steps of 1, 2, 3, -1, -2, offsets, broadcast dims) and of `out`, for the elementwise functions with exact
results and for the reductions.  Each case is checked against NumPy on host views with the same layout.  The kernel
families a case lands in (contiguous, rows, tile, flat, columns, short rows, generic ...) follow from the layout,
so the seeds walk through all of them; a failure message names the seed and the case."""
import numpy as np
import pytest

import dpnp_amd.tensor as dpt
from dpnp_amd.tensor._usmarray import usm_ndarray
from tests.helpers import dev, host, random_array

pytestmark = pytest.mark.gpu

INTS = ["i1", "u1", "i2", "u2", "i4", "u4", "i8", "u8"]
REAL = INTS + ["f2", "f4", "f8"]
ALL = ["?"] + REAL + ["c8", "c16"]


def random_view(rng, shape, dtype, allow_broadcast=True):
    """-> (host base, host view of `shape`): the view walks the base with random axis order, steps and offset."""
    nd = len(shape)
    perm = rng.permutation(nd) if nd else np.array([], dtype=int)
    steps = [int(rng.choice([1, 1, 1, 2, 3, -1, -2])) for _ in range(nd)]
    bcast = [allow_broadcast and shape[d] > 1 and rng.random() < 0.12 for d in range(nd)]
    lead = [int(rng.integers(0, 3)) for _ in range(nd)]
    # extents of the base along the view's axes
    ext = [1 if bcast[d] else lead[d] + abs(steps[d]) * (shape[d] - 1) + 1 + int(rng.integers(0, 2)) for d in range(nd)]
    base_shape = tuple(ext[int(p)] for p in perm)
    base = random_array(rng, base_shape, dtype) if base_shape else random_array(rng, (), dtype)
    v = np.transpose(base, np.argsort(perm)) if nd else base  # axis d of v is axis of extent ext[d]
    idx = []
    for d in range(nd):
        if bcast[d]:
            idx.append(slice(None))
        elif steps[d] > 0:
            idx.append(slice(lead[d], lead[d] + steps[d] * (shape[d] - 1) + 1, steps[d]))
        else:
            start = lead[d] + (-steps[d]) * (shape[d] - 1)
            stop = lead[d] - 1
            idx.append(slice(start, stop if stop >= 0 else None, steps[d]))
    v = v[tuple(idx)]
    if any(bcast):
        v = np.broadcast_to(v, shape)
    assert v.shape == tuple(shape), (v.shape, shape)
    return base, v


def device_view(base, view, with_base=False):
    """Device array laid out inside a device copy of `base` as `view` is inside `base`."""
    d = dev(np.ascontiguousarray(base))
    off = (view.__array_interface__["data"][0] - base.__array_interface__["data"][0]) // base.itemsize
    v = usm_ndarray(view.shape, dtype=view.dtype, buffer=d, offset=d._offset + off,
                    strides=[s // base.itemsize for s in view.strides])
    return (v, d) if with_base else v


def random_shape(rng):
    kind = rng.integers(0, 6)
    if kind == 0:
        return tuple(int(s) for s in rng.integers(1, 7, int(rng.integers(1, 6))))
    if kind == 1:
        return (int(rng.integers(1, 5000)),)
    if kind == 2:
        return (int(rng.integers(1, 200)), int(rng.integers(1, 200)))
    if kind == 3:
        return (int(rng.integers(500, 3000)), int(rng.integers(1, 40)))
    if kind == 4:
        return (int(rng.integers(1, 40)), int(rng.integers(500, 3000)))
    return (int(rng.integers(1, 12)), int(rng.integers(1, 70)), int(rng.integers(1, 70)))


BINARY = {
    "add": (np.add, ALL), "subtract": (np.subtract, REAL + ["c8", "c16"]), "multiply": (np.multiply, ["?"] + REAL),
    "maximum": (np.maximum, ["?"] + REAL), "minimum": (np.minimum, ["?"] + REAL),
    "bitwise_and": (np.bitwise_and, ["?"] + INTS), "bitwise_or": (np.bitwise_or, ["?"] + INTS),
    "bitwise_xor": (np.bitwise_xor, ["?"] + INTS), "equal": (np.equal, ALL), "not_equal": (np.not_equal, ALL),
    "less": (np.less, ["?"] + REAL), "greater_equal": (np.greater_equal, ["?"] + REAL),
    "logical_and": (np.logical_and, ALL), "logical_xor": (np.logical_xor, ALL),
    "copysign": (np.copysign, ["f2", "f4", "f8"]),
}
UNARY = {
    "negative": (np.negative, REAL + ["c8", "c16"]), "abs": (np.abs, ["?"] + REAL), "square": (np.square, INTS + ["f4", "f8"]),
    "sign": (np.sign, ["i1", "i2", "i4", "i8", "f2", "f4", "f8"]), "isnan": (np.isnan, ALL), "isfinite": (np.isfinite, ALL),
    "logical_not": (np.logical_not, ALL), "bitwise_invert": (np.invert, ["?"] + INTS), "signbit": (np.signbit, ["f2", "f4", "f8"]),
    "floor": (np.floor, ["f2", "f4", "f8"]), "trunc": (np.trunc, ["f2", "f4", "f8"]),
    "conj": (np.conj, ["c8", "c16"]), "real": (np.real, ["c8", "c16"]), "imag": (np.imag, ["c8", "c16"]),
    "positive": (np.positive, REAL + ["c8", "c16"]),
}


@pytest.mark.parametrize("seed", range(12))
def test_random_binary_calls_and_out_layouts(seed):
    rng = np.random.default_rng(1000 + seed)
    names = list(BINARY)
    for case in range(40):
        name = names[int(rng.integers(len(names)))]
        np_fn, dts = BINARY[name]
        dt = dts[int(rng.integers(len(dts)))]
        shape = random_shape(rng)
        what = f"seed {seed} case {case}: {name} {dt} {shape}"
        base_a, va = random_view(rng, shape, dt)
        base_b, vb = random_view(rng, shape, dt)
        with np.errstate(all="ignore"):
            want = np_fn(va, vb)
        a, b = device_view(base_a, va), device_view(base_b, vb)
        got = getattr(dpt, name)(a, b)
        assert got.dtype == want.dtype and got.shape == want.shape, what
        np.testing.assert_array_equal(host(got), want, err_msg=what)
        # into an `out` with a layout of its own; the elements around it stay as they were
        base_o, vo = random_view(rng, shape, want.dtype, allow_broadcast=False)
        o, o_base = device_view(base_o, vo, with_base=True)
        res = getattr(dpt, name)(a, b, out=o)
        assert res is o, what
        vo[...] = want
        np.testing.assert_array_equal(host(o_base), base_o, err_msg=what + " (out and the elements around it)")


@pytest.mark.parametrize("seed", range(8))
def test_random_unary_calls_where_and_casts(seed):
    rng = np.random.default_rng(2000 + seed)
    names = list(UNARY)
    for case in range(40):
        name = names[int(rng.integers(len(names)))]
        np_fn, dts = UNARY[name]
        dt = dts[int(rng.integers(len(dts)))]
        shape = random_shape(rng)
        what = f"seed {seed} case {case}: {name} {dt} {shape}"
        base_a, va = random_view(rng, shape, dt)
        with np.errstate(all="ignore"):
            want = np_fn(va)
        a = device_view(base_a, va)
        got = getattr(dpt, name)(a)
        assert got.dtype == want.dtype and got.shape == want.shape, what
        np.testing.assert_array_equal(host(got), want, err_msg=what)
        # where(cond, a, b) with a condition of any dtype and layout
        cdt = ALL[int(rng.integers(len(ALL)))]
        base_c, vc = random_view(rng, shape, cdt)
        base_b, vb = random_view(rng, shape, dt)
        got = dpt.where(device_view(base_c, vc), a, device_view(base_b, vb))
        np.testing.assert_array_equal(host(got), np.where(vc, va, vb), err_msg=what + f" where({cdt})")
        # cast to a random other type (same-kind or wider, values in range of every type)
        to = ALL[int(rng.integers(len(ALL)))]
        if np.can_cast(dt, to, casting="same_kind") or (np.dtype(dt).kind in "biu" and np.dtype(to).kind in "iufc"):
            small = np.abs(va) if np.dtype(to).kind == "u" and np.dtype(dt).kind != "c" else va
            base_s = np.ascontiguousarray(small)
            with np.errstate(all="ignore"):
                want = base_s.astype(to)
            got = dpt.astype(dev(base_s), to)
            np.testing.assert_array_equal(host(got), want, err_msg=what + f" astype({to})")


def reduce_axes(rng, nd):
    if nd == 0 or rng.random() < 0.25:
        return None
    k = int(rng.integers(1, nd + 1))
    axes = tuple(sorted(int(a) for a in rng.choice(nd, k, replace=False)))
    return axes[0] if len(axes) == 1 and rng.random() < 0.5 else axes


@pytest.mark.parametrize("seed", range(12))
def test_random_reductions_over_random_layouts(seed):
    rng = np.random.default_rng(3000 + seed)
    for case in range(30):
        shape = random_shape(rng)
        axis = reduce_axes(rng, len(shape))
        keepdims = bool(rng.random() < 0.3)
        dt = ALL[int(rng.integers(len(ALL)))]
        what = f"seed {seed} case {case}: {dt} {shape} axis={axis} keepdims={keepdims}"
        base, v = random_view(rng, shape, dt, allow_broadcast=False)
        a = device_view(base, v)
        # integer sums and products wrap as NumPy's do; floating ones are compared with a float64 result
        for name in ("sum", "prod"):
            got = getattr(dpt, name)(a, axis=axis, keepdims=keepdims)
            kind = np.dtype(dt).kind
            if kind in "biu":
                small = (v % 3).astype(dt) if name == "prod" else v
                if name == "prod":
                    got = dpt.prod(dev(np.ascontiguousarray(small)), axis=axis, keepdims=keepdims)
                want = getattr(np, name)(small, axis=axis, keepdims=keepdims, dtype=got.dtype)
                np.testing.assert_array_equal(host(got), want, err_msg=what + " " + name)
            elif name == "sum":
                wide = v.astype("c16" if kind == "c" else "f8")
                want = np.sum(wide, axis=axis, keepdims=keepdims)
                scale = np.sum(np.abs(wide), axis=axis, keepdims=keepdims)
                eps = float(np.finfo(dt).eps)
                tol = 2e-3 if eps > 1e-4 else (1e-5 if eps > 1e-10 else 1e-12)
                assert got.dtype == np.dtype(dt) and got.shape == want.shape, what
                err = np.abs(host(got).astype(wide.dtype) - want)
                in_range = np.abs(want) < 3e4 if dt == "f2" else np.ones(want.shape, dtype=bool)  # float16 overflows above
                assert (err <= tol * np.maximum(scale, 1e-30))[in_range].all(), what + " sum"
        if np.dtype(dt).kind != "c" and v.size:
            for name in ("max", "min"):
                got = getattr(dpt, name)(a, axis=axis, keepdims=keepdims)
                np.testing.assert_array_equal(host(got), getattr(np, name)(v, axis=axis, keepdims=keepdims),
                                              err_msg=what + " " + name)
            if axis is None or isinstance(axis, int):
                for name in ("argmax", "argmin"):
                    got = getattr(dpt, name)(a, axis=axis, keepdims=keepdims)
                    np.testing.assert_array_equal(host(got), getattr(np, name)(v, axis=axis, keepdims=keepdims),
                                                  err_msg=what + " " + name)
        for name in ("any", "all", "count_nonzero"):
            got = getattr(dpt, name)(a, axis=axis, keepdims=keepdims)
            np.testing.assert_array_equal(host(got), getattr(np, name)(v, axis=axis, keepdims=keepdims),
                                          err_msg=what + " " + name)
        # into a strided `out`
        want = np.max(v, axis=axis, keepdims=keepdims) if np.dtype(dt).kind != "c" and v.size else None
        if want is not None and want.ndim:
            base_o, vo = random_view(rng, want.shape, dt, allow_broadcast=False)
            o, o_base = device_view(base_o, vo, with_base=True)
            res = dpt.max(a, axis=axis, keepdims=keepdims, out=o)
            assert res.usm_data is o.usm_data and res.shape == o.shape, what
            vo[...] = want
            np.testing.assert_array_equal(host(o_base), base_o, err_msg=what + " max(out and the elements around it)")
