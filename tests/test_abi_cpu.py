"""The C-ABI library without a GPU: it loads, exports what the header declares, answers the
dtype queries, collapses strides, plans launches and rejects bad calls before launching."""
import ctypes
import os
import re

import numpy as np
import pytest

import dpnp_amd._lib as L
from oracle import oracle as orc
from tests.test_oracle import random_view_strides

lib = L.lib
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
NP = [np.dtype(c) for c in ("?", "i1", "u1", "i2", "u2", "i4", "u4", "i8", "u8", "f2", "f4", "f8", "c8", "c16")]
FAKE = 0x7F0000000000  # never dereferenced: plans and failed validations do not touch memory
P0, P1, P2 = FAKE, FAKE + (1 << 36), FAKE + (2 << 36)  # three disjoint "allocations"


def view(shape, strides=None, dt=L.FLOAT, ptr=FAKE, writable=True):
    shape = list(shape)
    if strides is None:
        strides, acc = [0] * len(shape), 1
        for d in range(len(shape) - 1, -1, -1):
            strides[d] = acc
            acc *= max(shape[d], 1)
    return L.make_view(ptr, shape, list(strides), dt, L.WRITABLE if writable else 0)


def test_header_symbols_are_exported():
    text = open(os.path.join(ROOT, "include", "dpnp_amd.h")).read()
    declared = set(re.findall(r"\b(dpx_[a-z0-9_]+)\s*\(", text))
    assert declared, "no declarations found"
    assert declared == set(L.SIGNATURES), declared ^ set(L.SIGNATURES)
    for name in declared:
        assert hasattr(lib, name)
    assert lib.dpx_abi_version() == 1
    assert [lib.dpx_dtype_itemsize(i) for i in range(14)] == [d.itemsize for d in NP]


def test_op_tables_match_header_enums():
    text = open(os.path.join(ROOT, "include", "dpnp_amd.h")).read()
    for prefix, names in (("DPX_U_", L.UNARY_OPS), ("DPX_B_", L.BINARY_OPS), ("DPX_R_", L.REDUCE_OPS)):
        body = re.search(r"typedef enum dpx_%s_op \{(.*?)\}" % {"DPX_U_": "unary", "DPX_B_": "binary",
                                                                "DPX_R_": "reduce"}[prefix], text, re.S).group(1)
        body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
        ids = [m for m in re.findall(prefix + r"([A-Z0-9_]+)", body) if m != "NUM_OPS"]
        want = [n.upper().replace("BITWISE_LEFT_SHIFT", "LEFT_SHIFT").replace("BITWISE_RIGHT_SHIFT", "RIGHT_SHIFT")
                for n in names]
        assert ids == want


def test_binary_result_types():
    B = L.BINARY_ID
    for i, d in enumerate(NP):
        assert lib.dpx_binary_result_type(B["add"], i, i) == i
        assert lib.dpx_binary_result_type(B["multiply"], i, i) == i
        assert lib.dpx_binary_result_type(B["subtract"], i, i) == (-1 if d.kind == "b" else i)
        assert lib.dpx_binary_result_type(B["divide"], i, i) == (i if d.kind in "fc" else -1)
        assert lib.dpx_binary_result_type(B["bitwise_and"], i, i) == (i if d.kind in "biu" else -1)
        assert lib.dpx_binary_result_type(B["greater"], i, i) == L.BOOL
        assert lib.dpx_binary_result_type(B["maximum"], i, i) == i
    # only same-dtype pairs, except int64/uint64 comparisons
    assert lib.dpx_binary_result_type(B["add"], L.FLOAT, L.DOUBLE) == -1
    # pairs whose conversion is folded into the kernel are reported separately
    assert lib.dpx_binary_fused_cast_result_type(B["add"], L.FLOAT, L.DOUBLE) == L.DOUBLE
    assert lib.dpx_binary_fused_cast_result_type(B["divide"], L.INT32, L.DOUBLE) == L.DOUBLE
    assert lib.dpx_binary_fused_cast_result_type(B["multiply"], L.FLOAT, L.BOOL) == L.FLOAT
    assert lib.dpx_binary_fused_cast_result_type(B["maximum"], L.FLOAT, L.DOUBLE) == -1
    assert lib.dpx_binary_fused_cast_result_type(B["add"], L.FLOAT, L.INT32) == L.DOUBLE  # both operands converted
    assert lib.dpx_binary_fused_cast_result_type(B["subtract"], L.INT64, L.FLOAT) == L.DOUBLE
    assert lib.dpx_binary_fused_cast_result_type(B["multiply"], L.INT16, L.FLOAT) == L.FLOAT
    assert lib.dpx_binary_fused_cast_result_type(B["add"], L.FLOAT, L.UINT16) == -1
    assert lib.dpx_binary_fused_cast_result_type(B["add"], L.INT32, L.INT64) == -1
    assert lib.dpx_binary_fused_cast_result_type(B["add"], L.FLOAT, L.FLOAT) == -1
    assert lib.dpx_binary_result_type(B["less"], L.INT64, L.UINT64) == L.BOOL
    assert lib.dpx_binary_result_type(B["less"], L.UINT64, L.INT64) == L.BOOL
    assert lib.dpx_binary_result_type(B["less"], L.INT32, L.UINT32) == -1
    assert lib.dpx_binary_inplace_supported(B["add"], L.FLOAT, L.FLOAT) == 1
    assert lib.dpx_binary_inplace_supported(B["greater"], L.FLOAT, L.FLOAT) == 0


def test_unary_result_types():
    U = L.UNARY_ID
    for i, d in enumerate(NP):
        assert lib.dpx_unary_result_type(U["exp"], i) == (i if d.kind in "fc" else -1)
        assert lib.dpx_unary_result_type(U["sqrt"], i) == (i if d.kind in "fc" else -1)
        assert lib.dpx_unary_result_type(U["cbrt"], i) == (i if d.kind == "f" else -1)
        assert lib.dpx_unary_result_type(U["real"], i) == {L.CFLOAT: L.FLOAT, L.CDOUBLE: L.DOUBLE}.get(i, i)
        assert lib.dpx_unary_result_type(U["angle"], i) == {L.CFLOAT: L.FLOAT, L.CDOUBLE: L.DOUBLE}.get(i, -1)
        assert lib.dpx_unary_result_type(U["round"], i) == (-1 if d.kind == "b" else i)
        assert lib.dpx_unary_result_type(U["isnan"], i) == L.BOOL
        want_abs = {L.CFLOAT: L.FLOAT, L.CDOUBLE: L.DOUBLE}.get(i, i)
        assert lib.dpx_unary_result_type(U["abs"], i) == want_abs
        assert lib.dpx_unary_result_type(U["negative"], i) == (-1 if d.kind == "b" else i)
        assert lib.dpx_unary_result_type(U["square"], i) == (L.INT8 if d.kind == "b" else i)
    assert lib.dpx_unary_result_type(U["erf"], L.HALF) == L.FLOAT
    assert lib.dpx_unary_result_type(U["erf"], L.DOUBLE) == L.DOUBLE


def test_reduction_dtype_support():
    R = L.REDUCE_ID
    for i, d in enumerate(NP):
        assert lib.dpx_reduce_dtype_supported(R["sum"], i, i) == 1
        dflt = orc.default_accumulation_dtype(d)
        assert lib.dpx_reduce_dtype_supported(R["sum"], i, NP.index(dflt)) == 1
        assert lib.dpx_reduce_dtype_supported(R["max"], i, i) == 1
        assert lib.dpx_search_dtype_supported(0, i, L.INT64) == 1
        assert lib.dpx_search_dtype_supported(0, i, L.INT32) == 0
    # every (input, result) pair of the reference's sum / prod tables has a kernel of its own
    import json
    import os

    gold = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_known_answers.json")))
    names = [d.str[1:] if d.kind != "b" else "?" for d in NP]
    pairs = gold["sum_prod_type_pairs"]["pairs"]
    assert sorted(pairs) == sorted(names)
    for src, outs in pairs.items():
        for dst in outs:
            assert lib.dpx_reduce_dtype_supported(R["sum"], names.index(src), names.index(dst)) == 1, (src, dst)
            assert lib.dpx_reduce_dtype_supported(R["prod"], names.index(src), names.index(dst)) == 1, (src, dst)
    assert lib.dpx_reduce_dtype_supported(R["sum"], L.FLOAT, L.DOUBLE) == 1
    assert lib.dpx_reduce_dtype_supported(R["sum"], L.DOUBLE, L.FLOAT) == 0
    assert lib.dpx_reduce_dtype_supported(R["max"], L.FLOAT, L.DOUBLE) == 0
    assert lib.dpx_reduce_dtype_supported(R["sumsqdev"], L.FLOAT, L.DOUBLE) == 1
    assert lib.dpx_reduce_dtype_supported(R["sumsqdev"], L.INT32, L.DOUBLE) == 1   # var of an integer array
    assert lib.dpx_reduce_dtype_supported(R["sumsqdev"], L.INT32, L.FLOAT) == 0
    assert lib.dpx_reduce_dtype_supported(R["sum"], L.INT32, L.DOUBLE) == 1        # mean of an integer array
    assert lib.dpx_reduce_dtype_supported(R["sum"], L.DOUBLE, L.INT32) == 0


def c_collapse(shape, strides_list, keep_order=False):
    nd, nops = len(shape), len(strides_list)
    sh = (ctypes.c_int64 * L.MAX_ND)(*shape)
    st = (ctypes.c_int64 * (L.MAX_ND * nops))()
    for k, s in enumerate(strides_list):
        for d, v in enumerate(s):
            st[k * L.MAX_ND + d] = v
    off = (ctypes.c_int64 * nops)()
    n = lib.dpx_collapse(nd, nops, sh, st, off, 1 if keep_order else 0)
    return list(sh[:n]), [[st[k * L.MAX_ND + d] for d in range(n)] for k in range(nops)], list(off)


def test_collapse_matches_brute_force_and_oracle():
    rng = np.random.default_rng(3)
    for _ in range(400):
        nd = int(rng.integers(1, 6))
        shape = [int(s) for s in rng.integers(1, 5, nd)]
        strides = [random_view_strides(rng, shape) for _k in range(int(rng.integers(1, 5)))]
        for keep in (False, True):
            sh, st, off = c_collapse(shape, strides, keep)
            assert orc.address_tuples(sh, st, off) == orc.address_tuples(shape, strides)
            osh, ost, ooff = orc.collapse(shape, strides, keep)
            assert len(sh) == len(osh)  # both reach the same number of dims


def test_collapse_examples():
    assert c_collapse([3, 4, 5], [[20, 5, 1], [20, 5, 1]]) == ([60], [[1], [1]], [0, 0])
    assert c_collapse([3, 4], [[-4, -1]]) == ([12], [[1]], [-11])
    assert c_collapse([8192, 8192], [[1, 8192], [1, 8192]]) == ([8192 * 8192], [[1], [1]], [0, 0])  # F-contig pair
    sh, st, _ = c_collapse([8192, 4096], [[8192, 2], [0, 1], [4096, 1]])
    assert sh == [8192, 4096] and st == [[8192, 2], [0, 1], [4096, 1]]
    assert c_collapse([3, 4], [[1, 3]], keep_order=True)[0] == [3, 4]


def plan_binary(op, a, b, o):
    p = L.Plan()
    L.check(lib.dpx_binary_plan(L.BINARY_ID[op], a, b, o, p))
    return p


def test_elementwise_plans():
    n = 1 << 20
    p = plan_binary("add", view([n]), view([n], ptr=P1), view([n], ptr=P2))
    assert L.PATH_NAMES[p.path] == "ew_contig" and p.vec == 4 and p.block == 64 and p.grid[0] == n // (64 * 4)
    # array (+) scalar: zero-stride operand still takes the contiguous kernel
    p = plan_binary("add", view([n]), view([n], [0], ptr=P1), view([n], ptr=P2))
    assert L.PATH_NAMES[p.path] == "ew_contig"
    # F-contiguous triple collapses to 1-D
    p = plan_binary("add", view([64, 32], [1, 64]), view([64, 32], [1, 64]), view([64, 32], [1, 64]))
    assert L.PATH_NAMES[p.path] == "ew_contig" and p.nd == 1
    # reversed views collapse too
    p = plan_binary("add", view([100], [-1], ptr=P0 + 396), view([100], [-1], ptr=P1 + 396),
                    view([100], [-1], ptr=P2 + 396))
    assert L.PATH_NAMES[p.path] == "ew_contig" and list(p.offsets[:3]) == [-99, -99, -99]
    # config 4: strided x broadcast row
    p = plan_binary("multiply", view([8192, 4096], [8192, 2]), view([8192, 4096], [0, 1], ptr=P1),
                    view([8192, 4096], ptr=P2))
    assert L.PATH_NAMES[p.path] == "ew_rows2" and p.nd == 2 and list(p.shape[:2]) == [8192, 4096]
    # the same with an odd number of rows, or rows that are no multiple of a wave's 256 floats: the general kernel
    p = plan_binary("multiply", view([8191, 4096], [8192, 2]), view([8191, 4096], [0, 1], ptr=P1),
                    view([8191, 4096], ptr=P2))
    assert L.PATH_NAMES[p.path] == "ew_rows"
    p = plan_binary("multiply", view([8192, 4000], [8192, 2]), view([8192, 4000], [0, 1], ptr=P1),
                    view([8192, 4000], ptr=P2))
    assert L.PATH_NAMES[p.path] == "ew_rows"
    # a 1-D stride-2 view is cut into rows for the same kernel
    p = plan_binary("add", view([1 << 20], [2]), view([1 << 20], [2], ptr=P1), view([1 << 20], ptr=P2))
    assert L.PATH_NAMES[p.path] == "ew_rows2" and p.nd == 2
    # a matrix with short rows and a row / a column: the contiguous kernel walks it flat
    p = plan_binary("subtract", view([100000, 17]), view([100000, 17], [0, 1], ptr=P1), view([100000, 17], ptr=P2))
    assert L.PATH_NAMES[p.path] == "ew_contig" and p.nd == 2 and p.grid[0] == -(-100000 * 17 // 256)
    p = plan_binary("divide", view([100000, 17]), view([100000, 17], [1, 0], ptr=P1), view([100000, 17], ptr=P2))
    assert L.PATH_NAMES[p.path] == "ew_contig"
    p = plan_binary("subtract", view([100000, 128]), view([100000, 128], [0, 1], ptr=P1), view([100000, 128], ptr=P2))
    assert L.PATH_NAMES[p.path] == "ew_rows"  # 512-byte rows
    p = plan_binary("subtract", view([100000, 17], [34, 2]), view([100000, 17], [0, 1], ptr=P1), view([100000, 17], ptr=P2))
    assert L.PATH_NAMES[p.path] == "ew_rows"  # strided matrix
    # rows of 2 MiB and more plus a row: flat as well; plus a column: the row kernel (one value per row there)
    n = 600001
    p = plan_binary("add", view([5, n]), view([5, n], [0, 1], ptr=P1), view([5, n], ptr=P2))
    assert L.PATH_NAMES[p.path] == "ew_contig" and p.nd == 2
    p = plan_binary("add", view([5, n]), view([5, n], [1, 0], ptr=P1), view([5, n], ptr=P2))
    assert L.PATH_NAMES[p.path] == "ew_rows"
    p = plan_binary("add", view([5, 100000]), view([5, 100000], [0, 1], ptr=P1), view([5, 100000], ptr=P2))
    assert L.PATH_NAMES[p.path] == "ew_rows"  # 400 KB rows
    # one full-size input and the output in aligned packs, the other input broadcast: one-wave blocks; an outer
    # sum (nothing full-size is read), two full-size inputs, rows off the 16-byte grid: four waves per block
    p = plan_binary("add", view([16384, 16384]), view([16384, 16384], [0, 1], ptr=P1), view([16384, 16384], ptr=P2))
    assert L.PATH_NAMES[p.path] == "ew_rows" and p.block == 64 and p.grid[0] == 16384 * 64
    p = plan_binary("multiply", view([16384, 16384]), view([16384, 16384], [1, 0], ptr=P1), view([16384, 16384], ptr=P2))
    assert L.PATH_NAMES[p.path] == "ew_rows" and p.block == 64
    p = plan_binary("add", view([16384, 16384], [0, 1]), view([16384, 16384], [1, 0], ptr=P1), view([16384, 16384], ptr=P2))
    assert L.PATH_NAMES[p.path] == "ew_rows" and p.block == 256
    p = plan_binary("add", view([16384, 8192], [16384, 1]), view([16384, 8192], [16384, 1], ptr=P1),
                    view([16384, 8192], [16384, 1], ptr=P2))
    assert L.PATH_NAMES[p.path] == "ew_rows" and p.block == 256
    p = plan_binary("add", view([16384, 16383]), view([16384, 16383], [0, 1], ptr=P1), view([16384, 16383], ptr=P2))
    assert L.PATH_NAMES[p.path] == "ew_rows" and p.block == 256
    # a row plus a column (nothing of the output's size is read): blocks of 8 rows x 256 packs
    p = plan_binary("add", view([16384, 16384], [0, 1]), view([16384, 16384], [1, 0], ptr=P1), view([16384, 16384], ptr=P2))
    assert L.PATH_NAMES[p.path] == "ew_rows" and p.block == 256 and p.grid[0] == (16384 // 8) * (16384 // 1024)
    # ... X[:, None, :] - Y[None, :, :] as well; a full-size operand keeps the general kernel's one row per thread
    p = plan_binary("subtract", view([64, 512, 1024], [1024, 0, 1]), view([64, 512, 1024], [0, 1024, 1], ptr=P1),
                    view([64, 512, 1024], ptr=P2))
    assert p.block == 256 and p.grid[0] == 64 * (512 // 8)
    p = plan_binary("add", view([16384, 16384]), view([16384, 16384], [1, 0], ptr=P1), view([16384, 16384], ptr=P2))
    assert p.grid[0] == 16384 * 16384 // 4 // p.block
    # empty
    p = plan_binary("add", view([0, 3]), view([0, 3]), view([0, 3]))
    assert L.PATH_NAMES[p.path] == "noop"


def plan_reduce(op, src, trailing, dst):
    p = L.Plan()
    L.check(lib.dpx_reduce_plan(L.REDUCE_ID[op], src, trailing, dst, p))
    return p


def test_reduction_plans():
    p = plan_reduce("sum", view([1 << 28]), 1, view([], ptr=P1))
    assert L.PATH_NAMES[p.path] == "red_rows_split" and p.splits > 1 and p.vec == 1
    assert p.scratch_bytes == 131072 + 4 * p.splits  # ticket counters (outputs + groups) + one float partial per block
    p = plan_reduce("sum", view([16384, 16384]), 1, view([16384], ptr=P1))
    assert L.PATH_NAMES[p.path] == "red_rows" and p.splits == 1 and p.grid[0] == 16384
    # axis=0 of a C-contiguous matrix: the caller passes the transposed view
    p = plan_reduce("sum", view([16384, 16384], [1, 16384]), 1, view([16384], ptr=P1))
    assert L.PATH_NAMES[p.path] == "red_cols_split" and p.vec == 1
    # rows of at most 256 bytes, one result per row: whole rows staged in LDS (32 KiB of padded rows per block)
    p = plan_reduce("sum", view([1 << 20, 4]), 1, view([1 << 20], ptr=P1))
    assert L.PATH_NAMES[p.path] == "red_short_rows" and p.block == 256 and p.grid[0] == -(-(1 << 20) // (32768 // 20))
    p = plan_reduce("max", view([1 << 20, 64]), 1, view([1 << 20], ptr=P1))
    assert L.PATH_NAMES[p.path] == "red_short_rows" and p.grid[0] == -(-(1 << 20) // (32768 // (65 * 4)))
    p = plan_reduce("sum", view([1 << 20, 65]), 1, view([1 << 20], ptr=P1))
    assert L.PATH_NAMES[p.path] in ("red_small", "red_rows")
    p = plan_reduce("sum", view([1 << 20, 4], [8, 1]), 1, view([1 << 20], ptr=P1))  # padded rows
    assert L.PATH_NAMES[p.path] in ("red_small", "red_rows")
    # reduce a middle axis of (a, r, c): outputs contiguous along c
    p = plan_reduce("max", view([8, 64, 1000], [64000, 1, 64]), 1, view([8, 64], ptr=P1))
    assert L.PATH_NAMES[p.path] in ("red_rows", "red_small", "red_generic", "red_cols", "red_cols_split")
    p = plan_reduce("sum", view([5, 0]), 1, view([5], ptr=P1))
    assert L.PATH_NAMES[p.path] == "red_small" and p.splits == 1  # identity fill
    pa = L.Plan()
    L.check(lib.dpx_argreduce_plan(0, view([1 << 28]), 1, view([], dt=L.INT64, ptr=P1), pa))
    assert L.PATH_NAMES[pa.path] == "red_rows_split"
    # axis=0 of a row-major matrix with short rows: flat stream, block size a multiple of the column period
    for cols, threads in ((17, 255), (64, 256), (3, 255), (10, 255), (100, 250), (127, 254)):
        p = plan_reduce("sum", view([cols, 1 << 20], [1, cols]), 1, view([cols], ptr=P1))
        assert L.PATH_NAMES[p.path] == "red_flat" and p.block == threads and p.splits == p.grid[0] > 1, (cols, p.block)
        assert p.scratch_bytes == 131072 + 4 * p.splits * cols
    p = plan_reduce("sum", view([17, 100], [1, 17]), 1, view([17], ptr=P1))
    assert L.PATH_NAMES[p.path] == "red_flat" and p.splits == 1 and p.scratch_bytes == 0
    p = plan_reduce("sum", view([128, 1 << 20], [1, 128]), 1, view([128], ptr=P1))  # 512-byte rows: column kernel
    assert L.PATH_NAMES[p.path] == "red_cols_split"
    p = plan_reduce("sum", view([17, 1 << 20], [1, 18]), 1, view([17], ptr=P1))  # padded rows: column kernel
    assert L.PATH_NAMES[p.path] == "red_cols_split"
    # reduced dims that do not collapse into one run.  A sliced matrix summed whole, axes (0, 2) of a 3-d array:
    # lanes along the reduced space, packs along its unit-stride last dim
    p = plan_reduce("sum", view([16384, 16382], [16384, 1]), 2, view([], ptr=P1))
    assert L.PATH_NAMES[p.path] == "red_generic" and p.red_nd == 2 and p.vec == 1 and p.splits > 1
    p = plan_reduce("max", view([1024, 256, 1024], [1024, 1 << 20, 1]), 2, view([1024], ptr=P1))
    assert L.PATH_NAMES[p.path] == "red_generic" and p.red_nd == 2 and p.vec == 1 and p.grid[0] == 1024
    # (512 to 4096 outputs: lanes per output for as many waves as a split plan runs, not a whole 256-thread block)
    assert p.block == 128
    p = plan_reduce("sum", view([2048, 128, 1024], [1024, 1 << 21, 1]), 2, view([2048], ptr=P1))
    assert p.grid[0] == 512 and p.block == 256  # a wave per output
    p = plan_reduce("sum", view([512, 512, 1024], [1024, 1 << 19, 1]), 2, view([512], ptr=P1))
    assert p.grid[0] == 512 and p.block == 256 and p.splits == 1  # a block per output
    # every other column summed along the rows: the lines the run touches are read as packs; every third: single
    # elements at a stride
    p = plan_reduce("sum", view([16384, 8192], [16384, 2]), 1, view([16384], ptr=P1))
    assert L.PATH_NAMES[p.path] == "red_generic" and p.red_nd == 1 and p.vec == 1
    p = plan_reduce("sum", view([16384, 5000], [16384, 3]), 1, view([16384], ptr=P1))
    assert L.PATH_NAMES[p.path] == "red_generic" and p.red_nd == 1 and p.vec == 0
    # axes (0, 2) of a 4-d array, every other column summed down the columns: src moves least along the inner
    # iteration dim, so threads sit side by side along it and walk the rows of the reduced space
    p = plan_reduce("sum", view([128, 128, 128, 128], [1 << 14, 1, 1 << 21, 128]), 2, view([128, 128], ptr=P1))
    assert L.PATH_NAMES[p.path] in ("red_cols", "red_cols_split") and p.red_nd == 2 and p.vec == 1
    p = plan_reduce("sum", view([8192, 16384], [2, 16384]), 1, view([8192], ptr=P1))
    assert L.PATH_NAMES[p.path] in ("red_cols", "red_cols_split") and p.red_nd == 1 and p.vec == 1  # whole lines
    p = plan_reduce("sum", view([5000, 16384], [3, 16384]), 1, view([5000], ptr=P1))
    assert L.PATH_NAMES[p.path] in ("red_cols", "red_cols_split") and p.red_nd == 1 and p.vec == 0
    # variance in one pass: contiguous reduced runs and columns (short rows stay with the plain row and column
    # kernels, whose lanes know the reference the means are kept relative to); other layouts are refused
    op = L.REDUCE_ID["sqdev_onepass"]
    p = L.Plan()
    L.check(lib.dpx_reduce_plan(op, view([1 << 28], dt=L.DOUBLE), 1, view([], dt=L.DOUBLE, ptr=P1), p))
    assert L.PATH_NAMES[p.path] == "red_rows_split" and p.scratch_bytes == 131072 + 24 * p.splits
    L.check(lib.dpx_reduce_plan(op, view([1 << 20, 4]), 1, view([1 << 20], dt=L.DOUBLE, ptr=P1), p))
    assert L.PATH_NAMES[p.path] in ("red_small", "red_rows")
    L.check(lib.dpx_reduce_plan(op, view([16384, 16384], [1, 16384]), 1, view([16384], dt=L.DOUBLE, ptr=P1), p))
    assert L.PATH_NAMES[p.path] == "red_cols_split"  # down the columns
    L.check(lib.dpx_reduce_plan(op, view([17, 1 << 20], [1, 17]), 1, view([17], dt=L.DOUBLE, ptr=P1), p))
    assert L.PATH_NAMES[p.path] == "red_cols_split"  # (not the flat stream of short rows)
    L.check(lib.dpx_reduce_plan(op, view([1024, 256, 1024], [1024, 1 << 20, 1]), 2, view([1024], dt=L.DOUBLE, ptr=P1),
                                p))
    assert L.PATH_NAMES[p.path] == "red_generic" and p.red_nd == 2  # lanes walk the reduced dims
    L.check(lib.dpx_reduce_plan(op, view([16384, 8192], [16384, 2]), 1, view([16384], dt=L.DOUBLE, ptr=P1), p))
    assert L.PATH_NAMES[p.path] == "red_generic"
    L.check(lib.dpx_reduce_plan(op, view([8192, 16384], [2, 16384]), 1, view([8192], dt=L.DOUBLE, ptr=P1), p))
    assert L.PATH_NAMES[p.path] == "red_cols_split"  # columns side by side at a stride, rows walked
    L.check(lib.dpx_reduce_plan(op, view([3, 4, 5, 6, 7, 8], [40320, 6720, 1008, 144, 16, 1]), 5,
                                view([3], dt=L.DOUBLE, ptr=P1), p))
    assert L.PATH_NAMES[p.path] == "red_generic" and p.red_nd == 5  # five reduced dims that stay apart
    L.check(lib.dpx_reduce_plan(op, view([128, 128, 128, 128], [1 << 14, 1, 1 << 21, 128]), 2,
                                view([128, 128], dt=L.DOUBLE, ptr=P1), p))
    assert L.PATH_NAMES[p.path] in ("red_cols", "red_cols_split") and p.red_nd == 2
    assert [(s, d) for s in range(14) for d in range(14) if lib.dpx_reduce_dtype_supported(op, s, d)] \
        == [(s, L.DOUBLE) for s in (L.INT8, L.UINT8, L.INT16, L.UINT16, L.INT32, L.UINT32, L.INT64, L.UINT64, L.HALF,
                                    L.FLOAT, L.DOUBLE)]
    # searches walk the reduced space too (its dims keep their order)
    L.check(lib.dpx_argreduce_plan(0, view([16384, 16382], [16384, 1]), 2, view([], dt=L.INT64, ptr=P1), pa))
    assert L.PATH_NAMES[pa.path] == "red_generic" and pa.red_nd == 2 and pa.vec == 1


def test_validation_errors_are_raised_before_any_launch():
    B = L.BINARY_ID["add"]
    a, o = view([4, 4]), view([4, 4])
    with pytest.raises(ValueError, match="read-only"):
        L.check(lib.dpx_binary(B, a, a, view([4, 4], writable=False), None))
    with pytest.raises(ValueError, match="dimensions"):
        L.check(lib.dpx_binary(B, a, a, view([16]), None))
    with pytest.raises(ValueError, match="shapes"):
        L.check(lib.dpx_binary(B, a, a, view([4, 5]), None))
    with pytest.raises(ValueError, match="result type"):
        L.check(lib.dpx_binary(B, a, a, view([4, 4], dt=L.DOUBLE), None))
    with pytest.raises(ValueError, match="ample"):
        L.check(lib.dpx_binary(B, a, a, view([4, 4], [0, 1]), None))
    with pytest.raises(ValueError, match="overlapping"):
        L.check(lib.dpx_binary(B, a, a, view([4, 4], ptr=FAKE + 4), None))
    with pytest.raises(ValueError, match="unexpected elemental data type"):
        L.check(lib.dpx_unary(L.UNARY_ID["exp"], view([4], dt=L.INT32), view([4], dt=L.INT32), None))
    R = L.REDUCE_ID
    with pytest.raises(ValueError, match="rank"):
        L.check(lib.dpx_reduce(R["sum"], view([4, 4]), 1, view([4, 1], ptr=P1), None, None))
    with pytest.raises(ValueError, match="Trailing"):
        L.check(lib.dpx_reduce(R["sum"], view([4, 4]), 0, view([4, 4], ptr=P1), None, None))
    with pytest.raises(ValueError, match="overlapping"):
        L.check(lib.dpx_reduce(R["sum"], view([4, 4]), 1, view([4]), None, None))
    with pytest.raises(RuntimeError, match="not supported"):
        L.check(lib.dpx_reduce(R["sum"], view([4, 4], dt=L.DOUBLE), 1, view([4], dt=L.FLOAT, ptr=FAKE + 4096), None, None))
    with pytest.raises(ValueError, match="zero-size"):
        L.check(lib.dpx_reduce(R["max"], view([4, 0]), 1, view([4], ptr=FAKE + 4096), None, None))
    with pytest.raises(ValueError, match="zero-size"):
        L.check(lib.dpx_argreduce(0, view([4, 0]), 1, view([4], dt=L.INT64, ptr=FAKE + 4096), None))
    # zero-size iteration spaces succeed without touching the device
    L.check(lib.dpx_binary(B, view([0]), view([0]), view([0]), None))
    L.check(lib.dpx_reduce(R["sum"], view([0, 4]), 1, view([0], ptr=P1), None, None))


def test_overlap_predicates():
    a = view([10], ptr=FAKE)
    assert lib.dpx_array_overlap(a, view([10], ptr=FAKE + 36)) == 1
    assert lib.dpx_array_overlap(a, view([10], ptr=FAKE + 40)) == 0
    assert lib.dpx_array_overlap(view([5], [2], ptr=FAKE), view([5], [2], ptr=FAKE + 4)) == 1  # interleaved: ranges meet
    assert lib.dpx_same_logical(a, view([10], ptr=FAKE)) == 1
    assert lib.dpx_same_logical(a, view([10], [2], ptr=FAKE)) == 0
    assert lib.dpx_same_logical(a, view([10], ptr=FAKE, dt=L.INT32)) == 0


def test_extension_module_binds_the_same_library_and_names_its_functions_like_the_reference():
    """dpnp_amd._dpx_ext (pybind11) links libdpnp_amd.so and makes the boundary functions under the
    reference's names and keyword arguments (tensor_elementwise.cpp:42, elementwise_common.cpp:118-188,
    reductions/sum.cpp: `_sum_over_axis(src, trailing_dims_to_reduce, dst, sycl_queue, depends)`)."""
    import dpnp_amd._lib as L
    from dpnp_amd.tensor import _tensor_elementwise_impl as tei
    from dpnp_amd.tensor import _tensor_impl as ti
    from dpnp_amd.tensor import _tensor_reductions_impl as tri

    ext = L.ext
    for fn, name, args in ((tei._add, "_add", ("src1", "src2", "dst", "sycl_queue", "depends")),
                           (tei._exp, "_exp", ("src", "dst", "sycl_queue", "depends")),
                           (tei._add_inplace, "_add_inplace", ("lhs", "rhs", "sycl_queue", "depends")),
                           (tri._sum_over_axis, "_sum_over_axis", ("src", "trailing_dims_to_reduce", "dst", "sycl_queue", "depends")),
                           (tri._argmax_over_axis, "_argmax_over_axis", ("src", "trailing_dims_to_reduce", "dst", "sycl_queue", "depends")),
                           (ti._where, "_where", ("condition", "x1", "x2", "dst", "sycl_queue", "depends")),
                           (ti._copy_usm_ndarray_into_usm_ndarray, "_copy_usm_ndarray_into_usm_ndarray", ("src", "dst", "sycl_queue", "depends"))):
        assert type(fn).__name__ == "builtin_function_or_method" and fn.__name__ == name
        sig = fn.__doc__.splitlines()[0]
        assert all(f"{a}:" in sig for a in args), sig
    # a wrong argument is a TypeError before anything reaches the library, as with the reference's bindings
    with pytest.raises(TypeError):
        tei._add(1, 2, 3)
    # the plain-call functions decline what they do not handle instead of guessing
    assert ext.binary_call(L.BINARY_ID["add"], 1.0, 2.0, None) is NotImplemented
    assert ext.reduce_call(L.REDUCE_ID["sum"], object(), None, None) is NotImplemented
    assert ext.where_call(None, None, None, None) is NotImplemented
    with pytest.raises(ValueError):
        ext.set_binary_type(10 ** 6, 0, 0)
