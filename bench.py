"""Throughput of the hot path on one MI355X.

A step = one pass over the metric's workloads, inputs resident in HBM:
  add      c = a + b          fp32, 2^28 elements             12 B/elem  3.221 GB
  sum_ax1  M.sum(axis=-1)     fp32, 16384 x 16384 (2^28)       4 B/elem  1.074 GB
  sum_ax0  M.sum(axis=0)      same matrix                      4 B/elem  1.074 GB
  argmax   x.argmax()         fp32, 2^28 elements -> int64     4 B/elem  1.074 GB
value = algorithmic bytes of the step / wall time of the step on the GPU (GB/s, 1 GB = 1e9 B).
All calls go through the dpnp-style Python surface, hence through the C ABI of libdpnp_amd.so.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


def cpu_baseline(n_log2=28, repeats=5):
    """The C restatement of the reference's algorithms (oracle/oracle_c.c) on the host cores, at
    the metric's own size (2^28 elements per array); the bounded sample is the number of passes."""
    import numpy as np

    from oracle.oracle_c import OracleC

    oc = OracleC()
    n = 1 << n_log2
    rng = np.random.default_rng(0)
    a = rng.random(n, dtype=np.float32)
    b = rng.random(n, dtype=np.float32)
    a *= 2
    a -= 1  # uniform[-1, 1), in place: three 1 GiB arrays are all the host memory this takes
    b *= 2
    b -= 1
    out = np.empty_like(a)
    oc.add(a, b, out)
    oc.sum(a)
    oc.argmax(a)  # warm-up (page faults, thread pool)
    t0 = time.perf_counter()
    for _ in range(repeats):
        oc.add(a, b, out)
        oc.sum(a)
        oc.sum(b)
        oc.argmax(a)
    dt = time.perf_counter() - t0
    nbytes = repeats * n * (12 + 4 + 4 + 4)
    # second stand-in: NumPy on one thread, one pass of the same calls
    t0 = time.perf_counter()
    np.add(a, b, out=out)
    a.sum()
    b.sum()
    a.argmax()
    dt_np = time.perf_counter() - t0
    return {
        "value": nbytes / dt / 1e9, "unit": "GB/s", "cores": oc.threads, "kind": "port",
        "sample": f"{repeats} passes of add + 2 x sum + argmax over 2^{n_log2} fp32 elements "
                  "(C/OpenMP restatement of the reference's kernels, oracle/oracle_c.c; the metric's own size)",
        "numpy_one_thread": {"value": n * (12 + 4 + 4 + 4) / dt_np / 1e9, "unit": "GB/s", "cores": 1,
                             "sample": "one pass of the same calls through NumPy"},
    }


PRIME_STEPS = 24
CONFIG_STEPS = 12  # timed steps of each of cfg1..cfg5 inside the default run
MALL_BYTES = 256 << 20  # last-level (memory-side) cache of the MI355X

WORKLOADS = {
    "metric": "fp32 add 2^28 + sum axis=-1 and axis=0 over 16384x16384 + argmax 2^28 (->int64)",
    "cfg1": "fp32 add of two 2^24 arrays, then sum of the result",
    "cfg2": "fp32 16384x16384: sum and max along axis=1 and axis=0",
    "cfg3": "fp32 2^28 normal(0,1), 1 % duplicated extrema, 0.1 % NaN: argmax, argmin, mean and var accumulated in fp64 "
            "(fp32 input and fp64 input)",
    "cfg4": "8192x8192 fp32 views A[:, ::2], A.T and a (1,4096) row: multiply, exp, where(A>0, A, B); int32 bitwise_and",
    "cfg5": "Black-Scholes over 2^26 fp64 options, call and put: one fused kernel, and the chain of elementwise calls",
    "floors": "access patterns and instruction streams on their own (dpnp_amd/csrc/floors.hip), each beside the product "
              "call it bounds: Black-Scholes split into its memory streams and its arithmetic, the 2^24 read with and "
              "without a cross-block step, every-other-column reads, 512-byte runs on both sides of a transposition",
    "survey": "functions outside the named configurations that run furthest below the HBM rate: fp64 pow / asinh / atanh / "
              "log1p / tan / sin / cos / logaddexp over 2^26 elements, complex128 exp / sin / cos / sinh / tanh / expm1 over "
              "2^25, float16 sin / sinh over 2^27, column sums of a 32768x32768 int8 matrix, the variance of a 16384x32768 "
              "float16 matrix down its columns",
    "colsearch": "argmax and max down the columns of fp32 matrices of 2^28 elements with 128 to 4096 columns, and argmax "
                 "along the middle axis of 65536x32x128",
    "ewlayouts": "fp32 elementwise calls over 16384x16384 outside the named configurations: a matrix with a row / a "
                 "column, calls that only write (an outer sum, pairwise differences, a fill), two operands over slices "
                 "of wider matrices (halves, every other row, the interior), a transposed operand",
    "layouts": "fp32 2^28 elements reduced over dims that do not collapse into one run: a sliced matrix summed whole, "
               "axes (0, 2) of 3-d and 4-d arrays, every other column (sum, max, mean, argmax)",
}


def _device_array(dpnp, torch, t):
    """A dpnp array (memory of the library's own pool) holding the values of torch tensor t.  torch only
    generates the synthetic data: its tensor is viewed as an array of this package without a copy (any
    object with data_ptr() and numel() serves as a buffer) and copied by the library's copy kernel on the
    library's stream, before anything is timed."""
    from dpnp_amd.tensor._usmarray import usm_ndarray

    names = {torch.float32: "f4", torch.float64: "f8", torch.int32: "i4", torch.int8: "i1", torch.bool: "?"}
    t = t.contiguous()
    arr = dpnp.empty(tuple(t.shape), dtype=names[t.dtype])
    torch.cuda.synchronize()  # t is complete (torch's stream) before the library's stream reads it
    src = usm_ndarray(tuple(t.shape), dtype=names[t.dtype], buffer=t.view(-1).view(torch.uint8))
    dpnp.copyto(arr, dpnp.ndarray._create_from_usm_ndarray(src))
    dpnp.synchronize()  # ... and the copy is complete before torch frees or reuses t
    return arr


def build_workload(name, dpnp, torch):
    """-> (ops, dtype, data): ops = [(label, callable, algorithmic bytes, elements[, physical bytes])].
    Algorithmic bytes = every input element read once + every output element written once."""
    g = torch.Generator(device="cuda").manual_seed(0)

    def uniform(shape, lo=-1.0, hi=1.0, dtype=torch.float32):
        t = torch.rand(shape, device="cuda", generator=g, dtype=dtype) * (hi - lo) + lo
        return _device_array(dpnp, torch, t)

    def normal(shape):
        return _device_array(dpnp, torch, torch.randn(shape, device="cuda", generator=g))

    if name == "metric":
        n, side = 1 << 28, 1 << 14
        a, b, x = uniform(n), uniform(n), normal(n)
        c = dpnp.empty(n, dtype="f4")
        M = a.reshape(side, side)
        r1, r0 = dpnp.empty(side, dtype="f4"), dpnp.empty(side, dtype="f4")
        idx = dpnp.empty((), dtype="i8")
        ops = [
            ("add", lambda: dpnp.add(a, b, out=c), 12 * n, n),
            ("sum_axis1", lambda: dpnp.sum(M, axis=1, out=r1), 4 * n + 4 * side, n),
            ("sum_axis0", lambda: dpnp.sum(M, axis=0, out=r0), 4 * n + 4 * side, n),
            ("argmax", lambda: dpnp.argmax(x, out=idx), 4 * n + 8, n),
            # plain copy of known size: calibrates the FETCH_SIZE / WRITE_SIZE counters (--ops copy)
            ("copy", lambda: dpnp.copyto(c, a), 8 * n, n),
        ]
        return ops, "f32", "synthetic (seeded uniform[-1,1) and normal(0,1), resident in HBM)"
    if name == "cfg1":
        n = 1 << 24
        a, b = uniform(n), uniform(n)
        c, s = dpnp.empty(n, dtype="f4"), dpnp.empty((), dtype="f4")
        ops = [("add", lambda: dpnp.add(a, b, out=c), 12 * n, n),
               ("sum", lambda: dpnp.sum(c, out=s), 4 * n + 4, n)]
        return ops, "f32", "synthetic (seeded uniform[-1,1), resident in HBM)"
    if name == "cfg2":
        side = 1 << 14
        n = side * side
        M = uniform((side, side))
        r = [dpnp.empty(side, dtype="f4") for _ in range(4)]
        nb = 4 * n + 4 * side
        ops = [("sum_axis1", lambda: dpnp.sum(M, axis=1, out=r[0]), nb, n),
               ("max_axis1", lambda: dpnp.max(M, axis=1, out=r[1]), nb, n),
               ("sum_axis0", lambda: dpnp.sum(M, axis=0, out=r[2]), nb, n),
               ("max_axis0", lambda: dpnp.max(M, axis=0, out=r[3]), nb, n)]
        return ops, "f32", "synthetic (seeded uniform[-1,1), resident in HBM)"
    if name == "cfg3":
        n = 1 << 28
        t = torch.randn(n, device="cuda", generator=g)
        # distinct places (a choice without replacement): 1 % maxima, 1 % minima, then 0.1 % NaN
        perm = torch.randperm(n, device="cuda", generator=g)
        t[perm[: n // 100]] = t.max()
        t[perm[n // 100: 2 * (n // 100)]] = t.min()
        clean = _device_array(dpnp, torch, t)
        clean64 = _device_array(dpnp, torch, t.double())
        pick = perm[2 * (n // 100): 2 * (n // 100) + n // 1000]
        del perm
        t[pick] = float("nan")
        x = _device_array(dpnp, torch, t)
        del t, pick
        i0, i1 = dpnp.empty((), dtype="i8"), dpnp.empty((), dtype="i8")
        m = [dpnp.empty((), dtype="f8") for _ in range(4)]
        m32 = dpnp.empty((), dtype="f4")
        ops = [("argmax_nan", lambda: dpnp.argmax(x, out=i0), 4 * n + 8, n),
               ("argmin_nan", lambda: dpnp.argmin(x, out=i1), 4 * n + 8, n),
               ("argmax", lambda: dpnp.argmax(clean, out=i0), 4 * n + 8, n),
               ("mean_f32_acc64", lambda: dpnp.mean(clean, dtype="f8", out=m[0]), 4 * n + 8, n),
               # one pass: count, mean and squared deviations travel together (the reference reads the input twice)
               ("var_f32_acc64", lambda: dpnp.var(clean, dtype="f8", out=m[1]), 4 * n + 8, n),
               ("mean_f64", lambda: dpnp.mean(clean64, out=m[2]), 8 * n + 8, n),
               ("var_f64", lambda: dpnp.var(clean64, out=m[3]), 8 * n + 8, n),
               # NaN-ignoring forms on the NaN variant, one pass each
               ("nanargmax_nan", lambda: dpnp.nanargmax(x, out=i0), 4 * n + 8, n),
               ("nanmean_nan", lambda: dpnp.nanmean(x, out=m32), 4 * n + 4, n)]
        return ops, "f32 (fp64 accumulation)", "synthetic (seeded normal(0,1) with planted extrema / NaN, resident in HBM)"
    if name == "cfg4":
        side = 8192
        A, B = normal((side, side)), normal((1, side // 2))
        ints = [_device_array(dpnp, torch, torch.randint(-2**31, 2**31, (side, side), device="cuda", generator=g,
                                                         dtype=torch.int64).to(torch.int32)) for _ in range(2)]
        V1, V2 = A[:, ::2], A.T
        h = side * side // 2
        o_half = dpnp.empty((side, side // 2), dtype="f4")
        o_f = dpnp.empty((side, side), dtype="f4").T  # F-contiguous, the layout order="K" gives exp(A.T)
        o_c = dpnp.empty((side, side), dtype="f4")
        o_b = dpnp.empty((side, side // 2), dtype="?")
        o_i = dpnp.empty((side, side), dtype="i4")
        o_ih = dpnp.empty((side, side // 2), dtype="i4")

        def where_unfused():
            dpnp.greater(V1, 0, out=o_b)
            dpnp.where(o_b, V1, B, out=o_half)

        # fifth field: the bytes moved physically.  A [:, ::2] view occupies every 128-byte line of its base
        # matrix, so reading it reads the whole matrix (8 bytes per element of the view instead of 4)
        row = 4 * (side // 2)
        ops = [("multiply_V1_B", lambda: dpnp.multiply(V1, B, out=o_half), 8 * h + row, h, 12 * h + row),
               ("exp_V1", lambda: dpnp.exp(V1, out=o_half), 8 * h, h, 12 * h),
               ("exp_AT_keep_layout", lambda: dpnp.exp(V2, out=o_f), 8 * 2 * h, 2 * h),
               ("exp_AT_to_C", lambda: dpnp.exp(V2, out=o_c), 8 * 2 * h, 2 * h),
               ("where_greater_fused", lambda: dpnp.where_compare("greater", V1, 0, V1, B, out=o_half),
                8 * h + row, h, 12 * h + row),
               ("where_greater_two_calls", where_unfused, (4 + 1) * h + (1 + 4 + 4) * h + row, h,
                (8 + 1) * h + (1 + 8 + 4) * h + row),
               ("bitwise_and", lambda: dpnp.bitwise_and(ints[0], ints[1], out=o_i), 12 * 2 * h, 2 * h),
               ("bitwise_and_V1", lambda: dpnp.bitwise_and(ints[0][:, ::2], ints[1][:, ::2], out=o_ih), 12 * h, h, 20 * h),
               # plain copy of known size: calibrates the FETCH_SIZE / WRITE_SIZE counters (--ops ...,copy)
               ("copy", lambda: dpnp.copyto(o_i, ints[0]), 8 * 2 * h, 2 * h)]
        return ops, "f32/i32/bool", "synthetic (seeded normal(0,1), uniform int32, resident in HBM)"
    if name == "cfg5":
        n = 1 << 26
        price = uniform(n, 10.0, 50.0, torch.float64)
        strike = uniform(n, 10.0, 50.0, torch.float64)
        t = uniform(n, 1.0, 2.0, torch.float64)
        call, put = dpnp.empty(n, dtype="f8"), dpnp.empty(n, dtype="f8")
        r, vol = 0.1, 0.2

        def chain():
            # the expression tree of the reference's example (examples/example_bs.py:50-78), one call per node
            a = dpnp.log(price / strike)
            b = t * (-r)
            z = t * (vol * vol * 2)
            c = 0.25 * z
            y = 1.0 / dpnp.sqrt(z)
            w1 = (a - b + c) * y
            w2 = (a - b - c) * y
            d1 = 0.5 + 0.5 * dpnp.erf(w1)
            d2 = 0.5 + 0.5 * dpnp.erf(w2)
            se = dpnp.exp(b) * strike
            res = price * d1 - se * d2
            dpnp.copyto(call, res)
            dpnp.subtract(res, price, out=put)
            dpnp.add(put, se, out=put)

        ops = [("black_scholes_fused", lambda: dpnp.black_scholes(price, strike, t, r, vol, call=call, put=put), 40 * n, n),
               ("black_scholes_chain", chain, 40 * n, n)]
        return ops, "f64", "synthetic (seeded uniform price, strike [10,50), T [1,2), resident in HBM)"
    if name == "layouts":
        side = 1 << 14
        n = side * side
        A = normal((side, side))
        X3, X3s, X4 = A.reshape(4096, 256, 256), A.reshape(256, 1024, 1024), A.reshape(128, 128, 128, 128)
        s0, i0 = dpnp.empty((), dtype="f4"), dpnp.empty((), dtype="i8")
        r256, r1024 = dpnp.empty(256, dtype="f4"), dpnp.empty(1024, dtype="f4")
        r44 = dpnp.empty((128, 128), dtype="f4")
        rs, rh, ri = dpnp.empty(side, dtype="f4"), dpnp.empty(side // 2, dtype="f4"), dpnp.empty(side, dtype="i8")
        inner = (side - 2) * (side - 2)
        # a [:, ::2] view occupies every line of its base: the bytes moved are the whole matrix
        ops = [("sum_sliced_matrix", lambda: dpnp.sum(A[1:-1, 1:-1], out=s0), 4 * inner, inner),
               ("argmax_sliced_matrix", lambda: dpnp.argmax(A[1:-1, 1:-1], out=i0), 4 * inner, inner),
               ("sum_axes02_4096x256x256", lambda: dpnp.sum(X3, axis=(0, 2), out=r256), 4 * n, n),
               ("max_axes02_4096x256x256", lambda: dpnp.max(X3, axis=(0, 2), out=r256), 4 * n, n),
               ("mean_axes02_256x1024x1024", lambda: dpnp.mean(X3s, axis=(0, 2), out=r1024), 4 * n, n),
               ("sum_axes02_128x128x128x128", lambda: dpnp.sum(X4, axis=(0, 2), out=r44), 4 * n, n),
               ("sum_every_other_column_axis1", lambda: dpnp.sum(A[:, ::2], axis=1, out=rs), 4 * n, n // 2),
               ("sum_every_other_column_axis0", lambda: dpnp.sum(A[:, ::2], axis=0, out=rh), 4 * n, n // 2),
               ("argmax_every_other_column_axis1", lambda: dpnp.argmax(A[:, ::2], axis=1, out=ri), 4 * n, n // 2),
               # (variance in one pass, float64 accumulation; the time includes the division and the rounding of
               # the 8192 results to float32, two small launches)
               ("var_every_other_column_axis0", lambda: dpnp.var(A[:, ::2], axis=0, out=rh), 4 * n, n // 2),
               ("var_axes02_256x1024x1024", lambda: dpnp.var(X3s, axis=(0, 2), out=r1024), 4 * n, n)]
        return ops, "f32", "synthetic (seeded normal(0,1), resident in HBM)"
    if name == "ewlayouts":
        side = 1 << 14
        n, h = side * side, side // 2
        A, B = normal((side, side)), normal((side, side))
        C = dpnp.empty((side, side), dtype="f4")
        row, col = normal((1, side)), normal((side, 1))
        X, Y = normal((1024, 1, 1024)), normal((1, 256, 1024))
        P = dpnp.empty((1024, 256, 1024), dtype="f4")
        inner = (side - 2) * (side - 2)
        ops = [("add_A_B", lambda: dpnp.add(A, B, out=C), 12 * n, n),
               ("add_A_row", lambda: dpnp.add(A, row, out=C), 8 * n, n),
               ("multiply_A_col", lambda: dpnp.multiply(A, col, out=C), 8 * n, n),
               ("fill", lambda: C.fill(1.5), 4 * n, n),
               ("outer_add_row_col", lambda: dpnp.add(row, col, out=C), 4 * n, n),
               ("pairwise_subtract_1024x256x1024", lambda: dpnp.subtract(X, Y, out=P), 4 * n, n),
               ("add_halves_of_the_columns", lambda: dpnp.add(A[:, :h], A[:, h:], out=C[:, :h]), 6 * n, n // 2),
               ("add_every_other_row", lambda: dpnp.add(A[::2], B[::2], out=C[::2]), 6 * n, n // 2),
               ("add_interior", lambda: dpnp.add(A[1:-1, 1:-1], B[1:-1, 1:-1], out=C[1:-1, 1:-1]), 12 * inner, inner),
               ("sqrt_interior", lambda: dpnp.sqrt(A[1:-1, 1:-1], out=C[1:-1, 1:-1]), 8 * inner, inner),
               ("add_A_BT", lambda: dpnp.add(A, B.T, out=C), 12 * n, n),
               ("copy_AT", lambda: dpnp.copyto(C, A.T), 8 * n, n)]
        return ops, "f32", "synthetic (seeded normal(0,1), resident in HBM)"
    if name == "floors":
        return build_floors(dpnp, torch, uniform, normal)
    if name == "survey":
        n, n2, n3 = 1 << 26, 1 << 25, 1 << 27
        x, y, xs = uniform(n, 0.1, 10.0, torch.float64), uniform(n, -3.0, 3.0, torch.float64), uniform(n, -1.0, 1.0, torch.float64)
        o = dpnp.empty(n, dtype="f8")
        z = dpnp.empty(n2, dtype="c16")
        z.real[...] = uniform(n2, -2.0, 2.0, torch.float64)
        z.imag[...] = uniform(n2, -2.0, 2.0, torch.float64)
        oz = dpnp.empty(n2, dtype="c16")
        xh = dpnp.astype(uniform(n3), "f2")
        oh = dpnp.empty(n3, dtype="f2")
        B8 = _device_array(dpnp, torch, torch.randint(-100, 100, (1 << 15, 1 << 15), device="cuda", generator=g,
                                                      dtype=torch.int8))
        o8 = dpnp.empty(1 << 15, dtype="i8")
        ops = [("pow_f64", lambda: dpnp.power(x, y, out=o), 24 * n, n)]
        for fn in ("arcsinh", "arctanh", "log1p", "tan"):
            ops.append((f"{fn}_f64", lambda f=getattr(dpnp, fn): f(xs, out=o), 16 * n, n))
        for fn in ("sin", "cos"):
            ops.append((f"{fn}_f64", lambda f=getattr(dpnp, fn): f(y, out=o), 16 * n, n))
        ops.append(("logaddexp_f64", lambda: dpnp.logaddexp(x, y, out=o), 24 * n, n))
        for fn in ("exp", "sin", "cos", "sinh", "tanh", "expm1"):
            ops.append((f"{fn}_c128", lambda f=getattr(dpnp, fn): f(z, out=oz), 32 * n2, n2))
        for fn in ("sin", "sinh"):
            ops.append((f"{fn}_f16", lambda f=getattr(dpnp, fn): f(xh, out=oh), 4 * n3, n3))
        ops.append(("sum_axis0_int8_32768sq", lambda: dpnp.sum(B8, axis=0, out=o8), 1 << 30, 1 << 30))
        H16 = dpnp.astype(uniform((1 << 14, 1 << 15)), "f2")
        ov = dpnp.empty(1 << 15, dtype="f2")
        # (variance in one pass, float64 accumulation; the time includes two small launches that finish the result)
        ops.append(("var_axis0_f16_16384x32768", lambda: dpnp.var(H16, axis=0, out=ov), 1 << 30, 1 << 29))
        # the real functions the complex ones are built from (only with --ops: for instruction counts)
        for fn in ("exp", "sin", "cos", "sinh", "cosh", "expm1", "log"):
            ops.append((f"ref:{fn}_f64", lambda f=getattr(dpnp, fn): f(xs, out=o), 16 * n, n))
        return ops, "f64/c128/f16/i8", "synthetic (seeded uniform, resident in HBM)"
    if name == "colsearch":
        n = 1 << 28
        ops, keep = [], []
        A = normal((1 << 14, 1 << 14))
        for cols in (128, 256, 512, 1024, 4096):
            M = A.reshape(n // cols, cols)
            oi, of = dpnp.empty(cols, dtype="i8"), dpnp.empty(cols, dtype="f4")
            ops.append((f"argmax_axis0_{n // cols}x{cols}", lambda M=M, oi=oi: dpnp.argmax(M, axis=0, out=oi), 4 * n, n))
            ops.append((f"max_axis0_{n // cols}x{cols}", lambda M=M, of=of: dpnp.max(M, axis=0, out=of), 4 * n, n))
        X = A.reshape(65536, 32, 128)
        om = dpnp.empty((65536, 128), dtype="i8")
        ops.append(("argmax_axis1_65536x32x128", lambda: dpnp.argmax(X, axis=1, out=om), 4 * n + 8 * 65536 * 128, n))
        return ops, "f32", "synthetic (seeded normal(0,1), resident in HBM)"
    raise SystemExit(f"--workload: unknown workload {name!r} (one of {', '.join(WORKLOADS)})")


def build_floors(dpnp, torch, uniform, normal):
    """Each measurement kernel of libdpx_floors.so (label "floor:<name>") next to the product call whose time it
    bounds (label "product:<call>").  The kernels run on the library's stream, on workspaces of the package's pool."""
    import ctypes

    from dpnp_amd.tensor import _device

    path = os.path.join(ROOT, "dpnp_amd", "libdpx_floors.so")
    if not os.path.exists(path):
        raise SystemExit("dpnp_amd/libdpx_floors.so is not built: make -C dpnp_amd/csrc")
    fl = ctypes.CDLL(path)
    fl.dpx_floors_name.restype = fl.dpx_floors_about.restype = ctypes.c_char_p
    fl.dpx_floors_bytes.restype = ctypes.c_double
    fl.dpx_floors_workspace.restype = ctypes.c_size_t
    fl.dpx_floors_prepare.argtypes = fl.dpx_floors_launch.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
    stream = _device.current_stream_ptr()
    index = {fl.dpx_floors_name(i).decode(): i for i in range(fl.dpx_floors_count())}

    def floor(name):
        i = index[name]
        ws = dpnp.empty(fl.dpx_floors_workspace(i), dtype="u1")
        ptr = ws.get_array()._buf.data_ptr()
        if fl.dpx_floors_prepare(i, ptr, stream):
            raise SystemExit(f"floors: preparing {name} failed")

        def run(ws=ws):  # (the closure keeps the workspace alive)
            if fl.dpx_floors_launch(i, ptr, stream):
                raise RuntimeError(f"floors: launch of {name} failed")
        nb = fl.dpx_floors_bytes(i)
        return (f"floor:{name}", run, nb, 0)

    n26, n24, side = 1 << 26, 1 << 24, 8192
    # the product calls the floors stand beside
    price, strike = uniform(n26, 10.0, 50.0, torch.float64), uniform(n26, 10.0, 50.0, torch.float64)
    t = uniform(n26, 1.0, 2.0, torch.float64)
    call, put = dpnp.empty(n26, dtype="f8"), dpnp.empty(n26, dtype="f8")
    c24, s24 = uniform(n24), dpnp.empty((), dtype="f4")
    A, A2, B = normal((side, side)), normal((side, side)), normal((1, side // 2))
    o_half, o_b = dpnp.empty((side, side // 2), dtype="f4"), dpnp.empty((side, side // 2), dtype="?")
    o_c = dpnp.empty((side, side), dtype="f4")
    V1, V1b = A[:, ::2], A2[:, ::2]
    h = side * side // 2
    ops = [
        floor("launch"),
        floor("bs_streams"), floor("stream5_f64"), floor("bs_arithmetic"),
        ("product:black_scholes_fused", lambda: dpnp.black_scholes(price, strike, t, 0.1, 0.2, call=call, put=put), 40 * n26, n26),
        floor("read_f32_2p24"), floor("read_f32_2p24_tickets"),
        ("product:sum_f32_2p24", lambda: dpnp.sum(c24, out=s24), 4 * n24, n24),
        floor("stride2_one_input"),
        ("product:multiply_V1_row", lambda: dpnp.multiply(V1, B, out=o_half), 12 * h, h),
        floor("stride2_predicate"),
        ("product:greater_V1_0", lambda: dpnp.greater(V1, 0, out=o_b), 9 * h, h),
        floor("stride2_two_inputs"),
        ("product:multiply_V1_V1b", lambda: dpnp.multiply(V1, V1b, out=o_half), 20 * h, h),
        floor("tile_runs_8192"),
        ("product:exp_AT_to_C", lambda: dpnp.exp(A.T, out=o_c), 16 * h, 2 * h),
    ]
    ops[0] = (ops[0][0], ops[0][1], 1, 0)  # (no bytes: keep the ratio defined)
    ops[3] = (ops[3][0], ops[3][1], 1, 0)
    return ops, "f64/f32", "synthetic; bytes of the strided calls are the whole lines they touch (physical bytes)"



def dpnp_cpu_probe():
    """Looks for an installed dpnp (the reference itself, with its SYCL CPU device) on this box, in a child
    process; when there is one, times the metric's calls on its CPU device there.  The expected answer is
    "unavailable on this box": the record then says that the reference path was looked for."""
    import subprocess

    code = r"""
import importlib.util, json, sys, time
if importlib.util.find_spec("dpnp") is None or importlib.util.find_spec("dpctl") is None:
    print(json.dumps("unavailable on this box")); sys.exit(0)
try:
    import dpctl, dpnp
    dev = dpctl.SyclDevice("cpu")
    n = 1 << 24
    a = dpnp.random.uniform(-1, 1, n, device=dev).astype(dpnp.float32)
    b = dpnp.random.uniform(-1, 1, n, device=dev).astype(dpnp.float32)
    q = a.sycl_queue
    def timed(f):
        for _ in range(5): f(); q.wait()
        ts = []
        for _ in range(20):
            t0 = time.perf_counter(); f(); q.wait(); ts.append(time.perf_counter() - t0)
        return sorted(ts)[10]
    out = {"cores": dev.max_compute_units, "elements": n,
           "add_GB/s": 12 * n / timed(lambda: dpnp.add(a, b)) / 1e9,
           "sum_GB/s": 4 * n / timed(lambda: dpnp.sum(a)) / 1e9,
           "argmax_GB/s": 4 * n / timed(lambda: dpnp.argmax(a)) / 1e9}
    print(json.dumps(out))
except Exception as e:
    print(json.dumps("present but not usable: %s: %s" % (type(e).__name__, e)))
"""
    try:
        r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120)
        return json.loads(r.stdout.strip().splitlines()[-1])
    except Exception as e:  # the probe must never take the bench down
        return f"probe failed: {type(e).__name__}: {e}"


def _pool_bytes_in_use():
    import ctypes

    from dpnp_amd import _lib

    used, cached = ctypes.c_size_t(), ctypes.c_size_t()
    _lib.check(_lib.lib.dpx_mem_stats(ctypes.byref(used), ctypes.byref(cached)))
    return used.value


def measure(name, dpnp, torch, steps, warmup, prime, ops_filter=None, dump=False):
    """Runs workload `name`: `prime` + `warmup` untimed steps, then exactly `steps` timed ones.  Every op is
    bracketed by HIP events recorded on the library's own stream (the one its kernels are launched on)."""
    from dpnp_amd.tensor import _device

    stream = torch.cuda.ExternalStream(_device.current_stream_ptr())

    def select(all_ops):
        if ops_filter is None:
            return [o for o in all_ops if o[0] != "copy" and not o[0].startswith("ref:")]
        wanted = [w for w in ops_filter.split(",") if w]
        sel = [o for o in all_ops if o[0] in wanted]
        if not sel or len(sel) != len(wanted):
            print(f"--ops: unknown op in {wanted}; {name} has {[o[0] for o in all_ops]}", file=sys.stderr)
            sys.exit(2)
        return sel

    mem0 = _pool_bytes_in_use()
    all_ops, dtype, data = build_workload(name, dpnp, torch)
    working_set = _pool_bytes_in_use() - mem0
    # A workload whose arrays fit the 256 MiB memory-side cache would be served from it when every
    # step reuses the same buffers: such a workload gets several buffer sets, enough that a set has
    # left the cache (3 x its size has streamed through) when its turn comes again.
    nsets = 1 if working_set >= MALL_BYTES else min(8, -(-3 * MALL_BYTES // max(working_set, 1)) + 1)
    op_sets = [select(all_ops)] + [select(build_workload(name, dpnp, torch)[0]) for _ in range(nsets - 1)]
    ops = op_sets[0]
    step_bytes = sum(o[2] for o in ops)

    host_us = []
    step_no = [0]

    def step(events=None):
        cur = op_sets[step_no[0] % nsets]
        step_no[0] += 1
        for k, o in enumerate(cur):
            if events is not None:
                events[k][0].record(stream)
            h0 = time.perf_counter()
            o[1]()
            host_us.append((time.perf_counter() - h0) * 1e6)
            if events is not None:
                events[k][1].record(stream)

    def sync():
        dpnp.synchronize()
        torch.cuda.synchronize()

    # Process start-up, not steady state: the first launch of each kernel loads its code object,
    # and the HIP runtime stalls the submitting thread once, for 30-40 ms, a few dozen launches
    # into a process (seen on the host clock around a launch, with the GPU idle).  Both are kept
    # out of the W + K steps whatever W is.
    for _ in range(prime):
        step()
    sync()
    for _ in range(warmup):
        step()
    sync()
    ev = [[[torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)] for _ in ops]
          for _ in range(steps)]
    t_begin, t_end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    sync()
    del host_us[:]
    wall0 = time.perf_counter()
    t_begin.record(stream)
    for s in range(steps):
        step(ev[s])
    t_end.record(stream)
    sync()
    wall = time.perf_counter() - wall0
    gpu_ms = t_begin.elapsed_time(t_end)
    ms_per_step = max(gpu_ms, wall * 1e3) / steps
    per_op = {}
    for k, o in enumerate(ops):
        label, nb, nel = o[0], o[2], o[3]
        times = sorted(ev[s][k][0].elapsed_time(ev[s][k][1]) for s in range(steps))
        ms = sum(times) / steps
        med = times[steps // 2] if steps % 2 else 0.5 * (times[steps // 2 - 1] + times[steps // 2])
        host = sorted(host_us[s * len(ops) + k] for s in range(steps))
        # host_us_median: time the submitting thread spends inside the call (Python layer, C ABI,
        # launch), which bounds the rate of calls whose kernels are shorter than that
        per_op[label] = {"ms": round(ms, 5), "ms_median": round(med, 5), "host_us_median": round(host[steps // 2], 1),
                         "GB/s": round(nb / ms / 1e6, 1),
                         "frac_of_peak": round(nb / ms / 1e6 / HBM_PEAK_GBS, 4),
                         "frac_of_peak_median": round(nb / med / 1e6 / HBM_PEAK_GBS, 4),
                         "elements/s": round(nel / ms * 1e3)}
        if len(o) > 4:  # bytes the call moves physically (whole lines of a strided view)
            per_op[label]["frac_physical"] = round(o[4] / ms / 1e6 / HBM_PEAK_GBS, 4)
    if dump:
        for s in range(steps):
            print(s, " ".join("%s=%.4f(host %.0fus)" % (ops[k][0], ev[s][k][0].elapsed_time(ev[s][k][1]),
                                                         host_us[s * len(ops) + k]) for k in range(len(ops))),
                  file=sys.stderr)
    del op_sets, all_ops
    return {"ops": [(o[0], o[2]) for o in ops], "dtype": dtype, "data": data, "nsets": nsets,
            "step_bytes": step_bytes, "ms_per_step": ms_per_step, "per_op": per_op}


def release_memory(torch):
    import gc

    from dpnp_amd import _lib

    gc.collect()
    _lib.check(_lib.lib.dpx_mem_release_cached())
    torch.cuda.empty_cache()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-configs", action="store_true",
                    help="metric workload only: leave out the short runs of cfg1..cfg5 that fill `configs`")
    ap.add_argument("--dump-steps", action="store_true", help="print every step's per-op times to stderr")
    ap.add_argument("--workload", default="metric",
                    help="metric (default, the headline step) or one of the parity configurations cfg1..cfg5, layouts, ewlayouts "
                         "or floors, measured the same way")
    ap.add_argument("--ops", default=None,
                    help="comma-separated subset of the workload's ops (profiling runs); 'copy' in the metric "
                         "workload is a plain copy of known size")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (--gpus must be 1)", file=sys.stderr)
        sys.exit(2)

    # torch generates the synthetic data and provides the timing events; it is imported before the package so
    # that both use one HIP runtime.  The package itself runs on its own memory pool and stream.
    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    import dpnp_amd as dpnp
    from dpnp_amd import _lib

    m = measure(args.workload, dpnp, torch, args.steps, args.warmup, PRIME_STEPS, args.ops, args.dump_steps)
    per_op, ms_per_step, step_bytes = m["per_op"], m["ms_per_step"], m["step_bytes"]
    # the roofline object describes the op with the largest share of the step
    dom_name, dom_bytes = max(m["ops"], key=lambda o: per_op[o[0]]["ms"])
    dom_ms = per_op[dom_name]["ms"]
    kernel = ("ew_contig_kernel<add,f32> (c = a + b, 2^28 elements)" if (args.workload, dom_name) == ("metric", "add")
              else f"{args.workload}:{dom_name}")
    workload = WORKLOADS[args.workload] if args.ops is None else f"{args.workload}, subset: {args.ops}"
    out = {
        "metric": "achieved HBM GB/s for fp32 add, axis-sum, argmax at 2^28 elements" if args.workload == "metric"
                  else f"achieved HBM GB/s (algorithmic bytes / time), configuration {args.workload}",
        "value": round(step_bytes / ms_per_step / 1e6, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "primed": PRIME_STEPS,  # untimed steps before the warm-up (process start-up, see above)
        "buffer_sets": m["nsets"],   # distinct sets of arrays the steps cycle through
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": m["dtype"],
        "data": m["data"],
        "memory_and_stream": _lib.MEMORY,  # "native": dpx_mem_alloc / dpx_stream_create
        "config": {"workload": workload, "bytes_per_step": step_bytes,
                   "frac_of_hbm_peak": round(step_bytes / ms_per_step / 1e6 / HBM_PEAK_GBS, 4)},
        "per_op": per_op,
        "roofline": {"bound": "hbm", "kernel": kernel,
                     "achieved": round(dom_bytes / dom_ms / 1e6, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(dom_bytes / dom_ms / 1e6 / HBM_PEAK_GBS, 4), "traffic": None},
    }
    traffic_file = os.path.join(ROOT, "profiles", "add_f32_2p28_traffic.json")
    if (args.workload, dom_name) == ("metric", "add") and os.path.exists(traffic_file):
        # HBM bytes per launch from the committed rocprofv3 --pmc summary
        out["roofline"]["traffic"] = json.load(open(traffic_file)).get("bytes_per_launch")
        out["roofline"]["traffic_source"] = "profiles/add_f32_2p28_traffic.json (rocprofv3 --pmc, not measured in this run)"
    if args.workload == "metric" and args.ops is None and not args.no_configs:
        # the other configurations, a few steps each (parity cases, not the headline: their own lines come
        # from --workload cfgN): per op, time and share of the HBM peak on algorithmic bytes, and on the
        # bytes physically moved where a strided view makes the two differ
        configs = {}
        for cfg in ("cfg1", "cfg2", "cfg3", "cfg4", "cfg5"):
            release_memory(torch)
            c = measure(cfg, dpnp, torch, CONFIG_STEPS, 3, 4)
            configs[cfg] = {
                "workload": WORKLOADS[cfg], "steps": CONFIG_STEPS, "buffer_sets": c["nsets"],
                "ms_per_step": round(c["ms_per_step"], 5),
                "sum_of_op_ms": round(sum(v["ms"] for v in c["per_op"].values()), 5),  # event times of the ops, launch gaps excluded
                "per_op": {k: {f: v[f] for f in ("ms", "host_us_median", "frac_of_peak", "frac_physical") if f in v}
                           for k, v in c["per_op"].items()}}
        out["configs"] = configs
        release_memory(torch)
    if not args.no_cpu_baseline and args.workload == "metric":
        out["cpu_baseline"] = cpu_baseline()
        out["cpu_baseline"]["dpnp_cpu"] = dpnp_cpu_probe()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
