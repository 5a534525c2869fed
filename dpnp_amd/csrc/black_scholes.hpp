// Black-Scholes pricing as one fused kernel: the device code, shared by the entry point (ew_misc.hip) and by
// the measurement kernels that run its two halves apart (floors.hip).
#pragma once
#include "ew_dispatch.hpp"
#include "erf_fine_table.hpp"

namespace dpx {

// ---- Black-Scholes, formula of examples/example_bs.py:50-78 --------------------------------------------
// One thread prices E options: 3 loads, 2 stores of 16 bytes.  Every product and sum is a
// separate rounding (the library is built with -ffp-contract=off), matching the
// reference's chain of one kernel per operation.
template <class T> struct BlackScholesFn {
    T mr, sig_sig_two, quarter, half_, one;
    // returns call; put through the second output of the kernel below
    DPX_D void price(T p, T s, T t, T &call, T &put) const
    {
        const T a = m_log(p / s);
        const T b = t * mr;
        const T z = t * sig_sig_two;
        const T c = quarter * z;
        const T y = one / m_sqrt(z);
        const T w1 = (a - b + c) * y;
        const T w2 = (a - b - c) * y;
        const T d1 = half_ + half_ * m_erf(w1);
        const T d2 = half_ + half_ * m_erf(w2);
        const T se = m_exp(b) * s;
        call = p * d1 - se * d2;
        put = call - p + se;
    }
};

// ---- the same formula for doubles with its elementary functions cut to the formula's needs -------
// price() above spends 198 vector instructions per option, and fp64 instruction issue, not HBM,
// bounds the kernel.  Every piece below is accurate to about one ULP of its own result (checked on
// the host against long double over 2e7 arguments each: quotient 2.2e-16, 1/sqrt 1.4e-16, exp
// 1.4e-16 relative, erf 2.7e-16 absolute), so prices agree with the chain of elementwise calls to a
// few ULP of the larger product (the entry point's contract is 1e-12), but no longer bit for bit.
//   * p / s and 1 / sqrt(z): hardware estimate (23 bits) and one cubically convergent step (the
//     IEEE division and square root sequences take 12 and 18 instructions, these 5 and 6);
//   * exp: k = rint(b log2 e), r = b - k ln 2 in two parts, Taylor polynomial of degree 13, ldexp;
//   * erf: the Taylor series about the nearest r = i/256 (erf_fine_table.hpp) to the fifth order;
//     the argument is rounded to the grid by adding 1.5 * 2^44, which leaves the index in the low
//     mantissa bits;
//   * no handling of special values in the pieces: BlackScholesFast::price() is for waves in which
//     every option has p / s and 2 vol^2 t positive and normal and |rate t| < 700; the kernel sends
//     every other wave through BlackScholesFn::price().
DPX_D double bs_rcp(double s)
{
    const double rc = __builtin_amdgcn_rcp(s);
    const double e = __builtin_fma(-s, rc, 1.0);
    return __builtin_fma(rc, __builtin_fma(e, e, e), rc); // rc (1 + e + e^2)
}
DPX_D double bs_rsqrt(double z)
{
    const double y = __builtin_amdgcn_rsq(z);
    const double e = __builtin_fma(-(z * y), y, 1.0);
    const double t = __builtin_fma(e, 0.375, 0.5) * e; // y (1 + e/2 + 3 e^2 / 8)
    return __builtin_fma(y, t, y);
}
DPX_D double bs_exp(double b) // |b| < 700
{
    constexpr double log2e = 1.4426950408889634074, ln2_hi = 6.93147180369123816490e-01,
                     ln2_lo = 1.90821492927058770002e-10;
    const double k = __builtin_rint(b * log2e);
    double r = __builtin_fma(-k, ln2_hi, b);
    r = __builtin_fma(-k, ln2_lo, r);
    double p = 1.0 / 6227020800.0;
    p = __builtin_fma(p, r, 1.0 / 479001600.0);
    p = __builtin_fma(p, r, 1.0 / 39916800.0);
    p = __builtin_fma(p, r, 1.0 / 3628800.0);
    p = __builtin_fma(p, r, 1.0 / 362880.0);
    p = __builtin_fma(p, r, 1.0 / 40320.0);
    p = __builtin_fma(p, r, 1.0 / 5040.0);
    p = __builtin_fma(p, r, 1.0 / 720.0);
    p = __builtin_fma(p, r, 1.0 / 120.0);
    p = __builtin_fma(p, r, 1.0 / 24.0);
    p = __builtin_fma(p, r, 1.0 / 6.0);
    p = __builtin_fma(p, r, 0.5);
    p = __builtin_fma(p, r, 1.0);
    p = __builtin_fma(p, r, 1.0);
    return __builtin_amdgcn_ldexp(p, (int)k);
}
struct erf_cell { // erf(r), erf'(r)
    double v, d;
};
DPX_D double bs_erf(double x, const erf_cell *table) // finite x; table: erf_fine_table or a copy of it in LDS
{
    constexpr double magic = 26388279066624.0; // 1.5 * 2^44: one unit in the last place is 2^-8
    const double a = __builtin_fabs(x);
    const double ac = a < 6.0 ? a : 6.0;
    const double tm = ac + magic;
    const double r = tm - magic; // ac rounded to a multiple of 1/256
    const double d = ac - r;     // |d| <= 1/512, exact
    const int i = (int)(uint32_t)__builtin_bit_cast(uint64_t, tm); // low mantissa bits: 256 r (at most 1536)
    const double r2 = r * r;
    const double c3 = __builtin_fma(r2, 2.0 / 3.0, -1.0 / 3.0);
    const double c4 = r * __builtin_fma(r2, -1.0 / 3.0, 0.5);
    const double c5 = __builtin_fma(r2, __builtin_fma(r2, 4.0 / 30.0, -12.0 / 30.0), 0.1);
    double p = __builtin_fma(c5, d, c4);
    p = __builtin_fma(p, d, c3);
    p = __builtin_fma(p, d, -r);
    p = __builtin_fma(p, d, 1.0);
    p = p * d;
    const erf_cell cell = table[i];
    const double y = __builtin_fma(cell.d, p, cell.v);
    return __builtin_copysign(y, x);
}
struct BlackScholesFast {
    double mr, sig_sig_two;
    DPX_D static bool normal_positive(double v)
    {
        return __builtin_amdgcn_class(v, 0x100); // positive normal
    }
    // Inputs the short routines are good for: p / s and z = 2 vol^2 t positive normal numbers (then p
    // and s are finite and not zero and t is a positive number) and exp's argument inside its range.
    DPX_D bool takes(double t, double q) const
    {
        return normal_positive(q) && normal_positive(t * sig_sig_two) && __builtin_fabs(t * mr) < 700.0;
    }
    DPX_D void price(double p, double s, double t, double q, const erf_cell *table, double &call, double &put) const
    {
        constexpr double ln2_hi = 6.93147180369123816490e-01, ln2_lo = 1.90821492927058770002e-10;
        double dk, f, hfsq, tail;
        log_f64_parts(q, dk, f, hfsq, tail);
        const double in = __builtin_fma(dk, ln2_lo, tail);
        const double a = __builtin_fma(dk, ln2_hi, -((hfsq - in) - f));
        const double b = t * mr;
        const double z = t * sig_sig_two;
        const double c = 0.25 * z;
        const double y = bs_rsqrt(z);
        const double w1 = (a - b + c) * y;
        const double w2 = (a - b - c) * y;
        const double d1 = __builtin_fma(0.5, bs_erf(w1, table), 0.5);
        const double d2 = __builtin_fma(0.5, bs_erf(w2, table), 0.5);
        const double se = bs_exp(b) * s;
        call = p * d1 - se * d2;
        put = call - p + se;
    }
};

template <class T>
__global__ __launch_bounds__(256) void black_scholes_kernel(BlackScholesFn<T> fn, const T *price, const T *strike,
                                                            const T *t, T *call, T *put, int64_t n)
{
    constexpr int E = 16 / sizeof(T);
    const int64_t base = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * E;
    if (base + E <= n) {
        pack<T, E> p = load_pack<T, E>(price + base), s = load_pack<T, E>(strike + base),
                   tt = load_pack<T, E>(t + base), c, q;
#pragma unroll
        for (int e = 0; e < E; ++e) fn.price(p.v[e], s.v[e], tt.v[e], c.v[e], q.v[e]);
        store_pack<T, E>(call + base, c);
        store_pack<T, E>(put + base, q);
    }
    else {
        for (int64_t i = base; i < n; ++i) fn.price(price[i], strike[i], t[i], call[i], put[i]);
    }
}

// The kernel for doubles.  The erf table lives in LDS: a gather of 64 different 16-byte cells costs
// a CU's vector memory pipeline 41 clocks from a 24 KB table in global memory (cached) and its LDS
// 14 clocks (measured on MI355X), and with four gathers per wave the memory pipeline was as busy
// with them as with the five streams.  A block of 512 threads prices 4096 options, so that the copy
// of the table (24 KB from L2) is small beside the 160 KB the block streams; every thread asks for
// its four packs of each input first, the copy of the table runs while they are on their way.
// Measured on one box, 2^26 options: this shape 0.46 ms; blocks of 256 x 4, 512 x 2, 512 x 8 and
// 1024 x 4 options 0.48 to 0.55 ms; persistent blocks that walk the options with a grid stride and
// load one chunk ahead 0.49 ms; one wave per block with the table in global memory 0.54 ms; the
// long routines alone 0.57 ms; a plain copy of the same five streams 0.42 to 0.44 ms.
// The last block prices the options past the last full chunk one by one.
// PART selects what the kernel does, for measurement: BS_WHOLE is the product kernel; BS_ARITHMETIC prices options
// made up from the thread's index and stores nothing (the instruction stream without the five memory streams);
// BS_STREAMS loads and stores as the product does and prices nothing (the five streams without the arithmetic).
constexpr int BS_BLOCK = 512, BS_PACKS = 4;
enum { BS_WHOLE = 0, BS_ARITHMETIC = 1, BS_STREAMS = 2 };
template <int PART>
__global__ __launch_bounds__(BS_BLOCK) void black_scholes_f64_kernel(BlackScholesFn<double> fn, const double *price,
                                                                     const double *strike, const double *t, double *call,
                                                                     double *put, int64_t n, int64_t nfull)
{
    constexpr int E = 2, U = BS_PACKS;
    constexpr int64_t CHUNK = (int64_t)BS_BLOCK * E * U; // a thread's packs of one chunk are BS_BLOCK * E options apart
    __shared__ erf_cell table[ERF_FINE_N];
    const int64_t chunk = blockIdx.x;
    if (chunk >= nfull) {
        for (int64_t i = nfull * CHUNK + threadIdx.x; i < n; i += BS_BLOCK)
            fn.price(price[i], strike[i], t[i], call[i], put[i]);
        return;
    }
    pack<double, E> p[U], s[U], tt[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int64_t base = chunk * CHUNK + (u * BS_BLOCK + threadIdx.x) * E;
        if constexpr (PART == BS_ARITHMETIC) {
#pragma unroll
            for (int e = 0; e < E; ++e) { // price and strike in [10, 50), maturity in [1, 2), from the index
                const double f = (double)((base + e) & 1023) * (1.0 / 1024);
                p[u].v[e] = 10.0 + 40.0 * f, s[u].v[e] = 50.0 - 40.0 * f, tt[u].v[e] = 1.0 + f;
            }
        }
        else
            p[u] = load_pack<double, E>(price + base), s[u] = load_pack<double, E>(strike + base),
            tt[u] = load_pack<double, E>(t + base);
    }
    if constexpr (PART == BS_STREAMS) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t base = chunk * CHUNK + (u * BS_BLOCK + threadIdx.x) * E;
            pack<double, E> c, q;
#pragma unroll
            for (int e = 0; e < E; ++e) c.v[e] = p[u].v[e] + s[u].v[e], q.v[e] = tt[u].v[e] * s[u].v[e];
            store_pack<double, E>(call + base, c);
            store_pack<double, E>(put + base, q);
        }
        return;
    }
    for (int i = threadIdx.x; i < ERF_FINE_N; i += BS_BLOCK) table[i] = erf_cell{erf_fine_table[i][0], erf_fine_table[i][1]};
    __syncthreads();
    const BlackScholesFast fast{fn.mr, fn.sig_sig_two};
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int64_t base = chunk * CHUNK + (u * BS_BLOCK + threadIdx.x) * E;
        pack<double, E> c, q;
        double quot[E];
        bool ok = true;
#pragma unroll
        for (int e = 0; e < E; ++e) {
            quot[e] = p[u].v[e] * bs_rcp(s[u].v[e]);
            ok = ok && fast.takes(tt[u].v[e], quot[e]);
        }
        // the short routines when every option of the wave qualifies
        if (__builtin_amdgcn_ballot_w64(!ok) == 0) {
#pragma unroll
            for (int e = 0; e < E; ++e) fast.price(p[u].v[e], s[u].v[e], tt[u].v[e], quot[e], table, c.v[e], q.v[e]);
        }
        else {
#pragma unroll
            for (int e = 0; e < E; ++e) fn.price(p[u].v[e], s[u].v[e], tt[u].v[e], c.v[e], q.v[e]);
        }
        if constexpr (PART == BS_ARITHMETIC) {
            // never true for prices (a call is at least 0): keeps the arithmetic without a memory stream
            if (c.v[0] + q.v[0] + c.v[1] + q.v[1] == -12345.678) store_pack<double, E>(call, c);
        }
        else {
            store_pack<double, E>(call + base, c);
            store_pack<double, E>(put + base, q);
        }
    }
}

} // namespace dpx
