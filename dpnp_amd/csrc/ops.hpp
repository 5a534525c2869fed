// Per-op device functors and their dtype maps.
//
// Each op struct gives, for an input element type T (binary ops: both inputs
// of type T): `ok<T>` whether a kernel exists, `out<T>` the result element
// type, and `apply` on values.  The maps restate the *OutputType structs of
// libtensor/include/kernels/elementwise_functions/<op>.hpp; everything not
// listed there is reached through casts chosen by the Python layer.
#pragma once
#include "types.hpp"
#include "erf_table.hpp"
#include "pow_log_table.hpp"
#include "powf_log_table.hpp"

namespace dpx {

// A constant kept in scalar registers: an fma then takes it as its scalar operand.  Without this the
// compiler materialises every 64-bit literal of a Horner chain in vector registers (two v_mov_b32)
// in order to use the accumulating form of fma, which costs a quarter of the chain's issue slots.
DPX_D double scalar_const(double c)
{
    asm("" : "+s"(c));
    return c;
}
// ---- complex arithmetic -------------------------------------------------------
template <class R> DPX_HD cplx<R> operator+(cplx<R> a, cplx<R> b) { return {a.re + b.re, a.im + b.im}; }
template <class R> DPX_HD cplx<R> operator-(cplx<R> a, cplx<R> b) { return {a.re - b.re, a.im - b.im}; }
template <class R> DPX_HD cplx<R> operator-(cplx<R> a) { return {-a.re, -a.im}; }
template <class R> DPX_HD cplx<R> operator*(cplx<R> a, cplx<R> b)
{
    return {a.re * b.re - a.im * b.im, a.re * b.im + a.im * b.re};
}
template <class R> DPX_HD cplx<R> operator/(cplx<R> a, cplx<R> b)
{
    // Smith's algorithm (what NumPy uses): no spurious overflow in |b|^2
    R abr = b.re < 0 ? -b.re : b.re, abi = b.im < 0 ? -b.im : b.im;
    if (abr >= abi) {
        if (abr == 0 && abi == 0) return {a.re / abr, a.im / abr};
        R rat = b.im / b.re, scl = R(1) / (b.re + b.im * rat);
        return {(a.re + a.im * rat) * scl, (a.im - a.re * rat) * scl};
    }
    R rat = b.re / b.im, scl = R(1) / (b.re * rat + b.im);
    return {(a.re * rat + a.im) * scl, (a.im * rat - a.re) * scl};
}
template <class R> DPX_HD bool operator==(cplx<R> a, cplx<R> b) { return a.re == b.re && a.im == b.im; }
template <class R> DPX_HD bool operator!=(cplx<R> a, cplx<R> b) { return !(a == b); }

template <class T> DPX_HD bool isnan_(T x)
{
    if constexpr (is_cplx_v<T>) return (x.re != x.re) || (x.im != x.im);
    else if constexpr (is_fp_v<T>) return x != x;
    else return false;
}

// ordering of complex numbers: libtensor/include/utils/math_utils.hpp:43-95
template <class R> DPX_HD bool c_less(cplx<R> a, cplx<R> b)
{
    return (a.re == b.re) ? (a.im < b.im) : (a.re < b.re && !isnan_(a.im) && !isnan_(b.im));
}
template <class R> DPX_HD bool c_greater(cplx<R> a, cplx<R> b)
{
    return (a.re == b.re) ? (a.im > b.im) : (a.re > b.re && !isnan_(a.im) && !isnan_(b.im));
}
template <class R> DPX_HD bool c_less_eq(cplx<R> a, cplx<R> b)
{
    return (a.re == b.re) ? (a.im <= b.im) : (a.re < b.re && !isnan_(a.im) && !isnan_(b.im));
}
template <class R> DPX_HD bool c_greater_eq(cplx<R> a, cplx<R> b)
{
    return (a.re == b.re) ? (a.im >= b.im) : (a.re > b.re && !isnan_(a.im) && !isnan_(b.im));
}

// NaN-propagating extrema: Maximum / Minimum, libtensor/include/utils/sycl_utils.hpp:332-376
// and max_complex / min_complex, math_utils.hpp:97-127
template <class T> DPX_HD T max_nan(T x, T y)
{
    if constexpr (is_cplx_v<T>) return (isnan_(x.re) || isnan_(x.im) || c_greater(x, y)) ? x : y;
    else if constexpr (is_fp_v<T>) return (x != x || x > y) ? x : y;
    else if constexpr (std::is_same_v<T, bool>) return x || y;
    else return (x > y) ? x : y;
}
template <class T> DPX_HD T min_nan(T x, T y)
{
    if constexpr (is_cplx_v<T>) return (isnan_(x.re) || isnan_(x.im) || c_less(x, y)) ? x : y;
    else if constexpr (is_fp_v<T>) return (x != x || x < y) ? x : y;
    else if constexpr (std::is_same_v<T, bool>) return x && y;
    else return (x < y) ? x : y;
}

// ---- math on real fp types (half computes in float) -----------------------------
// Natural logarithm of a double.  x = 2^k (1 + f) with sqrt(1/2) <= 1 + f < sqrt(2);
// s = f / (2 + f); log(1 + f) = f - (f^2/2 - s (f^2/2 + R(s^2))) with the degree-14 minimax
// polynomial R of the classic fdlibm log (Sun Microsystems' e_log.c: coefficients Lg1..Lg7 and
// the split of ln 2 into a part whose product with k is exact and a tail).  The quotient comes
// from the hardware reciprocal and two Newton steps: s only multiplies terms of order f^2, so
// its last bits do not reach the result.  Measured on MI355X against a long double reference
// over 4 M arguments (all binades, dense around 1): error below 0.82 ULP (the device
// library's: 0.63 ULP); 2^27 elements take 0.37 ms instead of 0.57 ms.
// k and log(m) = hi + lo for x = 2^k m, sqrt(1/2) <= m < sqrt(2) (x > 0 and finite)
// log(1 + f) = f - hfsq + tail for 1 + f in [sqrt(1/2), sqrt(2))
DPX_D void log_f64_series(double f, double &hfsq, double &tail)
{
    constexpr double Lg1 = 6.666666666666735130e-01, Lg2 = 3.999999999940941908e-01,
                     Lg3 = 2.857142874366239149e-01, Lg4 = 2.222219843214978396e-01,
                     Lg5 = 1.818357216161805012e-01, Lg6 = 1.531383769920937332e-01,
                     Lg7 = 1.479819860511658591e-01;
    const double d = 2.0 + f;
    double rc = __builtin_amdgcn_rcp(d);
    rc = __builtin_fma(__builtin_fma(-d, rc, 1.0), rc, rc);
    rc = __builtin_fma(__builtin_fma(-d, rc, 1.0), rc, rc);
    const double s = f * rc, z = s * s, w = z * z;
    const double t1 = w * __builtin_fma(w, __builtin_fma(w, Lg6, Lg4), Lg2);
    const double p2 = __builtin_fma(w, __builtin_fma(w, __builtin_fma(w, Lg7, Lg5), Lg3), Lg1);
    const double R = __builtin_fma(z, p2, t1);
    hfsq = (0.5 * f) * f;
    tail = s * (hfsq + R);
}
// k and m - 1 for x = 2^k m, sqrt(1/2) <= m < sqrt(2) (x > 0 and finite)
DPX_D void log_f64_split(double x, double &dk, double &f)
{
    double m = __builtin_amdgcn_frexp_mant(x); // [0.5, 1), subnormals included
    int e = __builtin_amdgcn_frexp_exp(x);
    const bool low = m < 0.70710678118654752440;
    m = low ? m * 2.0 : m;
    e = low ? e - 1 : e;
    f = m - 1.0;
    dk = (double)e;
}
DPX_D void log_f64_parts(double x, double &dk, double &f, double &hfsq, double &tail)
{
    log_f64_split(x, dk, f);
    log_f64_series(f, hfsq, tail); // log(m) = f - hfsq + tail
}
DPX_D double log_special(double x, double r)
{
    r = (x == 0.0) ? -__builtin_inf() : r;
    r = (x < 0.0) ? __builtin_nan("") : r;
    return !(x < __builtin_inf()) ? x : r; // +inf and NaN
}
DPX_D double log_f64(double x)
{
    constexpr double ln2_hi = 6.93147180369123816490e-01, ln2_lo = 1.90821492927058770002e-10;
    double dk, f, hfsq, tail;
    log_f64_parts(x, dk, f, hfsq, tail);
    const double in = __builtin_fma(dk, ln2_lo, tail);
    const double r = __builtin_fma(dk, ln2_hi, -((hfsq - in) - f));
    return log_special(x, r);
}
// log2 and log10 of a double from the same parts: log(m) times the constant (split in two) plus k
// (log2) or k log10(2).  Exact for powers of two (log2), within 1.6 ULP elsewhere; eleven vector
// instructions on top of log's 48 per element, which keeps the kernel at the HBM rate (the device
// library's routines, and a variant of this one that carried log(m) as a double-double for 0.7 ULP,
// run at 50-60 % of it).
DPX_D double log_scaled_f64(double x, double c_hi, double c_lo, double k_hi, double k_lo)
{
    double dk, f, hfsq, tail;
    log_f64_parts(x, dk, f, hfsq, tail);
    const double lm = f - (hfsq - tail);
    const double lo = __builtin_fma(dk, k_lo, lm * c_lo);
    const double r = __builtin_fma(lm, c_hi, dk * k_hi) + lo; // dk * k_hi is exact: k_hi has few significant bits
    return log_special(x, r);
}
DPX_D double log2_f64(double x)
{
    return log_scaled_f64(x, 1.44269504088896338700e+00, 2.03552737409310331e-17, 1.0, 0.0);
}
DPX_D double log10_f64(double x)
{
    // log10(2) split: the high part has its low 32 bits clear
    return log_scaled_f64(x, 4.34294481903251816668e-01, 1.09831965021676510e-17, 3.01029995663611771306e-01,
                          3.69423907715893078616e-13);
}
// n / d for doubles of moderate size through the hardware reciprocal: one Newton step on it (a relative error e of
// the reciprocal leaves e^2 in the corrected quotient, so 2^-40 after the step is plenty) and one correction of
// the quotient by its exact remainder (6 instructions, within 0.51 ULP; the IEEE division sequence takes 25).
// Not for results or divisors near the ends of the exponent range.
DPX_D double div_f64_fast(double n, double d)
{
    double r = __builtin_amdgcn_rcp(d);
    r = __builtin_fma(__builtin_fma(-d, r, 1.0), r, r);
    const double q = n * r;
    return __builtin_fma(__builtin_fma(-d, q, n), r, q);
}
template <class R> DPX_D R div_moderate(R n, R d)
{
    if constexpr (std::is_same_v<R, double>) return div_f64_fast(n, d);
    else return n / d;
}

// log(y + e) for a positive normal y and |e| far below an ULP of y (the low part of a two-double argument):
// the series of log_f64 with e / y among its low-order terms.  `extra` = e / y, to the accuracy the result needs.
DPX_D double log_f64_two(double y, double extra)
{
    constexpr double ln2_hi = 6.93147180369123816490e-01, ln2_lo = 1.90821492927058770002e-10;
    double dk, f, hfsq, tail;
    log_f64_parts(y, dk, f, hfsq, tail);
    const double in = __builtin_fma(dk, ln2_lo, extra) + tail;
    return __builtin_fma(dk, ln2_hi, -((hfsq - in) - f));
}
// log1p after fdlibm's s_log1p.c, without its branches: between sqrt(1/2) - 1 and sqrt(2) - 1 the series of log
// takes x itself (k = 0, nothing is rounded); elsewhere it takes u = 1 + x rounded, and the rounding error c of that
// sum over u joins the low-order terms (there the result is at least 0.29 in magnitude and c/u at most 2^-53, so
// the float reciprocal is more than enough).  60 vector instructions and no look-up: a form through a table
// logarithm (pow's table: 35 and a 16-byte gather per element, plus the correction's full-precision reciprocal) was
// 5 to 12 % slower.  Host check against long double over 3.6e7 arguments (|x| < 1, tiny and subnormal x, x up to
// 2^1023, x next to -1 and around both switches, the float reciprocal off by an ULP either way): mean 0.22,
// worst 0.89 ULP.
DPX_D double log1p_f64(double x)
{
    constexpr double ln2_hi = 6.93147180369123816490e-01, ln2_lo = 1.90821492927058770002e-10;
    const double u = 1.0 + x;
    const bool mid = x > -0.2928932188134525 && x < 0.4142135623730950;
    double dk, f, hfsq, tail;
    log_f64_split(u, dk, f);
    f = mid ? x : f;
    dk = mid ? 0.0 : dk;
    double c = (x < 1.0) ? x - (u - 1.0) : 1.0 - (u - x);
    c = mid ? 0.0 : c * (double)__builtin_amdgcn_rcpf((float)u);
    log_f64_series(f, hfsq, tail);
    const double in = __builtin_fma(dk, ln2_lo, c) + tail;
    const double r = __builtin_fma(dk, ln2_hi, -((hfsq - in) - f));
    return (x == 0.0) ? x : log_special(u, r); // (-0.0 stays; u = 0, u < 0, +inf, NaN as for log)
}
// ---- fp32 log1p and inverse hyperbolic functions through double arithmetic ------------------------
// The argument y of the logarithm (1 + x; a + sqrt(a^2 + 1); (1 + a)/(1 - a)) is formed in double, where
// the sums and products of floats are exact or good to 2^-44 with square roots and reciprocals from the
// float hardware seeds and one Newton step; then log y = log(yf) + (y - yf)/yf with yf = y rounded to
// float.  No ranges, no cancellation to guard except next to zero, 30 to 40 vector instructions where the
// float formulas (IEEE sqrt and division, a log1p of their result) took 60.  Host check against long double
// with every seed, log2 and reciprocal off by up to one ULP more than correctly rounded: 3.0 ULP at worst.
// (the hardware's log2 of a normal float times ln 2 split in two; y a positive normal float's worth, not inf)
DPX_D float log_f32_of_f64(double y)
{
    const float yf = (float)y;
    const float dy = (float)(y - (double)yf);
    const float l2 = __builtin_amdgcn_logf(yf);
    const float c = 0x1.62e42ep-1f, cc = 0x1.efa39ep-25f; // ln 2 = c + cc
    const float p = l2 * c;
    float t = __builtin_fmaf(l2, c, -p);
    t = __builtin_fmaf(l2, cc, t);
    t = __builtin_fmaf(dy, __builtin_amdgcn_rcpf(yf), t);
    return p + t;
}
DPX_D double sqrt_f64_seed_f32(double t) // t positive, in the float range
{
    const double r0 = (double)__builtin_amdgcn_rsqf((float)t);
    const double s = t * r0;
    return __builtin_fma(__builtin_fma(-s, s, t), 0.5 * r0, s);
}
DPX_D float log1p_f32(float x)
{
    float r = log_f32_of_f64(1.0 + (double)x);
    r = (__builtin_fabsf(x) < 0x1p-12f) ? __builtin_fmaf(-0.5f * x, x, x) : r; // also keeps -0.0
    r = (x == -1.0f) ? -__builtin_inff() : r; // (below -1: the logarithm of a negative number is NaN)
    return (x == __builtin_inff()) ? x : r;
}

// ---- fp64 inverse hyperbolic functions: the logarithm's argument as a sum of two doubles --------------
//   asinh a = log(a + sqrt(a^2 + 1)),  acosh x = log(x + sqrt(x^2 - 1)),  atanh a = log((1 + a)/(1 - a))/2
// with the argument y carried as yhi + ylo (the square with the error of its product, the sum with 1 as an exact
// two-sum, the square root from the hardware estimate with one coupled step and its residual, the quotient with
// its remainder) straight into the logarithm's series: log y = log_f64_two(yhi, ylo / yhi).  No division, no IEEE
// square root (17 fp64-FMA equivalents on this GPU; the estimate and its steps: 10), no log1p wrapper around the
// logarithm, no look-up (the same functions through pow's logarithm table were 5 to 8 % slower).  Host check
// against long double (4e6 arguments per range: ordinary, 2^-60 .. 2^709, next to 0, next to 1, around the switch
// to the series, hardware estimates off by an ULP either way): asinh 0.84, acosh 0.82, atanh 0.90 ULP at worst
// (the fdlibm forms through log1p: 1.69, 1.97, 1.79).
DPX_D void sqrt_f64_two(double thi, double tlo, double &g, double &slo) // sqrt(thi + tlo) = g + slo
{
    const double r0 = __builtin_amdgcn_rsq(thi);
    double h = 0.5 * r0;
    g = thi * r0;
    const double e = __builtin_fma(-h, g, 0.5);
    g = __builtin_fma(g, e, g);
    h = __builtin_fma(h, e, h);
    slo = (__builtin_fma(-g, g, thi) + tlo) * h;
}
// 1 / y to 2^-44 from the float hardware reciprocal (y within the float range)
DPX_D double rcp_f64_seed_f32(double y)
{
    const double rc = (double)__builtin_amdgcn_rcpf((float)y);
    return __builtin_fma(__builtin_fma(-y, rc, 1.0), rc, rc);
}
DPX_D double asinh_f64(double x)
{
    const double a = __builtin_fabs(x);
    const double p = a * a, pe = __builtin_fma(a, a, -p);
    const double thi = 1.0 + p, bb = thi - 1.0, te = (1.0 - (thi - bb)) + (p - bb); // 1 + p = thi + te
    double g, slo;
    sqrt_f64_two(thi, te + pe, g, slo);
    const double yhi = g + a, ylo = (a - (yhi - g)) + slo; // g >= a
    const bool big = a > 0x1p500;                           // a^2 + 1 = a^2 long before: log(2a)
    double r = log_f64_two(big ? a : yhi, big ? 0.0 : ylo * (double)__builtin_amdgcn_rcpf((float)yhi));
    r = big ? r + 0.69314718055994530942 : r;
    r = (a < 0x1p-13) ? __builtin_fma(a * p, -1.0 / 6, a) : r; // also keeps zeros and subnormals
    r = (a == (double)__builtin_inff()) ? a : r;
    return (x != x) ? x : __builtin_copysign(r, x);
}
DPX_D double acosh_f64(double x)
{
    const double p = x * x, pe = __builtin_fma(x, x, -p);
    const double thi = p - 1.0, bb = thi - p, te = (p - (thi - bb)) + (-1.0 - bb); // p - 1 = thi + te
    const double tlo = te + pe;
    double g, slo;
    sqrt_f64_two(thi, tlo, g, slo);
    const bool one = thi + tlo == 0.0; // x = 1: the estimate of 1/sqrt(0) is infinite
    g = one ? 0.0 : g;
    slo = one ? 0.0 : slo;
    const double yhi = x + g, ylo = (g - (yhi - x)) + slo; // x >= g
    const bool big = x > 0x1p500;
    // (next to x = 1 the result is of the order of ylo / yhi's 2^25-fold: the float reciprocal alone is too coarse)
    double r = log_f64_two(big ? x : yhi, big ? 0.0 : ylo * rcp_f64_seed_f32(yhi));
    r = big ? r + 0.69314718055994530942 : r;
    r = (x == (double)__builtin_inff()) ? x : r;
    r = (x < 1.0) ? (double)__builtin_nanf("") : r;
    return (x != x) ? x : r;
}
DPX_D double atanh_f64(double x)
{
    const double a = __builtin_fabs(x);
    const double nhi = 1.0 + a, nlo = a - (nhi - 1.0);   // 1 + a
    const double dhi = 1.0 - a, dlo = (1.0 - dhi) - a;   // 1 - a
    double rc = rcp_f64_seed_f32(dhi);
    rc = __builtin_fma(__builtin_fma(-dhi, rc, 1.0), rc, rc);
    const double qhi = nhi * rc;
    const double qlo = (__builtin_fma(-qhi, dhi, nhi) + __builtin_fma(-qhi, dlo, nlo)) * rc; // the remainder over 1 - a
    double r = 0.5 * log_f64_two(qhi, qlo * (double)__builtin_amdgcn_rcpf((float)qhi));
    r = (a < 0x1p-13) ? __builtin_fma(a * a * a, 1.0 / 3, a) : r; // also keeps zeros and subnormals
    r = (a == 1.0) ? (double)__builtin_inff() : r;
    r = (a > 1.0) ? (double)__builtin_nanf("") : r;
    return (x != x) ? x : __builtin_copysign(r, x);
}
// asinh a = log(a + sqrt(a^2 + 1)), log(a) + ln 2 where a^2 + 1 = a^2 in double; a itself below 2^-12
DPX_D float asinh_f32(float x)
{
    const float a = __builtin_fabsf(x);
    const double ad = (double)a;
    const double s = sqrt_f64_seed_f32(__builtin_fma(ad, ad, 1.0));
    const bool big = a > 0x1p30f;
    float r = log_f32_of_f64(big ? ad : ad + s);
    r = big ? r + 0.69314718055994530942f : r;
    r = (a < 0x1p-12f || a == __builtin_inff()) ? a : r;
    return __builtin_copysignf(r, x); // (NaN has gone through)
}
// acosh x = log(x + sqrt(x^2 - 1)); x^2 - 1 is exact in double
DPX_D float acosh_f32(float x)
{
    const double xd = (double)x;
    const double t = __builtin_fma(xd, xd, -1.0);
    double s = sqrt_f64_seed_f32(t);
    s = (t == 0.0) ? 0.0 : s;
    const bool big = x > 0x1p30f;
    float r = log_f32_of_f64(big ? xd : xd + s);
    r = big ? r + 0.69314718055994530942f : r;
    r = (x == __builtin_inff()) ? x : r;
    return (x < 1.0f) ? __builtin_nanf("") : r; // NaN goes through
}
// atanh a = log((1 + a)/(1 - a))/2; numerator and denominator are exact in double
DPX_D float atanh_f32(float x)
{
    const float a = __builtin_fabsf(x);
    const double ad = (double)a, n = 1.0 + ad, d = 1.0 - ad;
    const double r0 = (double)__builtin_amdgcn_rcpf((float)d);
    const double r1 = __builtin_fma(__builtin_fma(-d, r0, 1.0), r0, r0);
    float r = 0.5f * log_f32_of_f64(n * r1); // (good to 2^-44; beyond 1 the quotient is negative: NaN)
    r = (a < 0x1p-12f) ? a : r;
    r = (a == 1.0f) ? __builtin_inff() : r;
    return __builtin_copysignf(r, x);
}

// Hyperbolic functions from exp and expm1 (the forms of fdlibm's s_tanh.c, e_sinh.c, e_cosh.c):
//   tanh a = t / (t + 2), t = expm1(2a);   sinh a = (t + t/(t+1))/2, t = expm1(a);
//   cosh a = (e + 1/e)/2, e = exp(a), for a = |x|; where exp(a) would overflow and the function does
// not yet, (exp(a/2)/2) exp(a/2).
template <class R, class EXPM1> DPX_D R tanh_via(R x, EXPM1 expm1_fn)
{
    const R a = x < R(0) ? -x : x;
    const R big = std::is_same_v<R, double> ? R(22) : R(10);
    const R t = expm1_fn(a + a);
    R r = div_moderate<R>(t, t + R(2));
    r = (a > big) ? R(1) : r;
    r = (a == R(0)) ? a : r;
    return (x != x) ? x : __builtin_copysign(r, x);
}
template <class R, class EXP, class EXPM1> DPX_D R sinh_via(R x, EXP exp_fn, EXPM1 expm1_fn)
{
    const R a = x < R(0) ? -x : x;
    const R over = std::is_same_v<R, double> ? R(709) : R(88); // exp(a) and expm1(a) are finite up to here
    const R t = expm1_fn(a);
    const R q = div_moderate<R>(t, t + R(1));
    R r = R(0.5) * ((a < R(1)) ? R(2) * t - t * q : t + q);
    if (a > over) { // rare: the band where sinh is finite and exp is not, and beyond
        asm volatile("" ::: "memory"); // (not to be executed speculatively)
        const R w = exp_fn(R(0.5) * a);
        r = (R(0.5) * w) * w;
    }
    r = (a == R(0)) ? a : r;
    return (x != x) ? x : __builtin_copysign(r, x);
}
template <class R, class EXP> DPX_D R cosh_via(R x, EXP exp_fn)
{
    const R a = x < R(0) ? -x : x;
    const R over = std::is_same_v<R, double> ? R(709) : R(88);
    const R e = exp_fn(a);
    R r = R(0.5) * e + R(0.5) / e; // NaN goes through exp
    if (a > over) {
        asm volatile("" ::: "memory");
        const R w = exp_fn(R(0.5) * a);
        r = (R(0.5) * w) * w;
    }
    return r;
}
DPX_D double tanh_f64(double x) { return tanh_via<double>(x, [](double v) { return ::expm1(v); }); }
DPX_D double sinh_f64(double x)
{
    return sinh_via<double>(x, [](double v) { return ::exp(v); }, [](double v) { return ::expm1(v); });
}
DPX_D double cosh_f64(double x) { return cosh_via<double>(x, [](double v) { return ::exp(v); }); }
// fp32 sinh: the odd Taylor polynomial to a^11 below 1 (remainder 1e-10), (e - 1/e)/2 above, where 1/e is at
// most 0.14 e and the hardware reciprocal's ULP does not show; cosh: (e + 1/e)/2.  One expf each: sinh_via's
// expm1f and the second expf of the overflow band (executed for every element when left to the compiler) made
// 55 and 37 vector instructions per element, against 10 for expf.
DPX_D float sinh_f32(float x)
{
    const float a = __builtin_fabsf(x);
    const float z = a * a;
    float p = __builtin_fmaf(z, 1.0f / 39916800, 1.0f / 362880);
    p = __builtin_fmaf(z, p, 1.0f / 5040);
    p = __builtin_fmaf(z, p, 1.0f / 120);
    p = __builtin_fmaf(z, p, 1.0f / 6);
    p = __builtin_fmaf(a * z, p, a);
    const float e = ::expf(a);
    float r = __builtin_fmaf(0.5f, e, -0.5f * __builtin_amdgcn_rcpf(e));
    r = (a < 1.0f) ? p : r; // (NaN takes the other side)
    if (a > 88.0f) { // rare: the band where sinh is finite and exp is not, and beyond
        asm volatile("" ::: "memory"); // (not to be executed speculatively)
        const float w = ::expf(0.5f * a);
        r = (0.5f * w) * w;
    }
    return (x != x) ? x : __builtin_copysignf(r, x);
}
DPX_D float cosh_f32(float x)
{
    const float a = __builtin_fabsf(x);
    const float e = ::expf(a);
    float r = __builtin_fmaf(0.5f, e, 0.5f * __builtin_amdgcn_rcpf(e)); // NaN goes through exp
    if (a > 88.0f) {
        asm volatile("" ::: "memory");
        const float w = ::expf(0.5f * a);
        r = (0.5f * w) * w;
    }
    return r;
}

// fp64 erf from a table of erf(r) and erf'(r) at r = i/128 and the Taylor series of erf about r:
//   erf(r + d) = erf(r) + erf'(r) (d - r d^2 + (2r^2-1)/3 d^3 - r(2r^2-3)/6 d^4 + (4r^4-12r^2+3)/30 d^5
//                                  - r(4r^4-20r^2+15)/90 d^6 + (8r^6-60r^4+90r^2-15)/630 d^7),
// r = floor(128 |x|)/128, 0 <= d < 1/128 (d is exact and not negative: the correction adds to erf(r),
// nothing cancels).  About 40 vector instructions and one 16-byte table read
// where the device library's erf takes about 100 when the lanes of a wave need different ranges;
// measured error against an 80-bit evaluation over 4e7 arguments: 1.62 ULP at most.  |x| >= 6 gives
// +-1 (1 - erf(6) < 2^-54), NaN gives NaN.
DPX_D double erf_f64(double x)
{
    const double a = __builtin_fabs(x);
    const double ac = a < 6.0 ? a : 6.0; // also for NaN: the index stays inside the table
    const double ri = __builtin_floor(ac * 128.0);
    const int i = (int)ri;
    const double r = ri * 0.0078125;
    const double d = ac - r;
    const double r2 = r * r;
    const double c3 = __builtin_fma(r2, 2.0 / 3.0, -1.0 / 3.0);
    const double c4 = r * __builtin_fma(r2, -1.0 / 3.0, 0.5);
    const double c5 = __builtin_fma(r2, __builtin_fma(r2, 4.0 / 30.0, -12.0 / 30.0), 0.1);
    const double c6 = -r * __builtin_fma(r2, __builtin_fma(r2, 4.0 / 90.0, -20.0 / 90.0), 15.0 / 90.0);
    const double c7 = __builtin_fma(r2, __builtin_fma(r2, __builtin_fma(r2, 8.0 / 630.0, -60.0 / 630.0), 90.0 / 630.0),
                                    -15.0 / 630.0);
    double p = __builtin_fma(c7, d, c6);
    p = __builtin_fma(p, d, c5);
    p = __builtin_fma(p, d, c4);
    p = __builtin_fma(p, d, c3);
    p = __builtin_fma(p, d, -r);
    p = __builtin_fma(p, d, 1.0);
    p = p * d;
    const double y = __builtin_fma(erf_table[i][1], p, erf_table[i][0]);
    return (x != x) ? x : __builtin_copysign(y, x);
}

// ---- fp64 sin, cos ---------------------------------------------------------------------------------
// For |x| < 1e6 the argument is reduced by n = rint(x 2/pi) with pi/2 in three 53-bit parts, each
// subtracted by one fma: x - n P1 is exact (fewer than 53 significant bits are left), the next two
// steps round once each, also next to a multiple of pi/2 where the first difference is tiny.  Both
// fdlibm kernels (k_sin.c, k_cos.c: S1..S6, C1..C6) are evaluated and the quadrant picks one: about 45
// vector instructions per element, against 65-75 executed in the device library's routine (67 % of the
// HBM rate on 2^26 doubles).  Larger arguments, infinities and NaN go to the device library.
// Measured against an 80-bit evaluation over 4e7 arguments (dense below 50, up to 1e6, every small
// binade, neighbourhoods of multiples of pi/2): sin 1.50, cos 1.51 ULP.
DPX_D int sincos_f64(double x, double &s, double &c)
{
    auto K = [](double v) { return scalar_const(v); };
    constexpr double P1 = 0x1.921fb54442d18p+0, P2 = 0x1.1a62633145c07p-54, P3 = -0x1.f1976b7ed8fbcp-110,
                     TWO_OVER_PI = 0x1.45f306dc9c883p-1;
    constexpr double S1 = -1.66666666666666324348e-01, S2 = 8.33333333332248946124e-03,
                     S3 = -1.98412698298579493134e-04, S4 = 2.75573137070700676789e-06,
                     S5 = -2.50507602534068634195e-08, S6 = 1.58969099521155010221e-10;
    constexpr double C1 = 4.16666666666666019037e-02, C2 = -1.38888888888741095749e-03,
                     C3 = 2.48015872894767294178e-05, C4 = -2.75573143513906633035e-07,
                     C5 = 2.08757232129817482790e-09, C6 = -1.13596475577881948265e-11;
    const double n = __builtin_rint(x * K(TWO_OVER_PI));
    double r = __builtin_fma(-n, K(P1), x);
    r = __builtin_fma(-n, K(P2), r);
    r = __builtin_fma(-n, K(P3), r);
    const double z = r * r;
    double ps = __builtin_fma(z, K(S6), K(S5));
    ps = __builtin_fma(z, ps, K(S4));
    ps = __builtin_fma(z, ps, K(S3));
    ps = __builtin_fma(z, ps, K(S2));
    ps = __builtin_fma(z, ps, K(S1));
    s = __builtin_fma(z * r, ps, r);
    double pc = __builtin_fma(z, K(C6), K(C5));
    pc = __builtin_fma(z, pc, K(C4));
    pc = __builtin_fma(z, pc, K(C3));
    pc = __builtin_fma(z, pc, K(C2));
    pc = __builtin_fma(z, pc, K(C1));
    const double hz = 0.5 * z, w = 1.0 - hz;
    c = w + (((1.0 - w) - hz) + z * (z * pc));
    return (int)n;
}
constexpr double TRIG_FAST_LIMIT = 1e6; // n stays below 2^20
// (the *_below_limit forms: straight-line code, valid for |x| < TRIG_FAST_LIMIT, anything elsewhere)
DPX_D double sin_f64_below_limit(double x)
{
    double s, c;
    const int q = sincos_f64(x, s, c);
    double v = (q & 1) ? c : s;
    v = (q & 2) ? -v : v;
    return __builtin_fabs(x) < 0x1p-27 ? x : v; // sin x = x to the last bit, and -0 stays -0
}
DPX_D double cos_f64_below_limit(double x)
{
    double s, c;
    const int q = sincos_f64(x, s, c);
    const double v = (q & 1) ? s : c;
    return ((q + 1) & 2) ? -v : v;
}
DPX_D double sin_f64(double x)
{
    if (!(__builtin_fabs(x) < TRIG_FAST_LIMIT)) return ::sin(x);
    return sin_f64_below_limit(x);
}
DPX_D double cos_f64(double x)
{
    if (!(__builtin_fabs(x) < TRIG_FAST_LIMIT)) return ::cos(x);
    return cos_f64_below_limit(x);
}

// sin and cos of one argument from one reduction (the complex functions need both)
DPX_D void sincos_both_f64(double x, double &sn, double &cs)
{
    const double a = __builtin_fabs(x);
    if (!(a < TRIG_FAST_LIMIT)) {
        // (a statement the compiler may not execute speculatively: without it both device-library routines, about
        // 160 vector instructions, were evaluated for every element ahead of this test and their results selected)
        asm volatile("" ::: "memory");
        sn = ::sin(x);
        cs = ::cos(x);
        return;
    }
    double s, c;
    const int q = sincos_f64(x, s, c);
    double vs = (q & 1) ? c : s;
    vs = (q & 2) ? -vs : vs;
    sn = a < 0x1p-27 ? x : vs;
    const double vc = (q & 1) ? s : c;
    cs = ((q + 1) & 2) ? -vc : vc;
}

// ---- fp64 tan ----------------------------------------------------------------------------------------
// For |x| < 1e6: x = n pi/2 + r as for sin and cos, with r carried as a sum of two doubles (the product n P2 with the
// error of its rounding, the difference as an exact two-term sum: next to a multiple of pi/2 the result is r or
// -1/r, so r's relative error is the result's); t = tan(r/2) from the fdlibm kernel (k_tan.c: T0..T12, good
// for arguments up to 0.67, here at most pi/8), again as two doubles; then tan r = 2t / (1 - t^2) in even
// quadrants and -(1 - t^2) / 2t in odd ones: one quotient of two-double operands through the hardware reciprocal,
// a Newton step and the exact remainder.  About 60 vector instructions and no branch where the device library's
// routine executes 185 (65 % of the HBM rate on 2^26 doubles).  Host check against an 80-bit evaluation over 4e7
// arguments (dense below 50 and up to 1e6, every small binade, neighbourhoods of multiples of pi/4 down to the
// neighbouring doubles, the reciprocal estimate off by 2^-22): mean 0.19, worst 0.66 ULP.
DPX_D double tan_f64_below_limit(double x)
{
    auto K = [](double v) { return scalar_const(v); };
    constexpr double P1 = 0x1.921fb54442d18p+0, P2 = 0x1.1a62633145c07p-54, P3 = -0x1.f1976b7ed8fbcp-110,
                     TWO_OVER_PI = 0x1.45f306dc9c883p-1;
    constexpr double T0 = 3.33333333333334091986e-01, T1 = 1.33333333333201242699e-01,
                     T2 = 5.39682539762260521377e-02, T3 = 2.18694882948595424599e-02,
                     T4 = 8.86323982359930005737e-03, T5 = 3.59207910759131235356e-03,
                     T6 = 1.45620945432529025516e-03, T7 = 5.88041240820264096874e-04,
                     T8 = 2.46463134818469906812e-04, T9 = 7.81794442939557092300e-05,
                     T10 = 7.14072491382608190305e-05, T11 = -1.85586374855275456654e-05,
                     T12 = 2.59073051863633712884e-05;
    const double n = __builtin_rint(x * K(TWO_OVER_PI));
    const double r1 = __builtin_fma(-n, K(P1), x); // exact
    const double p2 = n * K(P2), p2e = __builtin_fma(n, K(P2), -p2);
    const double r0 = r1 - p2;
    double tail = ((r1 - r0) - p2) - p2e;
    tail = 0.5 * __builtin_fma(-n, K(P3), tail);
    const double r = 0.5 * r0;
    const double z = r * r, w = z * z;
    double pr = __builtin_fma(w, K(T11), K(T9));
    pr = __builtin_fma(w, pr, K(T7));
    pr = __builtin_fma(w, pr, K(T5));
    pr = __builtin_fma(w, pr, K(T3));
    pr = __builtin_fma(w, pr, K(T1));
    double pv = __builtin_fma(w, K(T12), K(T10));
    pv = __builtin_fma(w, pv, K(T8));
    pv = __builtin_fma(w, pv, K(T6));
    pv = __builtin_fma(w, pv, K(T4));
    pv = __builtin_fma(w, pv, K(T2));
    pv = z * pv;
    const double s = z * r;
    double rr = __builtin_fma(z, __builtin_fma(s, pr + pv, tail), tail);
    rr = __builtin_fma(K(T0), s, rr);             // tan(r + tail) = r + rr
    const double th = r + rr, tl = (r - th) + rr; // = th + tl, |tl| below half an ULP of th
    const double p = th * th, pe = __builtin_fma(th, th, -p);
    const double uh = 0.5 - 0.5 * p;              // (1 - t^2) / 2 = uh + ul
    const double ul = ((0.5 - uh) - 0.5 * p) - __builtin_fma(th, tl, 0.5 * pe);
    const bool odd = ((int)n & 1) != 0;
    const double nh = odd ? -uh : th, nl = odd ? -ul : tl, dh = odd ? th : uh, dl = odd ? tl : ul;
    double rc = __builtin_amdgcn_rcp(dh);
    rc = __builtin_fma(__builtin_fma(-dh, rc, 1.0), rc, rc);
    const double q = nh * rc;
    const double rem = __builtin_fma(-q, dh, nh) + __builtin_fma(-q, dl, nl);
    const double res = __builtin_fma(rem, rc, q);
    return __builtin_fabs(x) < 0x1p-27 ? x : res; // tan x = x to the last bit, and -0 stays -0
}
DPX_D double tan_f64(double x)
{
    if (!(__builtin_fabs(x) < TRIG_FAST_LIMIT)) {
        asm volatile("" ::: "memory"); // (not to be executed speculatively, see sincos_both_f64)
        return ::tan(x);
    }
    return tan_f64_below_limit(x);
}

// ---- fp64 asin, acos -----------------------------------------------------------------------------
// The device library's routines run at 49 % (asin) and 69 % (acos) of the HBM rate on 2^26 doubles:
// two branches with a full division each and a square root, and a wave whose lanes straddle |x| = 1/2
// runs both.  Here one pass serves every lane: the fdlibm rational R(z) = P(z) / Q(z) (e_asin.c:
// pS0..pS5, qS1..qS4) is evaluated on z = x^2 below 1/2 and on z = (1 - |x|) / 2 above, where
// asin = pi/2 - 2 sqrt(z) (1 + R); the quotient uses the hardware reciprocal with two Newton steps and
// a residual correction (Q lies in [0.5, 1]); the square root is carried as s + slo with the exact
// residual z - s^2 (fma), so s needs no final rounding, and pi/2 - 2 s is an exact two-term sum, which
// replaces fdlibm's truncated-word trick and its third division.
// Measured against an 80-bit evaluation (dense on [-1, 1], towards +-1 down to 1 - 2^-50, around
// +-1/2, every small binade): asin and acos within 1 ULP.
struct AsinParts {
    double R;     // R(z)
    double s, t;  // upper range: sqrt(z) = s + slo and (s + slo)(1 + R) = s + t
    bool upper;   // |x| >= 1/2
};
DPX_D AsinParts asin_parts_f64(double x, double a)
{
    constexpr double pS0 = 1.66666666666666657415e-01, pS1 = -3.25565818622400915405e-01,
                     pS2 = 2.01212532134862925881e-01, pS3 = -4.00555345006794114027e-02,
                     pS4 = 7.91534994289814532176e-04, pS5 = 3.47933107596021167570e-05;
    constexpr double qS1 = -2.40339491173441421878e+00, qS2 = 2.02094576023350569471e+00,
                     qS3 = -6.88283971605453293030e-01, qS4 = 7.70381505559019352791e-02;
    AsinParts r;
    r.upper = a >= 0.5;
    const double zu = 0.5 * (1.0 - a);
    const double z = r.upper ? zu : x * x;
    auto K = [](double c) { return scalar_const(c); };
    double p = __builtin_fma(z, K(pS5), K(pS4));
    p = __builtin_fma(z, p, K(pS3));
    p = __builtin_fma(z, p, K(pS2));
    p = __builtin_fma(z, p, K(pS1));
    p = __builtin_fma(z, p, K(pS0));
    p = z * p;
    double q = __builtin_fma(z, K(qS4), K(qS3));
    q = __builtin_fma(z, q, K(qS2));
    q = __builtin_fma(z, q, K(qS1));
    q = __builtin_fma(z, q, 1.0);
    double rc = __builtin_amdgcn_rcp(q);
    rc = __builtin_fma(__builtin_fma(-q, rc, 1.0), rc, rc);
    rc = __builtin_fma(__builtin_fma(-q, rc, 1.0), rc, rc);
    double R = p * rc;
    R = __builtin_fma(__builtin_fma(-q, R, p), rc, R);
    r.R = R;
    // zu = 0 (x = +-1): the reciprocal square root of the smallest normal number instead, finite, so that
    // s and slo come out as zeros
    const double rs = __builtin_amdgcn_rsq(__builtin_fmax(zu, 0x1p-1022)), h = 0.5 * rs;
    const double s0 = zu * rs;
    const double s = __builtin_fma(__builtin_fma(-s0, s0, zu), h, s0);
    const double slo = __builtin_fma(-s, s, zu) * h;
    r.s = s;
    r.t = slo + __builtin_fma(s, R, slo * R);
    return r;
}
constexpr double PIO2_HI = 0x1.921fb54442d18p+0, PIO2_LO = 0x1.1a62633145c07p-54;
DPX_D double asin_f64(double x)
{
    const double a = __builtin_fabs(x);
    const AsinParts k = asin_parts_f64(x, a);
    const double b = -2.0 * k.s, hi = PIO2_HI + b, lo = (PIO2_HI - hi) + b;
    const double up = __builtin_copysign(hi + (lo + (PIO2_LO - 2.0 * k.t)), x);
    const double r = k.upper ? up : __builtin_fma(x, k.R, x);
    return a <= 1.0 ? r : __builtin_nan("");
}
DPX_D double acos_f64(double x)
{
    const double a = __builtin_fabs(x);
    const AsinParts k = asin_parts_f64(x, a);
    const double low = PIO2_HI - (x - (PIO2_LO - x * k.R));
    const double b = -2.0 * k.s, hi = 2.0 * PIO2_HI + b, lo = (2.0 * PIO2_HI - hi) + b;
    const double neg = hi + (lo + (2.0 * PIO2_LO - 2.0 * k.t)), pos = 2.0 * (k.s + k.t);
    const double r = k.upper ? (x > 0.0 ? pos : neg) : low;
    return a <= 1.0 ? r : __builtin_nan("");
}

#define DPX_FP_FN1(NAME, F32, F64)                                      \
    template <class T> DPX_D T NAME(T x)                                \
    {                                                                   \
        if constexpr (std::is_same_v<T, double>) return F64(x);         \
        else if constexpr (std::is_same_v<T, float>) return F32(x);     \
        else return (T)F32((float)x);                                   \
    }
DPX_FP_FN1(m_sqrt, ::sqrtf, ::sqrt)
DPX_FP_FN1(m_exp, ::expf, ::exp)
DPX_FP_FN1(m_log, ::logf, log_f64)
DPX_FP_FN1(m_erf, ::erff, erf_f64)
DPX_FP_FN1(m_sin, ::sinf, sin_f64)
DPX_FP_FN1(m_cos, ::cosf, cos_f64)
DPX_FP_FN1(m_tan, ::tanf, tan_f64)
DPX_FP_FN1(m_tanh, ::tanhf, tanh_f64)
DPX_FP_FN1(m_exp2, ::exp2f, ::exp2)
DPX_FP_FN1(m_expm1, ::expm1f, ::expm1)
DPX_FP_FN1(m_log2, ::log2f, log2_f64)
DPX_FP_FN1(m_log10, ::log10f, log10_f64)
DPX_FP_FN1(m_log1p, log1p_f32, log1p_f64)
DPX_FP_FN1(m_cbrt, ::cbrtf, ::cbrt)
DPX_FP_FN1(m_floor, ::floorf, ::floor)
DPX_FP_FN1(m_ceil, ::ceilf, ::ceil)
DPX_FP_FN1(m_trunc, ::truncf, ::trunc)
DPX_FP_FN1(m_rint, ::rintf, ::rint)
DPX_FP_FN1(m_asin, ::asinf, asin_f64)
DPX_FP_FN1(m_acos, ::acosf, acos_f64)
DPX_FP_FN1(m_atan, ::atanf, ::atan)
DPX_FP_FN1(m_sinh, sinh_f32, sinh_f64)
DPX_FP_FN1(m_cosh, cosh_f32, cosh_f64)
DPX_FP_FN1(m_asinh, asinh_f32, asinh_f64)
DPX_FP_FN1(m_acosh, acosh_f32, acosh_f64)
DPX_FP_FN1(m_atanh, atanh_f32, atanh_f64)
DPX_FP_FN1(m_erfc, ::erfcf, ::erfc)
DPX_FP_FN1(m_erfcx, ::erfcxf, ::erfcx)
DPX_FP_FN1(m_erfinv, ::erfinvf, ::erfinv)
DPX_FP_FN1(m_erfcinv, ::erfcinvf, ::erfcinv)
DPX_FP_FN1(m_i0, ::cyl_bessel_i0f, ::cyl_bessel_i0)
DPX_FP_FN1(m_sinpi, ::sinpif, ::sinpi)
#undef DPX_FP_FN1
// ---- fp32 pow ------------------------------------------------------------------------------------
// powf of the device library runs at 36 % of the HBM rate (2^27 floats).  For a positive normal base
// and a finite exponent whose result is a normal number, x^y = 2^(y log2 x) is evaluated here in float
// arithmetic with the logarithm carried as a sum of two floats (float instructions issue at twice the rate of
// double ones on this GPU; the same scheme in double precision, 45 instructions, ran at 67 %):
//  * x = 2^k m with m in [sqrt(1/2), sqrt(2)); q = rint(128 / m) from the hardware reciprocal, an integer between
//    90 and 182, so that r = m q / 128 - 1 comes out of one fma without error and |r| < 0.0056;
//  * log2 x = (k - log2(q/128)) + log2(1 + r): the first part from powf_log_table.hpp as {hi, lo} with hi a
//    multiple of 2^-16, so that k + hi is exact; log2(1 + r) = r log2e (1 - r/2 + r^2/3 - r^3/4 + r^4/5) with
//    r log2e as an exact product in two floats; the sum of the large terms keeps its rounding error.  Relative
//    error about 2^-33, also next to x = 1 (q = 128, table entry 0);
//  * t = y log2 x in two floats, n = rint(t), 2^f by the degree-9 Taylor series on |f| <= 1/2, ldexp.
// Host check against double-precision pow over 2.3e7 arguments (every binade of base and result, bases within
// 0.001 of 1 with exponents up to 3e4): mean 0.26, worst 0.97 ULP (0.89 away from such bases).  About 50 float
// instructions, one reciprocal and one 8-byte table look-up per element.  Every other argument (zero, negative,
// subnormal or infinite base, infinite or NaN exponent, results beyond the normal range) goes to powf.
// The short routine: NaN where it does not apply.  Straight-line code, so that the chains of a thread's
// elements interleave when the kernel runs it for all of them before it looks at the NaNs.
DPX_D float pow_f32_fast(float x, float y)
{
    constexpr float LOG2E_HI = 0x1.715476p+0f, LOG2E_LO = 0x1.4ae0cp-26f;
    const uint32_t ix = __float_as_uint(x);
    const int32_t k = (int32_t)(ix - 0x3f3504f3u) >> 23;               // x = 2^k m
    const float m = __uint_as_float(ix - ((uint32_t)k << 23));        // [sqrt(1/2), sqrt(2))
    const float q = __builtin_rintf(128.0f * __builtin_amdgcn_rcpf(m)); // 90 .. 182
    const float r = __builtin_fmaf(m, q * 0.0078125f, -1.0f);           // exact, |r| < 0.0056
    int idx = (int)q - POWF_LOG_Q0;
    idx = idx < 0 ? 0 : (idx > POWF_LOG_N - 1 ? POWF_LOG_N - 1 : idx);  // (arguments the routine is not for)
    const powf_log_entry ent = powf_log_table[idx];
    // log2(1 + r) = r log2e (1 + p), p = -r/2 + r^2/3 - r^3/4 + r^4/5
    float p = __builtin_fmaf(r, 0.2f, -0.25f);
    p = __builtin_fmaf(r, p, 1.0f / 3);
    p = __builtin_fmaf(r, p, -0.5f);
    p = p * r;
    const float h = r * LOG2E_HI, herr = __builtin_fmaf(r, LOG2E_HI, -h);
    const float A = (float)k + ent.hi; // exact
    const float s = A + h;
    const float e = h - (s - A);       // the sum's rounding error: |A| >= |h| or A == 0
    float lo = __builtin_fmaf(h, p, __builtin_fmaf(r, LOG2E_LO, herr));
    lo = (lo + ent.lo) + e;
    // t = y log2 x
    const float thi = y * s;
    const float tlo = __builtin_fmaf(y, lo, __builtin_fmaf(y, s, -thi));
    const float tc = __builtin_fminf(__builtin_fmaxf(thi, -126.0f), 126.0f); // keeps the conversion of n in range
    const float n = __builtin_rintf(tc);
    const float f = (tc - n) + tlo;
    // 2^f = sum (f ln 2)^k / k!
    float g = __builtin_fmaf(f, 0x1.b5253ep-24f, 0x1.62c022p-20f);
    g = __builtin_fmaf(f, g, 0x1.ffcbfcp-17f);
    g = __builtin_fmaf(f, g, 0x1.430912p-13f);
    g = __builtin_fmaf(f, g, 0x1.5d87fep-10f);
    g = __builtin_fmaf(f, g, 0x1.3b2ab6p-7f);
    g = __builtin_fmaf(f, g, 0x1.c6b08ep-5f);
    g = __builtin_fmaf(f, g, 0x1.ebfbep-3f);
    g = __builtin_fmaf(f, g, 0x1.62e43p-1f);
    const float res = __builtin_amdgcn_ldexpf(__builtin_fmaf(f, g, 1.0f), (int)n);
    // +normal base, finite exponent, normal result; NaN in thi fails the comparison
    const bool own = __builtin_amdgcn_classf(x, 0x100) && __builtin_amdgcn_classf(y, 0x1f8) && __builtin_fabsf(thi) < 125.5f;
    return own ? res : __builtin_nanf("");
}
DPX_D float pow_f32(float x, float y)
{
    const float r = pow_f32_fast(x, y);
    return (r != r) ? ::powf(x, y) : r;
}

// ---- fp64 pow ------------------------------------------------------------------------------------
// pow of the device library runs at 37 % of the HBM rate (2^26 doubles, 24 bytes per element).  For a
// positive normal base and a finite exponent whose result is far from the ends of the normal range,
// x^y = exp(y log x) is evaluated here with the logarithm carried as a sum of two doubles:
//  * log x = k ln 2 + log c + log1p(r): the mantissa z of x (scaled into [0.705, 1.41), so that k = 0 around 1)
//    falls into one of 128 intervals (pow_log_table.hpp, 16 bytes per interval: 1/c as a float, log c as a
//    double that is a multiple of 2^-42 and a float for the rest, 1/c chosen so that this rest is below 2^-54);
//    r = z / c - 1 is formed without error as (z * invc - 1) + the product's rounding error (|r| <= 2^-8);
//    k LN2_HI + log c is exact (both multiples of 2^-42), the sums with r and with -r^2/2 keep their
//    rounding errors (the larger term first), and r^3/3 - ... - r^8/8 follows in plain arithmetic.
//    Relative error of the logarithm about 2^-66, also next to x = 1, where the interval around 1 has
//    c = 1 and log c = 0;
//  * t = y log x as a product of the two-term logarithm with y, again in two terms;
//  * exp t = 2^n exp(f), n = rint(t / ln 2), f = t - n ln 2 in two steps plus the low term of t, |f| <= 0.35,
//    Taylor polynomial of degree 13.
// Measured on the host against long double powl over 2.8e7 arguments (ordinary ranges, |t| up to 690, bases
// within 0.03 and within a few thousand ULP of 1 with huge exponents, every binade, interval edges, integer
// exponents): mean 0.26, worst 1.71 ULP.  About 85 vector instructions and one 16-byte table look-up per element.
// Straight-line code: NaN where it does not apply (pow_f64 then asks the device library).
DPX_D double pow_f64_fast(double x, double y)
{
    auto K = [](double v) { return scalar_const(v); };
    constexpr double LN2_HI = 0x1.62e42fefa3800p-1, LN2_LO = 0x1.ef35793c76730p-45, LOG2E = 0x1.71547652b82fep+0;
    const uint64_t ix = (uint64_t)__double_as_longlong(x), tmp = ix - POW_LOG_OFF;
    const int i = (int)((tmp >> 45) & 127);
    const double kd = (double)(int)((int64_t)tmp >> 52);
    const double z = __longlong_as_double((long long)(ix - (tmp & (0xfffull << 52))));
    const pow_log_entry ent = pow_log_table[i]; // one 16-byte look-up
    const double invc = (double)ent.invc, logc = ent.logc, logctail = (double)ent.logctail;
    const double ph = z * invc, r_lo = __builtin_fma(z, invc, -ph); // z * invc = ph + r_lo exactly
    const double r = ph - 1.0;                                       // exact: ph lies within 2^-8 of 1
    const double t1 = __builtin_fma(kd, K(LN2_HI), logc);            // exact
    const double t2 = t1 + r;
    const double lo1 = __builtin_fma(kd, K(LN2_LO), logctail);
    const double lo2 = t1 - t2 + r; // |t1| >= |r| or t1 == 0: the sum's rounding error
    const double ar = -0.5 * r, ar2 = r * ar, ar3 = r * ar2;
    const double hi = t2 + ar2;
    const double lo3 = __builtin_fma(ar, r, -ar2);
    const double lo4 = t2 - hi + ar2;
    double q = __builtin_fma(r, K(1.0 / 4), K(-2.0 / 7));
    q = __builtin_fma(r, q, K(1.0 / 3));
    q = __builtin_fma(r, q, K(-2.0 / 5));
    q = __builtin_fma(r, q, K(1.0 / 2));
    q = __builtin_fma(r, q, K(-2.0 / 3));
    const double lo = lo1 + lo2 + lo3 + lo4 + __builtin_fma(-r, r_lo, r_lo) + ar3 * q;
    const double lhi = hi + lo, llo = hi - lhi + lo;
    const double ehi = y * lhi, elo = __builtin_fma(y, llo, __builtin_fma(y, lhi, -ehi));
    const double ec = __builtin_fmin(__builtin_fmax(ehi, -745.0), 745.0); // keeps the conversion of n in range
    const double n = __builtin_rint(ec * K(LOG2E));
    double f = __builtin_fma(-n, K(LN2_HI), ec);
    f = __builtin_fma(-n, K(LN2_LO), f);
    f += elo;
    double p = K(1.0 / 6227020800.0);
    p = __builtin_fma(p, f, K(1.0 / 479001600.0));
    p = __builtin_fma(p, f, K(1.0 / 39916800.0));
    p = __builtin_fma(p, f, K(1.0 / 3628800.0));
    p = __builtin_fma(p, f, K(1.0 / 362880.0));
    p = __builtin_fma(p, f, K(1.0 / 40320.0));
    p = __builtin_fma(p, f, K(1.0 / 5040.0));
    p = __builtin_fma(p, f, K(1.0 / 720.0));
    p = __builtin_fma(p, f, K(1.0 / 120.0));
    p = __builtin_fma(p, f, K(1.0 / 24.0));
    p = __builtin_fma(p, f, K(1.0 / 6.0));
    p = __builtin_fma(p, f, 0.5);
    p = __builtin_fma(p, f, 1.0);
    p = __builtin_fma(p, f, 1.0);
    const double res = __builtin_amdgcn_ldexp(p, (int)n);
    // +normal base, finite exponent, result well inside the normal range; NaN in ehi fails the comparison
    const bool own = __builtin_amdgcn_class(x, 0x100) && __builtin_amdgcn_class(y, 0x1f8) && __builtin_fabs(ehi) < 700.0;
    return own ? res : (double)__builtin_nanf("");
}
DPX_D double pow_f64(double x, double y)
{
    const double r = pow_f64_fast(x, y);
    return (r != r) ? ::pow(x, y) : r;
}

#define DPX_FP_FN2(NAME, F32, F64)                                          \
    template <class T> DPX_D T NAME(T x, T y)                               \
    {                                                                       \
        if constexpr (std::is_same_v<T, double>) return F64(x, y);          \
        else if constexpr (std::is_same_v<T, float>) return F32(x, y);      \
        else return (T)F32((float)x, (float)y);                             \
    }
DPX_FP_FN2(m_pow, pow_f32, pow_f64)
DPX_FP_FN2(m_atan2, ::atan2f, ::atan2)
DPX_FP_FN2(m_hypot, ::hypotf, ::hypot)
DPX_FP_FN2(m_copysign, ::copysignf, ::copysign)
DPX_FP_FN2(m_fmod, ::fmodf, ::fmod)
DPX_FP_FN2(m_nextafter, ::nextafterf, ::nextafter)
DPX_FP_FN2(m_fmax, ::fmaxf, ::fmax)
DPX_FP_FN2(m_fmin, ::fminf, ::fmin)
#undef DPX_FP_FN2

template <class T> DPX_D bool m_signbit(T x)
{
    if constexpr (std::is_same_v<T, double>) return (__double_as_longlong(x) >> 63) != 0;
    else if constexpr (std::is_same_v<T, float>) return (__float_as_int(x) >> 31) != 0;
    else return (__float_as_int((float)x) >> 31) != 0;
}
template <class T> DPX_D bool m_isinf(T x)
{
    if constexpr (is_fp_v<T>) { T a = x < T(0) ? -x : x; return a == (T)__builtin_inff(); }
    else return false;
}

// ---- complex elementary functions (textbook formulas on the real functions above; the
// reference gets these from the SYCL complex library, results agree to rounding error for
// finite arguments of moderate size) -----------------------------------------------------------
template <class R> DPX_D bool m_finite(R v) { return v == v && !m_isinf(v); }
template <class R> DPX_D void m_sincos(R x, R &s, R &c)
{
    if constexpr (std::is_same_v<R, double>) sincos_both_f64(x, s, c);
    else ::sincosf(x, &s, &c);
}

// In the complex functions below every real function is evaluated ONCE, ahead of the case analysis, and the
// cases only choose among products of the values: written with the calls inside the branches (sin y and cos y of
// the finite case, again in the cases of an infinite real part), the compiler moved the branches' calls in front
// of the case analysis and kept the finite case's own copy, so that every element paid for sin and cos twice
// (complex128 exp: 257 vector instructions per element, 108 for the function on its own).

// sinh and cosh of one argument from one expm1 (the forms of sinh_via and cosh_via above): t = expm1(|x|),
// w = t + 1 = exp(|x|), sinh = (t + t/w)/2, cosh = (w + 1/w)/2.  Host check against long double over 2e7
// arguments: sinh 1.9, cosh 1.3 ULP.
template <class R> DPX_D void m_sinhcosh(R x, R &sh, R &ch)
{
    if constexpr (std::is_same_v<R, double>) {
        const R a = __builtin_fabs(x);
        if (!(a <= R(709))) { // rare: where exp overflows and the functions do not yet, infinities, NaN
            asm volatile("" ::: "memory"); // (not to be executed speculatively, see sincos_both_f64)
            sh = sinh_f64(x);
            ch = cosh_f64(x);
            return;
        }
        const R t = ::expm1(a), w = t + R(1);
        const R rc = div_moderate<R>(R(1), w), q = t * rc;
        R s = R(0.5) * ((a < R(1)) ? R(2) * t - t * q : t + q);
        s = (a == R(0)) ? a : s;
        sh = __builtin_copysign(s, x);
        ch = R(0.5) * w + R(0.5) * rc;
    }
    else {
        sh = m_sinh(x);
        ch = m_cosh(x);
    }
}

// exp with the non-finite cases of libtensor/include/kernels/elementwise_functions/exp.hpp:75-132
template <class R> DPX_D cplx<R> c_exp(cplx<R> z)
{
    const R x = z.re, y = z.im;
    R sn, cs;
    m_sincos(y, sn, cs);
    const R e = m_exp(x);
    const bool xf = m_finite(x), yf = m_finite(y);
    if (xf && yf) return (y == R(0)) ? cplx<R>{e, y} : cplx<R>{e * cs, e * sn};
    const R q_nan = (R)__builtin_nanf("");
    if (xf) return {q_nan, q_nan};
    if (x != x) return (y == R(0)) ? z : cplx<R>{x, q_nan};
    if (!m_signbit(x)) { // +inf
        if (y == R(0)) return {x, y};
        if (yf) return {x * cs, x * sn};
        return {x, q_nan};
    }
    if (yf) return {R(0) * cs, R(0) * sn}; // exp(-inf) = 0
    return {R(0), R(0)};
}
// 2^z = exp(z ln 2) (exp2.hpp:75-133)
template <class R> DPX_D cplx<R> c_exp2(cplx<R> z)
{
    const R ln2 = R(0.69314718055994530941723212145817657);
    const cplx<R> t{z.re * ln2, z.im * ln2};
    if (t.re != t.re && t.im == R(0)) return z; // the reference hands back its argument here
    return c_exp(t);
}
// expm1(x + iy) = expm1(x) cos y - 2 sin^2(y/2) + i exp(x) sin y (expm1.hpp:75-138), with
// 2 sin^2(y/2) = 1 - cos y = sin^2 y / (1 + cos y): the quotient where cos y >= 0 (no cancellation), the
// difference elsewhere
template <class R> DPX_D cplx<R> c_expm1(cplx<R> z)
{
    const R x = z.re, y = z.im;
    R sn, cs;
    m_sincos(y, sn, cs);
    const R t = m_expm1(x), e = m_exp(x);
    const R q_nan = (R)__builtin_nanf("");
    const bool yf = m_finite(y);
    if (m_isinf(x)) {
        if (x > R(0)) {
            if (!yf) return {x, q_nan};
            if (y == R(0)) return z;
            return {m_copysign(x, cs), m_copysign(x, sn)};
        }
        if (!yf) return {R(-1), m_copysign(R(0), y)};
        return {R(-1), m_copysign(R(0), sn)};
    }
    if (x != x) return (y == R(0)) ? z : cplx<R>{q_nan, q_nan};
    if (x == R(0) && y == R(0)) return {R(0), y};
    const R h = (cs >= R(0)) ? div_moderate<R>(sn * sn, R(1) + cs) : R(1) - cs; // NaN y: NaN either way
    const R sy = (y == R(0)) ? y : sn;
    return {t * cs - h, e * sy};
}
template <class R> DPX_D cplx<R> c_log(cplx<R> z) { return {m_log(m_hypot(z.re, z.im)), m_atan2(z.im, z.re)}; }
// log1p.hpp:75-100, log2.hpp:75-83, log10.hpp:75-84
template <class R> DPX_D cplx<R> c_log1p(cplx<R> z)
{
    const R x = z.re, y = z.im;
    const R im = m_atan2(y, x + R(1));
    const R ax = x < R(0) ? -x : x, ay = y < R(0) ? -y : y;
    if ((ax > ay ? ax : ay) < R(0.1)) return {m_log1p(x * (R(2) + x) + y * y) / R(2), im};
    return {m_log(m_hypot(x + R(1), y)), im};
}
template <class R> DPX_D cplx<R> c_log2(cplx<R> z)
{
    const cplx<R> l = c_log(z);
    const R ln2 = m_log(R(2));
    return {l.re / ln2, l.im / ln2};
}
template <class R> DPX_D cplx<R> c_log10(cplx<R> z)
{
    const cplx<R> l = c_log(z);
    const R ln10 = m_log(R(10));
    return {l.re / ln10, l.im / ln10};
}
template <class R> DPX_D cplx<R> c_sqrt(cplx<R> z)
{
    if (z.re == R(0) && z.im == R(0)) return {R(0), z.im};
    if (m_isinf(z.im)) return {(R)__builtin_inff(), z.im};
    const R ar = z.re < R(0) ? -z.re : z.re;
    const R t = m_sqrt((ar + m_hypot(z.re, z.im)) * R(0.5));
    if (z.re >= R(0)) return {t, z.im / (t + t)};
    const R ai = m_copysign(z.im, R(1)); // |im| also for -0.0: the real part of a root is never -0.0
    return {ai / (t + t), m_copysign(t, z.im)};
}
// sinh, cosh, tanh: finite arguments by the textbook formulas, the others case by case as in
// libtensor/include/kernels/elementwise_functions/{sinh.hpp:75-160, cosh.hpp:75-150, tanh.hpp:75-135}
template <class R> DPX_D cplx<R> c_sinh(cplx<R> z)
{
    const R x = z.re, y = z.im;
    R sn, cs, sh, ch;
    m_sincos(y, sn, cs);
    m_sinhcosh(x, sh, ch);
    const bool xf = m_finite(x), yf = m_finite(y);
    if (xf && yf) return (y == R(0)) ? cplx<R>{sh, y} : cplx<R>{sh * cs, ch * sn};
    if (x == R(0) && !yf) return {m_copysign(R(0), x * (y - y)), y - y};
    if (y == R(0) && !xf) return (x != x) ? cplx<R>{x, y} : cplx<R>{x, m_copysign(R(0), y)};
    if (xf && !yf) return {y - y, x * (y - y)};
    if (x == x) { // +-inf
        if (!yf) return {x * x, x * (y - y)};
        return {x * cs, (R)__builtin_inff() * sn};
    }
    return {(x * x) * (y - y), (x + x) * (y - y)};
}
template <class R> DPX_D cplx<R> c_cosh(cplx<R> z)
{
    const R x = z.re, y = z.im;
    R sn, cs, sh, ch;
    m_sincos(y, sn, cs);
    m_sinhcosh(x, sh, ch);
    const R q_nan = (R)__builtin_nanf("");
    const bool xf = m_finite(x), yf = m_finite(y);
    if (xf && yf) return (y == R(0)) ? cplx<R>{ch, x * y} : cplx<R>{ch * cs, sh * sn};
    if (x == R(0) && !yf) return {q_nan, m_copysign(R(0), x * q_nan)};
    if (y == R(0) && !xf) return {x * x, m_copysign(R(0), x) * y};
    if (xf && !yf) return {q_nan, x * q_nan};
    if (m_isinf(x)) {
        if (!yf) return {x * x, x * q_nan};
        return {(x * x) * cs, x * sn};
    }
    return {(x * x) * (y - y), (x + x) * (y - y)};
}
template <class R> DPX_D cplx<R> c_tanh(cplx<R> z)
{
    const R x = z.re, y = z.im;
    // Kahan's formulation: no cancellation near the poles at x = 0, y = pi/2 + k pi.  rho = sqrt(1 + sinh^2 x) is
    // cosh x; the sign of sin y cos y and of sin 2y, which the large and infinite cases ask for, is that of tan y
    const R t = m_tan(y);
    R sh, rho;
    m_sinhcosh(x, sh, rho);
    const R q_nan = (R)__builtin_nanf("");
    if (!m_finite(x)) {
        if (x != x) return {q_nan, (y == R(0)) ? y : q_nan};
        return {m_copysign(R(1), x), m_copysign(R(0), m_isinf(y) ? y : t)};
    }
    if (!m_finite(y)) return (x == R(0)) ? cplx<R>{x, q_nan} : cplx<R>{q_nan, q_nan};
    const R ax = x < R(0) ? -x : x;
    if (ax > R(20)) return {m_copysign(R(1), x), m_copysign(R(0), t)};
    const R beta = R(1) + t * t;
    if (m_isinf(t)) return {rho / sh, R(1) / t};
    const R rd = div_moderate<R>(R(1), R(1) + beta * sh * sh);
    return {(beta * rho * sh) * rd, t * rd};
}
// sin z = -i sinh(iz), cos z = cosh(iz), tan z = -i tanh(iz)
template <class R> DPX_D cplx<R> c_sin(cplx<R> z)
{
    const cplx<R> w = c_sinh(cplx<R>{-z.im, z.re});
    // a zero real part of a finite argument keeps its sign (sin.hpp:84-92)
    if (z.re == R(0) && m_finite(z.im)) return {m_copysign(R(0), z.re), -w.re};
    return {w.im, -w.re};
}
template <class R> DPX_D cplx<R> c_cos(cplx<R> z) { return c_cosh(cplx<R>{-z.im, z.re}); }
template <class R> DPX_D cplx<R> c_tan(cplx<R> z) { const cplx<R> w = c_tanh(cplx<R>{-z.im, z.re}); return {w.im, -w.re}; }

// Inverse functions.  Ordinary arguments after W. Kahan, "Branch cuts for complex elementary
// functions" (1987): the square roots of 1 -/+ z (or z -/+ 1) carry the branch cuts, signed zeros
// pick the side.  NaN parts and large arguments are handled around them as the reference does
// (libtensor/include/kernels/elementwise_functions/complex_math.hpp:57-262, acosh.hpp:76-105).
template <class R> DPX_D cplx<R> c_asin_ordinary(cplx<R> z)
{
    const cplx<R> s1 = c_sqrt(cplx<R>{R(1) - z.re, -z.im}), s2 = c_sqrt(cplx<R>{R(1) + z.re, z.im});
    return {m_atan2(z.re, s1.re * s2.re - s1.im * s2.im), m_asinh(s1.re * s2.im - s1.im * s2.re)};
}
// beyond sqrt(1/eps)/2 the functions are log(2z) to working precision
template <class R> inline constexpr R inv_big = std::is_same_v<R, double> ? R(33554432.0) : R(1448.15466);
template <class R> DPX_D R m_abs(R v) { return m_copysign(v, R(1)); }
template <class R> DPX_D cplx<R> c_acos(cplx<R> z)
{
    const R x = z.re, y = z.im;
    const R q_nan = (R)__builtin_nanf("");
    const R ln2 = R(0.6931471805599453094172321214581765);
    if (x != x) return m_isinf(y) ? cplx<R>{q_nan, -y} : cplx<R>{q_nan, q_nan};
    if (y != y) {
        if (m_isinf(x)) return {q_nan, -(R)__builtin_inff()};
        if (x == R(0)) return {R(1.5707963267948966192313216916397514), q_nan};
        return {q_nan, q_nan};
    }
    if (m_abs(x) > inv_big<R> || m_abs(y) > inv_big<R>) {
        const cplx<R> l = c_log(z);
        const R ry = l.re + ln2;
        return {m_abs(l.im), m_signbit(y) ? ry : -ry};
    }
    const cplx<R> s1 = c_sqrt(cplx<R>{R(1) - x, -y}), s2 = c_sqrt(cplx<R>{R(1) + x, y});
    return {R(2) * m_atan2(s1.re, s2.re), m_asinh(s2.re * s1.im - s2.im * s1.re)};
}
template <class R> DPX_D cplx<R> c_acosh(cplx<R> z)
{
    // from acos: acosh z = +-i acos z, with the sign that makes the real part positive
    const cplx<R> a = c_acos(z);
    if (a.re != a.re && a.im != a.im) return {a.im, a.re};
    if (a.re != a.re) return {m_abs(a.im), a.re};
    return {m_abs(a.im), m_copysign(a.re, z.im)};
}
template <class R> DPX_D cplx<R> c_asinh(cplx<R> z)
{
    const R x = z.re, y = z.im;
    const R q_nan = (R)__builtin_nanf("");
    const R ln2 = R(0.6931471805599453094172321214581765);
    if (x != x) {
        if (m_isinf(y)) return {y, q_nan};
        if (y == R(0)) return {q_nan, y};
        return {q_nan, q_nan};
    }
    if (y != y) return m_isinf(x) ? cplx<R>{x, q_nan} : cplx<R>{q_nan, q_nan};
    if (m_abs(x) > inv_big<R> || m_abs(y) > inv_big<R>) {
        const cplx<R> l = m_signbit(x) ? c_log(cplx<R>{-x, -y}) : c_log(z);
        return {m_copysign(l.re + ln2, x), m_copysign(l.im, y)};
    }
    // asinh z = -i asin(iz)
    const cplx<R> w = c_asin_ordinary(cplx<R>{-y, x});
    return {w.im, -w.re};
}
// asin(x + iy) = swap(asinh(y + ix))
template <class R> DPX_D cplx<R> c_asin(cplx<R> z) { const cplx<R> w = c_asinh(cplx<R>{z.im, z.re}); return {w.im, w.re}; }
template <class R> DPX_D cplx<R> c_atanh(cplx<R> z)
{
    const R pi_2 = R(1.5707963267948966192313216916397514);
    const R q_nan = (R)__builtin_nanf("");
    if (z.re != z.re) {
        if (m_isinf(z.im)) return {m_copysign(R(0), z.re), m_copysign(pi_2, z.im)};
        return {q_nan, q_nan};
    }
    if (z.im != z.im) {
        if (m_isinf(z.re)) return {m_copysign(R(0), z.re), q_nan};
        if (z.re == R(0)) return {z.re, q_nan};
        return {q_nan, q_nan};
    }
    const R huge = std::is_same_v<R, double> ? R(4503599627370496.0) : R(8388608.0); // 1/eps
    if (m_abs(z.re) > huge || m_abs(z.im) > huge) return {R(0), m_copysign(pi_2, z.im)};
    // odd function: work in the right half plane
    const bool neg = m_signbit(z.re);
    const R x = neg ? -z.re : z.re, y = neg ? -z.im : z.im;
    cplx<R> w;
    if (x == R(1) && y == R(0)) {
        w = {(R)__builtin_inff(), y};
    }
    else {
        const R d = (R(1) - x) * (R(1) - x) + y * y;
        w = {R(0.25) * m_log1p(R(4) * x / d), R(0.5) * m_atan2(R(2) * y, (R(1) - x) * (R(1) + x) - y * y)};
    }
    return neg ? cplx<R>{-w.re, -w.im} : w;
}
// atan(x + iy) = swap(atanh(y + ix))
template <class R> DPX_D cplx<R> c_atan(cplx<R> z) { const cplx<R> w = c_atanh(cplx<R>{z.im, z.re}); return {w.im, w.re}; }

template <class T> using V = value_of_t<T>;

// =========================== binary ops =============================================
// ok<T>: same-dtype pair (T, T) has a kernel.

struct AddOp { // add.hpp:63-114,140-204; bool + bool is logical or
    template <class T> static constexpr bool ok = true;
    template <class T> using out = T;
    template <class T> DPX_D static V<T> apply(V<T> a, V<T> b)
    {
        if constexpr (is_bool_v<T>) return a || b;
        else return a + b;
    }
};
struct SubOp { // subtract.hpp:62: every type but bool
    template <class T> static constexpr bool ok = !is_bool_v<T>;
    template <class T> using out = T;
    template <class T> DPX_D static V<T> apply(V<T> a, V<T> b) { return a - b; }
};
struct MulOp { // multiply.hpp:64; bool * bool is logical and
    template <class T> static constexpr bool ok = true;
    template <class T> using out = T;
    template <class T> DPX_D static V<T> apply(V<T> a, V<T> b)
    {
        if constexpr (is_bool_v<T>) return a && b;
        else return a * b;
    }
};
struct DivOp { // true_divide.hpp:63: floating and complex only
    template <class T> static constexpr bool ok = is_fp_v<T> || is_cplx_v<T>;
    template <class T> using out = T;
    template <class T> DPX_D static V<T> apply(V<T> a, V<T> b) { return a / b; }
};
template <int WHICH> struct BitOp { // bitwise_and.hpp:59-118 (or/xor alike); bool: logical
    template <class T> static constexpr bool ok = is_bool_v<T> || is_int_v<T>;
    template <class T> using out = T;
    template <class T> DPX_D static V<T> apply(V<T> a, V<T> b)
    {
        if constexpr (is_bool_v<T>) {
            if constexpr (WHICH == 0) return a && b;
            else if constexpr (WHICH == 1) return a || b;
            else return a != b;
        }
        else {
            if constexpr (WHICH == 0) return a & b;
            else if constexpr (WHICH == 1) return a | b;
            else return a ^ b;
        }
    }
};
// comparisons, greater.hpp:62-146 and siblings: all 14 same-dtype pairs -> bool;
// CMP: 0 ==, 1 !=, 2 <, 3 <=, 4 >, 5 >=
template <int CMP> struct CmpOp {
    template <class T> static constexpr bool ok = true;
    template <class T> using out = bool_t;
    template <class T> DPX_D static bool apply(V<T> a, V<T> b)
    {
        if constexpr (CMP == 0) return a == b;
        else if constexpr (CMP == 1) return a != b;
        else if constexpr (is_cplx_v<T>) {
            if constexpr (CMP == 2) return c_less(a, b);
            else if constexpr (CMP == 3) return c_less_eq(a, b);
            else if constexpr (CMP == 4) return c_greater(a, b);
            else return c_greater_eq(a, b);
        }
        else {
            if constexpr (CMP == 2) return a < b;
            else if constexpr (CMP == 3) return a <= b;
            else if constexpr (CMP == 4) return a > b;
            else return a >= b;
        }
    }
    // mixed int64/uint64 pairs compare exactly, without promotion to double
    DPX_D static bool apply_iu(int64_t a, uint64_t b)
    {
        if constexpr (CMP == 0) return a >= 0 && (uint64_t)a == b;
        else if constexpr (CMP == 1) return a < 0 || (uint64_t)a != b;
        else if constexpr (CMP == 2) return a < 0 || (uint64_t)a < b;
        else if constexpr (CMP == 3) return a < 0 || (uint64_t)a <= b;
        else if constexpr (CMP == 4) return a >= 0 && (uint64_t)a > b;
        else return a >= 0 && (uint64_t)a >= b;
    }
    DPX_D static bool apply_ui(uint64_t a, int64_t b)
    {
        if constexpr (CMP == 0) return b >= 0 && a == (uint64_t)b;
        else if constexpr (CMP == 1) return b < 0 || a != (uint64_t)b;
        else if constexpr (CMP == 2) return b >= 0 && a < (uint64_t)b;
        else if constexpr (CMP == 3) return b >= 0 && a <= (uint64_t)b;
        else if constexpr (CMP == 4) return b < 0 || a > (uint64_t)b;
        else return b < 0 || a >= (uint64_t)b;
    }
};
struct MaxOp { // maximum.hpp:63-90
    template <class T> static constexpr bool ok = true;
    template <class T> using out = T;
    template <class T> DPX_D static V<T> apply(V<T> a, V<T> b) { return max_nan(a, b); }
};
struct MinOp { // minimum.hpp
    template <class T> static constexpr bool ok = true;
    template <class T> using out = T;
    template <class T> DPX_D static V<T> apply(V<T> a, V<T> b) { return min_nan(a, b); }
};
template <int WHICH> struct LogicalOp { // logical_and.hpp / logical_or.hpp / logical_xor.hpp
    template <class T> static constexpr bool ok = true;
    template <class T> using out = bool_t;
    template <class T> DPX_D static bool apply(V<T> a, V<T> b)
    {
        bool x = convert<bool_t, T>(to_storage<T>(a)).v, y = convert<bool_t, T>(to_storage<T>(b)).v;
        if constexpr (WHICH == 0) return x && y;
        else if constexpr (WHICH == 1) return x || y;
        else return x != y;
    }
};
// Truncated quotient of two integers of at most 16 bits, b != 0, through the float reciprocal: the
// integer division sequence is about 35 instructions and a pack of 1-byte elements holds sixteen.
// Two such numbers have a quotient that is either an integer or at least 2^-16 away from one in
// relative terms, the product with the reciprocal is off by 2^-22 at most, and the factor
// 1 + 2^-20 lifts exact quotients back over the integer without carrying any other across one.
template <class T> DPX_D int small_int_quotient(T a, T b)
{
    static_assert(sizeof(T) <= 2);
    return (int)(((float)(int)a * __builtin_amdgcn_rcpf((float)(int)b)) * 1.00000095367431640625f);
}
struct FloorDivOp { // floor_divide.hpp:63-86: ints (x // 0 == 0) and real fp
    template <class T> static constexpr bool ok = is_int_v<T> || is_fp_v<T>;
    template <class T> using out = T;
    template <class T> DPX_D static T apply(T a, T b)
    {
        if constexpr (is_int_v<T> && sizeof(T) <= 2) {
            // branch-free for the narrow types: 32-bit arithmetic, the quotient of -128 by -1 wraps in the cast
            const int q = small_int_quotient(a, b), m = (int)a - q * (int)b;
            const int r = q - ((m != 0) && ((m < 0) != ((int)b < 0)));
            return b == T(0) ? T(0) : (T)r;
        }
        else if constexpr (is_int_v<T> && sizeof(T) == 4) {
            // 32-bit operands through the double quotient, branch-free: both are exact as doubles, and a
            // quotient that is not an integer lies at least 1 / |b| from the next one, 2^-31 of its size and
            // more, so the correctly rounded double quotient never lands on an integer it does not equal and
            // its floor is the floored quotient (a third of the instructions of the integer division with its
            // sign cases; int32 // scalar: 67 % of the HBM rate before)
            const double q = __builtin_floor((double)a / (double)b);
            T r;
            if constexpr (std::is_signed_v<T>) {
                r = (T)(int64_t)q; // (-2^31 // -1 = 2^31 wraps to -2^31 in the cast)
            }
            else r = (T)q;
            return b == T(0) ? T(0) : r;
        }
        else if constexpr (is_int_v<T>) {
            if (b == T(0)) return T(0);
            if constexpr (std::is_signed_v<T>) {
                if (b == T(-1)) return (T)(0 - (std::make_unsigned_t<T>)a); // INT_MIN // -1 wraps
                T d = a / b, m = a % b;
                return (T)(d - ((m != 0) && ((m < 0) != (b < 0))));
            }
            else return a / b;
        }
        else {
            T d = a / b;
            return (d == T(0)) ? d : m_floor(d);
        }
    }
};
struct RemainderOp { // remainder.hpp: Python-style modulo, x % 0 == 0 for ints
    template <class T> static constexpr bool ok = is_int_v<T> || is_fp_v<T>;
    template <class T> using out = T;
    template <class T> DPX_D static T apply(T a, T b)
    {
        if constexpr (is_int_v<T> && sizeof(T) <= 2) {
            const int q = small_int_quotient(a, b), m = (int)a - q * (int)b;
            const int r = (m != 0 && ((m < 0) != ((int)b < 0))) ? m + (int)b : m;
            return b == T(0) ? T(0) : (T)r;
        }
        else if constexpr (is_int_v<T> && sizeof(T) == 4) {
            // a - floor(a / b) * b with the floored quotient of FloorDivOp (exact for 32-bit operands), in
            // wrapping 32-bit arithmetic: the sign follows the divisor, -2^31 % -1 comes out as 0
            using U = std::make_unsigned_t<T>;
            const double q = __builtin_floor((double)a / (double)b);
            U qi;
            if constexpr (std::is_signed_v<T>) qi = (U)(int64_t)q;
            else qi = (U)q;
            return b == T(0) ? T(0) : (T)((U)a - qi * (U)b);
        }
        else if constexpr (is_int_v<T>) {
            if (b == T(0)) return T(0);
            if constexpr (std::is_signed_v<T>) {
                if (b == T(-1)) return T(0);
                T m = a % b;
                return (m != 0 && ((m < 0) != (b < 0))) ? (T)(m + b) : m;
            }
            else return a % b;
        }
        else {
            T m = m_fmod(a, b);
            if (m != T(0)) {
                if ((b < T(0)) != (m < T(0))) m += b;
            }
            else m = m_copysign(T(0), b);
            return m;
        }
    }
};
// float16 operands: 2^(y log2 x) on the hardware's float log2 and exp2 for a positive finite base and a finite
// exponent.  |y log2 x| is below 2^5 wherever the result is a finite nonzero float16, so the ULP of the hardware
// logarithm and the rounding of the product move the result by 2^-18 of itself, 1/128 ULP of a float16; six
// vector instructions where the double-precision routine of the float operands takes 45 (4 bytes of traffic per
// element hide about a dozen).  NaN where it does not apply.
DPX_D float pow_f16_fast(float x, float y)
{
    const bool ok = x > 0.0f && x < __builtin_inff() && __builtin_fabsf(y) < __builtin_inff();
    const float r = __builtin_amdgcn_exp2f(y * __builtin_amdgcn_logf(x));
    return ok ? r : __builtin_nanf("");
}
struct PowOp { // pow.hpp: ints by repeated squaring (negative exponent -> 0), fp via pow
    template <class T> static constexpr bool ok = is_int_v<T> || is_fp_v<T> || is_cplx_v<T>;
    template <class T> using out = T;
    template <class T> DPX_D static T apply(T a, T b)
    {
        if constexpr (is_cplx_v<T>) {
            using R = real_of_t<T>;
            if (b.re == R(0) && b.im == R(0)) return T{R(1), R(0)};
            // a zero base is zero only under a positive real exponent; every other exponent goes
            // through exp(b log 0) like any base (0 ** -1 = inf + nan j, 0 ** 1j = nan + nan j)
            if (a.re == R(0) && a.im == R(0) && b.re > R(0) && b.im == R(0)) return T{R(0), R(0)};
            return c_exp(b * c_log(a));
        }
        else if constexpr (is_int_v<T>) {
            if constexpr (std::is_signed_v<T>) {
                if (b < 0) return T(0); // pow.hpp:72-78: invalid, 0 for every base
            }
            using U = std::make_unsigned_t<T>;
            U r = 1, base = (U)a;
            U e = (U)b;
            while (e) {
                if (e & 1) r = (U)(r * base);
                base = (U)(base * base);
                e >>= 1;
            }
            return (T)r;
        }
        else {
            // x ** 2, the most common power: the product is the correctly rounded square and agrees with pow
            // on every special value (NaN, infinities, signed zeros); a wave whose exponents are all 2 never
            // enters the device library's routine (doubles: 36 % -> 85 % of the HBM rate)
            if (b == T(2)) return a * a;
            return m_pow(a, b);
        }
    }
    // the short routine (pow_f32_fast, pow_f64_fast) for the whole pack first, the device library for what it leaves
    template <class T> static constexpr bool two_phase = is_fp_v<T>;
    template <class T, class R> DPX_D static R fast(R a, R b)
    {
        R r;
        if constexpr (std::is_same_v<R, double>) r = pow_f64_fast(a, b);
        else if constexpr (std::is_same_v<T, half_t>) r = (R)pow_f16_fast((float)a, (float)b);
        else r = (R)pow_f32_fast((float)a, (float)b);
        return b == R(2) ? a * a : r; // squares as in apply()
    }
    template <class T, class R> DPX_D static bool cheap_applies(R, R b) { return b == R(2); }
    template <class T, class R> DPX_D static R cheap(R a, R) { return a * a; }
    template <class T, class R> DPX_D static R fixup(R r, R a, R b)
    {
        if constexpr (std::is_same_v<R, double>) return (r != r) ? ::pow(a, b) : r;
        else return (r != r) ? (R)::powf((float)a, (float)b) : r;
    }
};
struct Atan2Op {
    template <class T> static constexpr bool ok = is_fp_v<T>;
    template <class T> using out = T;
    template <class T> DPX_D static T apply(T a, T b) { return m_atan2(a, b); }
};
struct HypotOp {
    template <class T> static constexpr bool ok = is_fp_v<T>;
    template <class T> using out = T;
    template <class T> DPX_D static T apply(T a, T b) { return m_hypot(a, b); }
};
struct CopysignOp {
    template <class T> static constexpr bool ok = is_fp_v<T>;
    template <class T> using out = T;
    template <class T> DPX_D static T apply(T a, T b) { return m_copysign(a, b); }
};
template <bool LEFT> struct ShiftOp { // bitwise_left_shift.hpp / bitwise_right_shift.hpp
    template <class T> static constexpr bool ok = is_int_v<T>;
    template <class T> using out = T;
    template <class T> DPX_D static T apply(T a, T b)
    {
        // bitwise_left_shift.hpp:88-103, bitwise_right_shift.hpp:88-105: a negative count gives 0
        // in both directions; a count of the width or more gives 0, except that a right shift of
        // a negative value gives -1
        constexpr int bits = 8 * sizeof(T);
        if constexpr (std::is_signed_v<T>) {
            if (b < 0) return T(0);
            if (b >= bits) return (!LEFT && a < 0) ? T(-1) : T(0);
        }
        else if (b >= (T)bits) return T(0);
        if constexpr (LEFT) return (T)((std::make_unsigned_t<T>)a << b);
        else return (T)(a >> b);
    }
};

// =========================== unary ops ==============================================

struct AbsOp { // abs.hpp:61-90: complex -> real
    template <class T> static constexpr bool ok = true;
    template <class T> using out = real_of_t<T>;
    template <class T> DPX_D static V<out<T>> apply(V<T> x)
    {
        if constexpr (is_bool_v<T> || is_uint_v<T>) return x;
        else if constexpr (is_cplx_v<T>) return m_hypot(x.re, x.im);
        else if constexpr (is_fp_v<T>) return m_signbit(x) ? -x : x;
        else return (T)(x < 0 ? (T)(0 - (std::make_unsigned_t<T>)x) : x);
    }
};
struct NegOp { // negative.hpp: all but bool
    template <class T> static constexpr bool ok = !is_bool_v<T>;
    template <class T> using out = T;
    template <class T> DPX_D static T apply(T x)
    {
        if constexpr (is_int_v<T>) return (T)(0 - (std::make_unsigned_t<T>)x);
        else return -x;
    }
};
struct PosOp {
    template <class T> static constexpr bool ok = !is_bool_v<T>;
    template <class T> using out = T;
    template <class T> DPX_D static T apply(T x) { return x; }
};
struct SquareOp { // square.hpp:64-90; bool -> int8
    template <class T> static constexpr bool ok = true;
    template <class T> using out = std::conditional_t<is_bool_v<T>, int8_t, T>;
    template <class T> DPX_D static V<out<T>> apply(V<T> x)
    {
        if constexpr (is_bool_v<T>) return (int8_t)(x ? 1 : 0);
        else if constexpr (is_int_v<T>) return (T)((std::make_unsigned_t<T>)x * (std::make_unsigned_t<T>)x);
        else return x * x;
    }
};
// real floating-point functions; exp.hpp:153-163 and siblings list f2 f4 f8 (+ complex,
// which this library does not implement for transcendentals)
#define DPX_FP_UNARY(NAME, EXPR)                                   \
    struct NAME {                                                  \
        template <class T> static constexpr bool ok = is_fp_v<T>;  \
        template <class T> using out = T;                          \
        template <class T> DPX_D static T apply(T x) { return EXPR; } \
    };
// same, with a complex form CEXPR
#define DPX_FPC_UNARY(NAME, EXPR, CEXPR)                                        \
    struct NAME {                                                               \
        template <class T> static constexpr bool ok = is_fp_v<T> || is_cplx_v<T>; \
        template <class T> using out = T;                                       \
        template <class T> DPX_D static T apply(T x)                            \
        {                                                                       \
            if constexpr (is_cplx_v<T>) return CEXPR;                           \
            else return EXPR;                                                   \
        }                                                                       \
    };
DPX_FPC_UNARY(SqrtOp, m_sqrt(x), c_sqrt(x))
DPX_FPC_UNARY(ExpOp, m_exp(x), c_exp(x))
DPX_FPC_UNARY(LogOp, m_log(x), c_log(x))
// sin, cos, tan: for doubles the contiguous kernel runs the straight-line routine for the arguments below 1e6 over
// a whole pack first, so that the elements' chains interleave, and then the device library's for what is left
// (with the hand-over test in front of each element's routine the elements ran one after the other: tan 5 % slower)
#define DPX_TRIG_UNARY(NAME, EXPR, CEXPR, BELOW, LIBM)                            \
    struct NAME {                                                               \
        template <class T> static constexpr bool ok = is_fp_v<T> || is_cplx_v<T>; \
        template <class T> using out = T;                                       \
        template <class T> DPX_D static T apply(T x)                            \
        {                                                                       \
            if constexpr (is_cplx_v<T>) return CEXPR;                           \
            else return EXPR;                                                   \
        }                                                                       \
        template <class T> static constexpr bool two_phase = std::is_same_v<T, double>; \
        template <class T> DPX_D static double fast(double x) { return BELOW(x); } \
        template <class T> DPX_D static double fixup(double r, double x)        \
        {                                                                       \
            if (!(__builtin_fabs(x) < TRIG_FAST_LIMIT)) {                       \
                asm volatile("" ::: "memory"); /* (not to be executed speculatively) */ \
                r = LIBM(x);                                                    \
            }                                                                   \
            return r;                                                           \
        }                                                                       \
    };
DPX_TRIG_UNARY(SinOp, (x == T(0)) ? x : m_sin(x), c_sin(x), sin_f64_below_limit, ::sin) // sin.hpp:186-194: a zero comes back as it is
DPX_TRIG_UNARY(CosOp, m_cos(x), c_cos(x), cos_f64_below_limit, ::cos)
DPX_TRIG_UNARY(TanOp, m_tan(x), c_tan(x), tan_f64_below_limit, ::tan)
#undef DPX_TRIG_UNARY
DPX_FPC_UNARY(TanhOp, m_tanh(x), c_tanh(x))
DPX_FPC_UNARY(Exp2Op, m_exp2(x), c_exp2(x))
DPX_FPC_UNARY(Expm1Op, (x == T(0)) ? x : m_expm1(x), c_expm1(x)) // expm1.hpp:139-146
DPX_FPC_UNARY(Log2Op, m_log2(x), c_log2(x))
DPX_FPC_UNARY(Log10Op, m_log10(x), c_log10(x))
DPX_FPC_UNARY(Log1pOp, (x == T(0)) ? x : m_log1p(x), c_log1p(x))
DPX_FP_UNARY(RsqrtOp, T(1) / m_sqrt(x))
DPX_FP_UNARY(CbrtOp, m_cbrt(x))
DPX_FPC_UNARY(ReciprocalOp, T(1) / x, (T{real_of_t<T>(1), real_of_t<T>(0)} / x))
DPX_FPC_UNARY(SinhOp, m_sinh(x), c_sinh(x))
DPX_FPC_UNARY(CoshOp, m_cosh(x), c_cosh(x))
DPX_FPC_UNARY(AsinOp, m_asin(x), c_asin(x))
DPX_FPC_UNARY(AcosOp, m_acos(x), c_acos(x))
DPX_FPC_UNARY(AtanOp, m_atan(x), c_atan(x))
DPX_FPC_UNARY(AsinhOp, m_asinh(x), c_asinh(x))
DPX_FPC_UNARY(AcoshOp, m_acosh(x), c_acosh(x))
DPX_FPC_UNARY(AtanhOp, m_atanh(x), c_atanh(x))
#undef DPX_FP_UNARY
#undef DPX_FPC_UNARY
struct ErfOp { // dpnp/backend/kernels/elementwise_functions/erf.hpp:52-95; f2 -> f4
    template <class T> static constexpr bool ok = is_fp_v<T>;
    template <class T> using out = std::conditional_t<std::is_same_v<T, half_t>, float, T>;
    template <class T> DPX_D static out<T> apply(T x) { return m_erf((out<T>)x); }
};
template <int WHICH> struct RoundOp { // floor.hpp / ceil.hpp / trunc.hpp: identity on ints and bool
    template <class T> static constexpr bool ok = !is_cplx_v<T>;
    template <class T> using out = T;
    template <class T> DPX_D static V<T> apply(V<T> x)
    {
        if constexpr (is_fp_v<T>) {
            if constexpr (WHICH == 0) return m_floor(x);
            else if constexpr (WHICH == 1) return m_ceil(x);
            else return m_trunc(x);
        }
        else return x;
    }
};
struct SignOp { // sign.hpp:63-110 (NaN -> NaN; complex: z / |z|, 0 for 0)
    template <class T> static constexpr bool ok = is_int_v<T> || is_fp_v<T> || is_cplx_v<T>;
    template <class T> using out = T;
    template <class T> DPX_D static T apply(T x)
    {
        if constexpr (is_cplx_v<T>) {
            using R = real_of_t<T>;
            if (x.re == R(0) && x.im == R(0)) return T{R(0), R(0)};
            const R a = m_hypot(x.re, x.im);
            return T{x.re / a, x.im / a};
        }
        else if constexpr (is_uint_v<T>) return (T)(x > 0);
        else if constexpr (is_fp_v<T>) return (x != x) ? x : (T)((T(0) < x) - (x < T(0)));
        else return (T)((T(0) < x) - (x < T(0)));
    }
};
template <int WHICH> struct FpClassOp { // isnan.hpp / isinf.hpp / isfinite.hpp -> bool
    template <class T> static constexpr bool ok = true;
    template <class T> using out = bool_t;
    template <class T> DPX_D static bool apply(V<T> x)
    {
        if constexpr (is_cplx_v<T>) {
            bool n = isnan_(x), i = m_isinf(x.re) || m_isinf(x.im);
            if constexpr (WHICH == 0) return n;
            else if constexpr (WHICH == 1) return i;
            else return !n && !i;
        }
        else if constexpr (is_fp_v<T>) {
            if constexpr (WHICH == 0) return x != x;
            else if constexpr (WHICH == 1) return m_isinf(x);
            else return !(x != x) && !m_isinf(x);
        }
        else return WHICH == 2;
    }
};
struct LogicalNotOp {
    template <class T> static constexpr bool ok = true;
    template <class T> using out = bool_t;
    template <class T> DPX_D static bool apply(V<T> x) { return !convert<bool_t, T>(to_storage<T>(x)).v; }
};
struct InvertOp { // bitwise_invert.hpp: bool -> logical not, ints -> ~x
    template <class T> static constexpr bool ok = is_bool_v<T> || is_int_v<T>;
    template <class T> using out = T;
    template <class T> DPX_D static V<T> apply(V<T> x)
    {
        if constexpr (is_bool_v<T>) return !x;
        else return (T)~x;
    }
};
struct SignbitOp {
    template <class T> static constexpr bool ok = is_fp_v<T>;
    template <class T> using out = bool_t;
    template <class T> DPX_D static bool apply(T x) { return m_signbit(x); }
};

struct RoundOp2 { // round.hpp:74-96: rint (ties to even) on floats and complex parts, identity on ints
    template <class T> static constexpr bool ok = !is_bool_v<T>;
    template <class T> using out = T;
    template <class T> DPX_D static T apply(T x)
    {
        if constexpr (is_cplx_v<T>) return T{m_rint(x.re), m_rint(x.im)};
        else if constexpr (is_fp_v<T>) return m_rint(x);
        else return x;
    }
};
struct ConjOp { // conj.hpp: bool -> int8, real types unchanged
    template <class T> static constexpr bool ok = true;
    template <class T> using out = std::conditional_t<is_bool_v<T>, int8_t, T>;
    template <class T> DPX_D static V<out<T>> apply(V<T> x)
    {
        if constexpr (is_bool_v<T>) return (int8_t)(x ? 1 : 0);
        else if constexpr (is_cplx_v<T>) return T{x.re, -x.im};
        else return x;
    }
};
template <bool IMAG> struct PartOp { // real.hpp / imag.hpp: complex -> its real type, others unchanged (imag: zero)
    template <class T> static constexpr bool ok = true;
    template <class T> using out = real_of_t<T>;
    template <class T> DPX_D static V<out<T>> apply(V<T> x)
    {
        if constexpr (is_cplx_v<T>) return IMAG ? x.im : x.re;
        else if constexpr (IMAG) return V<T>(0);
        else return x;
    }
};
struct ProjOp { // proj.hpp: complex only; infinities map to (inf, copysign(0, im))
    template <class T> static constexpr bool ok = is_cplx_v<T>;
    template <class T> using out = T;
    template <class T> DPX_D static T apply(T x)
    {
        using R = real_of_t<T>;
        if (m_isinf(x.re) || m_isinf(x.im)) return T{(R)__builtin_inff(), m_copysign(R(0), x.im)};
        return x;
    }
};
struct AngleOp { // angle.hpp: complex -> real, atan2(im, re)
    template <class T> static constexpr bool ok = is_cplx_v<T>;
    template <class T> using out = real_of_t<T>;
    template <class T> DPX_D static real_of_t<T> apply(T x) { return m_atan2(x.im, x.re); }
};
struct LogaddexpOp { // logaddexp.hpp with libtensor/include/utils/math_utils.hpp:129-150
    template <class T> static constexpr bool ok = is_fp_v<T>;
    template <class T> using out = T;
    template <class T> DPX_D static T apply(T x, T y)
    {
        if constexpr (std::is_same_v<T, half_t>) {
            // float16: the same formula on the hardware's float exp2 and log2 (absolute error 1e-7 in a term of
            // at most ln 2, far below a float16 ULP of the result's operands): 10 vector instructions for 35
            const float xf = (float)x, yf = (float)y, d = xf - yf;
            const float e = __builtin_amdgcn_exp2f(-__builtin_fabsf(d) * 1.44269504088896340736f);
            const float r = (d > 0.0f ? xf : yf) + __builtin_amdgcn_logf(1.0f + e) * 0.69314718055994530942f;
            return (half_t)((xf == yf) ? xf + 0.69314718055994530942f : r);
        }
        // one evaluation serves both orders of the operands (a wave with lanes of both kinds ran two):
        // max + log1p(exp(-|d|)); a NaN operand passes
        // through the arithmetic as NaN and the equal case is picked at the end
        const T d = x - y;
        const T hi = d > T(0) ? x : y;
        const T r = hi + m_log1p(m_exp(d > T(0) ? -d : d));
        return (x == y) ? x + T(0.693147180559945309417232121458176568) : r; // equal, also equal infinities
    }
};
struct NextafterOp {
    template <class T> static constexpr bool ok = is_fp_v<T>;
    template <class T> using out = T;
    template <class T> DPX_D static T apply(T x, T y)
    {
        if constexpr (std::is_same_v<T, half_t>) {
            // step in half precision: operate on the 16-bit pattern
            if (x != x || y != y) return x + y;
            if (x == y) return y;
            union { half_t h; uint16_t u; } v;
            v.h = x;
            if (x == half_t(0)) { v.u = (uint16_t)((y < half_t(0)) ? 0x8001 : 0x0001); return v.h; }
            const bool up = (x < y) == (x > half_t(0));
            v.u = (uint16_t)(up ? v.u + 1 : v.u - 1);
            return v.h;
        }
        else return m_nextafter(x, y);
    }
};


struct FabsOp { // fabs.hpp: real floating types
    template <class T> static constexpr bool ok = is_fp_v<T>;
    template <class T> using out = T;
    template <class T> DPX_D static T apply(T x) { return m_copysign(x, T(1)); }
};
template <bool TO_DEG> struct DegreesOp { // degrees.hpp / radians.hpp
    template <class T> static constexpr bool ok = is_fp_v<T>;
    template <class T> using out = T;
    template <class T> DPX_D static T apply(T x)
    {
        if constexpr (std::is_same_v<T, half_t>) return (half_t)apply<float>((float)x);
        else {
            constexpr T k = TO_DEG ? T(57.295779513082320876798154814105170332) : T(0.017453292519943295769236907684886127134);
            return x * k;
        }
    }
};
struct SincOp { // sinc.hpp: sin(pi x) / (pi x), 1 at 0
    template <class T> static constexpr bool ok = is_fp_v<T> || is_cplx_v<T>;
    template <class T> using out = T;
    template <class T> DPX_D static T apply(T x)
    {
        if constexpr (is_cplx_v<T>) {
            using R = real_of_t<T>;
            constexpr R pi = R(3.1415926535897932384626433832795029);
            const T y{pi * x.re, pi * x.im};
            if (y.re == R(0) && y.im == R(0)) return T{R(1), R(0)};
            return c_sin(y) / y;
        }
        else if constexpr (std::is_same_v<T, half_t>) return (half_t)apply<float>((float)x);
        else {
            constexpr T pi = T(3.1415926535897932384626433832795029);
            const T y = pi * x;
            if (y == T(0)) return T(1);
            return m_sinpi(x) / y;
        }
    }
};
struct SpacingOp { // spacing.hpp: distance to the next representable value away from zero
    template <class T> static constexpr bool ok = is_fp_v<T>;
    template <class T> using out = T;
    template <class T> DPX_D static T apply(T x)
    {
        if (x != x) return x;
        if (m_isinf(x)) return (T)__builtin_nanf("");
        const T inf = (T)__builtin_inff();
        // float16 steps towards +inf whatever the sign (as NumPy does)
        if constexpr (std::is_same_v<T, half_t>) return NextafterOp::apply<T>(x, inf) - x;
        else return m_nextafter(x, m_copysign(inf, x)) - x;
    }
};
struct BitCountOp { // bitwise_count.hpp: set bits of |x| -> uint8
    template <class T> static constexpr bool ok = is_int_v<T>;
    template <class T> using out = uint8_t;
    template <class T> DPX_D static uint8_t apply(T x)
    {
        using U = std::make_unsigned_t<T>;
        const U u = x < T(0) ? (U)0 - (U)x : (U)x;
        return (uint8_t)__popcll((unsigned long long)u);
    }
};
// erf.hpp:52-95 (erfc, erfcx, erfinv, erfcinv) and i0.hpp; float16 input computes and returns float32
// for the erf family
template <int WHICH> struct ErfFamilyOp {
    template <class T> static constexpr bool ok = is_fp_v<T>;
    template <class T> using out = std::conditional_t<std::is_same_v<T, half_t>, float, T>;
    template <class T> DPX_D static out<T> apply(T x)
    {
        const out<T> v = (out<T>)x;
        if constexpr (WHICH == 0) return m_erfc(v);
        else if constexpr (WHICH == 1) return m_erfcx(v);
        else if constexpr (WHICH == 2) return m_erfinv(v);
        else return m_erfcinv(v);
    }
};
struct I0Op {
    template <class T> static constexpr bool ok = is_fp_v<T>;
    template <class T> using out = T;
    template <class T> DPX_D static T apply(T x) { return m_i0(x); }
};

// ---- functions of the reference's ufunc extension (dpnp/backend/extensions/ufunc) -------------
template <bool IS_MAX> struct FmaxOp { // dpnp/backend/kernels/elementwise_functions/fmax.hpp, fmin.hpp: NaN loses
    template <class T> static constexpr bool ok = true;
    template <class T> using out = T;
    template <class T> DPX_D static V<T> apply(V<T> a, V<T> b)
    {
        if constexpr (is_cplx_v<T>) {
            // fmax.hpp: keep a when b holds a NaN or a >= b (lexicographic order)
            if constexpr (IS_MAX) return (isnan_(b.re) || isnan_(b.im) || c_greater_eq(a, b)) ? a : b;
            else return (isnan_(b.re) || isnan_(b.im) || c_less_eq(a, b)) ? a : b;
        }
        else if constexpr (is_fp_v<T>) return IS_MAX ? m_fmax(a, b) : m_fmin(a, b);
        else if constexpr (is_bool_v<T>) return IS_MAX ? (a || b) : (a && b);
        else return IS_MAX ? (a >= b ? a : b) : (a <= b ? a : b);
    }
};
struct FmodOp { // fmod.hpp: C remainder (sign of the dividend); integer x fmod 0 == 0; bool -> int8
    template <class T> static constexpr bool ok = !is_cplx_v<T>;
    template <class T> using out = std::conditional_t<is_bool_v<T>, int8_t, T>;
    template <class T> DPX_D static out<T> apply(V<T> a, V<T> b)
    {
        if constexpr (is_fp_v<T>) return m_fmod(a, b);
        else if constexpr (is_bool_v<T>) return (int8_t)0; // {0,1} % 1 == 0 and x % 0 == 0
        else {
            if (b == T(0)) return T(0);
            if constexpr (std::is_signed_v<T>)
                if (b == T(-1)) return T(0); // also keeps INT_MIN % -1 away from the hardware division
            return (T)(a % b);
        }
    }
};
struct Logaddexp2Op { // logaddexp2.hpp: log2(2**x + 2**y)
    template <class T> static constexpr bool ok = is_fp_v<T>;
    template <class T> using out = T;
    template <class T> DPX_D static T apply(T x, T y)
    {
        if constexpr (std::is_same_v<T, half_t>) { // (as in LogaddexpOp)
            const float xf = (float)x, yf = (float)y, d = xf - yf;
            const float e = __builtin_amdgcn_exp2f(-__builtin_fabsf(d));
            const float r = (d > 0.0f ? xf : yf) + __builtin_amdgcn_logf(1.0f + e);
            return (half_t)((xf == yf) ? xf + 1.0f : r);
        }
        constexpr T log2e = T(1.442695040888963407359924681001892137);
        const T d = x - y; // as in LogaddexpOp: one evaluation for both orders
        const T hi = d > T(0) ? x : y;
        const T r = hi + log2e * m_log1p(m_exp2(d > T(0) ? -d : d));
        return (x == y) ? x + T(1) : r; // equal, also equal infinities
    }
};
struct HeavisideOp { // heaviside.hpp: NaN -> NaN, 0 -> second argument, else x > 0
    template <class T> static constexpr bool ok = is_fp_v<T>;
    template <class T> using out = T;
    template <class T> DPX_D static T apply(T a, T b)
    {
        if (a != a) return a;
        if (a == T(0)) return b;
        return a > T(0) ? T(1) : T(0);
    }
};
template <bool LCM> struct GcdOp { // gcd.hpp / lcm.hpp: integers; the result is non-negative
    template <class T> static constexpr bool ok = is_int_v<T>;
    template <class T> using out = T;
    template <class T> DPX_D static T apply(T a, T b)
    {
        using U = std::make_unsigned_t<T>;
        U x = a < T(0) ? (U)0 - (U)a : (U)a, y = b < T(0) ? (U)0 - (U)b : (U)b;
        const U ax = x, ay = y;
        while (y != 0) {
            const U t = x % y;
            x = y;
            y = t;
        }
        if constexpr (!LCM) return (T)x;
        else return x == 0 ? T(0) : (T)(ax / x * ay);
    }
};

// Arithmetic on operands of two different types with the conversion folded into the load:
// (A, B) -> T where one operand already has the result type T, or (float32 with int32 / int64 -> float64)
// neither has.  The reference has same-type
// kernels only and its Python layer casts the other operand into a temporary first
// (_find_buf_dtype2, dpnp/tensor/_type_utils.py:389-485); converting while reading gives the same
// values without the extra pass.  f(tag<T>, tag<A>, tag<B>) is called for a supported pair.
inline bool is_mixed_arith(int op)
{
    return op == DPX_B_ADD || op == DPX_B_SUBTRACT || op == DPX_B_MULTIPLY || op == DPX_B_DIVIDE;
}
template <class F> inline bool for_mixed_pair(int dt1, int dt2, F &&f)
{
#define DPX_MIX(T, X)                                       \
    if (dt1 == id_of_v<T> && dt2 == id_of_v<X>) {           \
        f(tag<T>{}, tag<T>{}, tag<X>{});                    \
        return true;                                        \
    }                                                       \
    if (dt1 == id_of_v<X> && dt2 == id_of_v<T>) {           \
        f(tag<T>{}, tag<X>{}, tag<T>{});                    \
        return true;                                        \
    }
    DPX_MIX(double, float) DPX_MIX(double, int32_t) DPX_MIX(double, int64_t) DPX_MIX(double, bool_t)
    DPX_MIX(float, bool_t) DPX_MIX(float, int16_t) DPX_MIX(float, int8_t) DPX_MIX(float, uint8_t)
#undef DPX_MIX
    // both operands converted: float32 with a 32- or 64-bit integer gives float64
#define DPX_MIX3(T, X, Y)                                   \
    if (dt1 == id_of_v<X> && dt2 == id_of_v<Y>) {           \
        f(tag<T>{}, tag<X>{}, tag<Y>{});                    \
        return true;                                        \
    }                                                       \
    if (dt1 == id_of_v<Y> && dt2 == id_of_v<X>) {           \
        f(tag<T>{}, tag<Y>{}, tag<X>{});                    \
        return true;                                        \
    }
    DPX_MIX3(double, float, int32_t) DPX_MIX3(double, float, int64_t)
#undef DPX_MIX3
    return false;
}
template <class Op, class T, class A, class B> struct MixedFn {
    DPX_D V<T> operator()(V<A> a, V<B> b) const
    {
        return Op::template apply<T>(to_value(convert<T, A>(to_storage<A>(a))),
                                     to_value(convert<T, B>(to_storage<B>(b))));
    }
};

// op id -> op struct; f(tag<Op>{}) is called for a valid id.  A translation unit built with
// -DDPX_GROUP=g -DDPX_NGROUPS=n instantiates f only for the ids with id % n == g (the others
// still return true, without a call), so the kernels of an op are compiled exactly once.
#ifdef DPX_GROUP
constexpr bool op_in_group(int id) { return id % DPX_NGROUPS == DPX_GROUP; }
#else
constexpr bool op_in_group(int) { return true; }
#endif
template <class F> inline bool for_binary_op(int op, F &&f)
{
    switch (op) {
    case DPX_B_ADD: if constexpr (op_in_group(DPX_B_ADD)) f(tag<AddOp>{}); return true;
    case DPX_B_SUBTRACT: if constexpr (op_in_group(DPX_B_SUBTRACT)) f(tag<SubOp>{}); return true;
    case DPX_B_MULTIPLY: if constexpr (op_in_group(DPX_B_MULTIPLY)) f(tag<MulOp>{}); return true;
    case DPX_B_DIVIDE: if constexpr (op_in_group(DPX_B_DIVIDE)) f(tag<DivOp>{}); return true;
    case DPX_B_BITWISE_AND: if constexpr (op_in_group(DPX_B_BITWISE_AND)) f(tag<BitOp<0>>{}); return true;
    case DPX_B_BITWISE_OR: if constexpr (op_in_group(DPX_B_BITWISE_OR)) f(tag<BitOp<1>>{}); return true;
    case DPX_B_BITWISE_XOR: if constexpr (op_in_group(DPX_B_BITWISE_XOR)) f(tag<BitOp<2>>{}); return true;
    case DPX_B_EQUAL: if constexpr (op_in_group(DPX_B_EQUAL)) f(tag<CmpOp<0>>{}); return true;
    case DPX_B_NOT_EQUAL: if constexpr (op_in_group(DPX_B_NOT_EQUAL)) f(tag<CmpOp<1>>{}); return true;
    case DPX_B_LESS: if constexpr (op_in_group(DPX_B_LESS)) f(tag<CmpOp<2>>{}); return true;
    case DPX_B_LESS_EQUAL: if constexpr (op_in_group(DPX_B_LESS_EQUAL)) f(tag<CmpOp<3>>{}); return true;
    case DPX_B_GREATER: if constexpr (op_in_group(DPX_B_GREATER)) f(tag<CmpOp<4>>{}); return true;
    case DPX_B_GREATER_EQUAL: if constexpr (op_in_group(DPX_B_GREATER_EQUAL)) f(tag<CmpOp<5>>{}); return true;
    case DPX_B_MAXIMUM: if constexpr (op_in_group(DPX_B_MAXIMUM)) f(tag<MaxOp>{}); return true;
    case DPX_B_MINIMUM: if constexpr (op_in_group(DPX_B_MINIMUM)) f(tag<MinOp>{}); return true;
    case DPX_B_LOGICAL_AND: if constexpr (op_in_group(DPX_B_LOGICAL_AND)) f(tag<LogicalOp<0>>{}); return true;
    case DPX_B_LOGICAL_OR: if constexpr (op_in_group(DPX_B_LOGICAL_OR)) f(tag<LogicalOp<1>>{}); return true;
    case DPX_B_LOGICAL_XOR: if constexpr (op_in_group(DPX_B_LOGICAL_XOR)) f(tag<LogicalOp<2>>{}); return true;
    case DPX_B_POW: if constexpr (op_in_group(DPX_B_POW)) f(tag<PowOp>{}); return true;
    case DPX_B_FLOOR_DIVIDE: if constexpr (op_in_group(DPX_B_FLOOR_DIVIDE)) f(tag<FloorDivOp>{}); return true;
    case DPX_B_REMAINDER: if constexpr (op_in_group(DPX_B_REMAINDER)) f(tag<RemainderOp>{}); return true;
    case DPX_B_ATAN2: if constexpr (op_in_group(DPX_B_ATAN2)) f(tag<Atan2Op>{}); return true;
    case DPX_B_HYPOT: if constexpr (op_in_group(DPX_B_HYPOT)) f(tag<HypotOp>{}); return true;
    case DPX_B_COPYSIGN: if constexpr (op_in_group(DPX_B_COPYSIGN)) f(tag<CopysignOp>{}); return true;
    case DPX_B_LEFT_SHIFT: if constexpr (op_in_group(DPX_B_LEFT_SHIFT)) f(tag<ShiftOp<true>>{}); return true;
    case DPX_B_RIGHT_SHIFT: if constexpr (op_in_group(DPX_B_RIGHT_SHIFT)) f(tag<ShiftOp<false>>{}); return true;
    case DPX_B_LOGADDEXP: if constexpr (op_in_group(DPX_B_LOGADDEXP)) f(tag<LogaddexpOp>{}); return true;
    case DPX_B_NEXTAFTER: if constexpr (op_in_group(DPX_B_NEXTAFTER)) f(tag<NextafterOp>{}); return true;
    case DPX_B_FMAX: if constexpr (op_in_group(DPX_B_FMAX)) f(tag<FmaxOp<true>>{}); return true;
    case DPX_B_FMIN: if constexpr (op_in_group(DPX_B_FMIN)) f(tag<FmaxOp<false>>{}); return true;
    case DPX_B_FMOD: if constexpr (op_in_group(DPX_B_FMOD)) f(tag<FmodOp>{}); return true;
    case DPX_B_LOGADDEXP2: if constexpr (op_in_group(DPX_B_LOGADDEXP2)) f(tag<Logaddexp2Op>{}); return true;
    case DPX_B_HEAVISIDE: if constexpr (op_in_group(DPX_B_HEAVISIDE)) f(tag<HeavisideOp>{}); return true;
    case DPX_B_GCD: if constexpr (op_in_group(DPX_B_GCD)) f(tag<GcdOp<false>>{}); return true;
    case DPX_B_LCM: if constexpr (op_in_group(DPX_B_LCM)) f(tag<GcdOp<true>>{}); return true;
    default: return false;
    }
}
template <class F> inline bool for_unary_op(int op, F &&f)
{
    switch (op) {
    case DPX_U_ABS: if constexpr (op_in_group(DPX_U_ABS)) f(tag<AbsOp>{}); return true;
    case DPX_U_NEGATIVE: if constexpr (op_in_group(DPX_U_NEGATIVE)) f(tag<NegOp>{}); return true;
    case DPX_U_POSITIVE: if constexpr (op_in_group(DPX_U_POSITIVE)) f(tag<PosOp>{}); return true;
    case DPX_U_SQUARE: if constexpr (op_in_group(DPX_U_SQUARE)) f(tag<SquareOp>{}); return true;
    case DPX_U_SQRT: if constexpr (op_in_group(DPX_U_SQRT)) f(tag<SqrtOp>{}); return true;
    case DPX_U_EXP: if constexpr (op_in_group(DPX_U_EXP)) f(tag<ExpOp>{}); return true;
    case DPX_U_LOG: if constexpr (op_in_group(DPX_U_LOG)) f(tag<LogOp>{}); return true;
    case DPX_U_ERF: if constexpr (op_in_group(DPX_U_ERF)) f(tag<ErfOp>{}); return true;
    case DPX_U_SIN: if constexpr (op_in_group(DPX_U_SIN)) f(tag<SinOp>{}); return true;
    case DPX_U_COS: if constexpr (op_in_group(DPX_U_COS)) f(tag<CosOp>{}); return true;
    case DPX_U_TAN: if constexpr (op_in_group(DPX_U_TAN)) f(tag<TanOp>{}); return true;
    case DPX_U_TANH: if constexpr (op_in_group(DPX_U_TANH)) f(tag<TanhOp>{}); return true;
    case DPX_U_EXP2: if constexpr (op_in_group(DPX_U_EXP2)) f(tag<Exp2Op>{}); return true;
    case DPX_U_EXPM1: if constexpr (op_in_group(DPX_U_EXPM1)) f(tag<Expm1Op>{}); return true;
    case DPX_U_LOG2: if constexpr (op_in_group(DPX_U_LOG2)) f(tag<Log2Op>{}); return true;
    case DPX_U_LOG10: if constexpr (op_in_group(DPX_U_LOG10)) f(tag<Log10Op>{}); return true;
    case DPX_U_LOG1P: if constexpr (op_in_group(DPX_U_LOG1P)) f(tag<Log1pOp>{}); return true;
    case DPX_U_RSQRT: if constexpr (op_in_group(DPX_U_RSQRT)) f(tag<RsqrtOp>{}); return true;
    case DPX_U_CBRT: if constexpr (op_in_group(DPX_U_CBRT)) f(tag<CbrtOp>{}); return true;
    case DPX_U_RECIPROCAL: if constexpr (op_in_group(DPX_U_RECIPROCAL)) f(tag<ReciprocalOp>{}); return true;
    case DPX_U_FLOOR: if constexpr (op_in_group(DPX_U_FLOOR)) f(tag<RoundOp<0>>{}); return true;
    case DPX_U_CEIL: if constexpr (op_in_group(DPX_U_CEIL)) f(tag<RoundOp<1>>{}); return true;
    case DPX_U_TRUNC: if constexpr (op_in_group(DPX_U_TRUNC)) f(tag<RoundOp<2>>{}); return true;
    case DPX_U_SIGN: if constexpr (op_in_group(DPX_U_SIGN)) f(tag<SignOp>{}); return true;
    case DPX_U_ISNAN: if constexpr (op_in_group(DPX_U_ISNAN)) f(tag<FpClassOp<0>>{}); return true;
    case DPX_U_ISINF: if constexpr (op_in_group(DPX_U_ISINF)) f(tag<FpClassOp<1>>{}); return true;
    case DPX_U_ISFINITE: if constexpr (op_in_group(DPX_U_ISFINITE)) f(tag<FpClassOp<2>>{}); return true;
    case DPX_U_LOGICAL_NOT: if constexpr (op_in_group(DPX_U_LOGICAL_NOT)) f(tag<LogicalNotOp>{}); return true;
    case DPX_U_BITWISE_INVERT: if constexpr (op_in_group(DPX_U_BITWISE_INVERT)) f(tag<InvertOp>{}); return true;
    case DPX_U_SIGNBIT: if constexpr (op_in_group(DPX_U_SIGNBIT)) f(tag<SignbitOp>{}); return true;
    case DPX_U_ASIN: if constexpr (op_in_group(DPX_U_ASIN)) f(tag<AsinOp>{}); return true;
    case DPX_U_ACOS: if constexpr (op_in_group(DPX_U_ACOS)) f(tag<AcosOp>{}); return true;
    case DPX_U_ATAN: if constexpr (op_in_group(DPX_U_ATAN)) f(tag<AtanOp>{}); return true;
    case DPX_U_SINH: if constexpr (op_in_group(DPX_U_SINH)) f(tag<SinhOp>{}); return true;
    case DPX_U_COSH: if constexpr (op_in_group(DPX_U_COSH)) f(tag<CoshOp>{}); return true;
    case DPX_U_ASINH: if constexpr (op_in_group(DPX_U_ASINH)) f(tag<AsinhOp>{}); return true;
    case DPX_U_ACOSH: if constexpr (op_in_group(DPX_U_ACOSH)) f(tag<AcoshOp>{}); return true;
    case DPX_U_ATANH: if constexpr (op_in_group(DPX_U_ATANH)) f(tag<AtanhOp>{}); return true;
    case DPX_U_ROUND: if constexpr (op_in_group(DPX_U_ROUND)) f(tag<RoundOp2>{}); return true;
    case DPX_U_CONJ: if constexpr (op_in_group(DPX_U_CONJ)) f(tag<ConjOp>{}); return true;
    case DPX_U_REAL: if constexpr (op_in_group(DPX_U_REAL)) f(tag<PartOp<false>>{}); return true;
    case DPX_U_IMAG: if constexpr (op_in_group(DPX_U_IMAG)) f(tag<PartOp<true>>{}); return true;
    case DPX_U_PROJ: if constexpr (op_in_group(DPX_U_PROJ)) f(tag<ProjOp>{}); return true;
    case DPX_U_ANGLE: if constexpr (op_in_group(DPX_U_ANGLE)) f(tag<AngleOp>{}); return true;
    case DPX_U_FABS: if constexpr (op_in_group(DPX_U_FABS)) f(tag<FabsOp>{}); return true;
    case DPX_U_DEGREES: if constexpr (op_in_group(DPX_U_DEGREES)) f(tag<DegreesOp<true>>{}); return true;
    case DPX_U_RADIANS: if constexpr (op_in_group(DPX_U_RADIANS)) f(tag<DegreesOp<false>>{}); return true;
    case DPX_U_SINC: if constexpr (op_in_group(DPX_U_SINC)) f(tag<SincOp>{}); return true;
    case DPX_U_SPACING: if constexpr (op_in_group(DPX_U_SPACING)) f(tag<SpacingOp>{}); return true;
    case DPX_U_BITWISE_COUNT: if constexpr (op_in_group(DPX_U_BITWISE_COUNT)) f(tag<BitCountOp>{}); return true;
    case DPX_U_ERFC: if constexpr (op_in_group(DPX_U_ERFC)) f(tag<ErfFamilyOp<0>>{}); return true;
    case DPX_U_ERFCX: if constexpr (op_in_group(DPX_U_ERFCX)) f(tag<ErfFamilyOp<1>>{}); return true;
    case DPX_U_ERFINV: if constexpr (op_in_group(DPX_U_ERFINV)) f(tag<ErfFamilyOp<2>>{}); return true;
    case DPX_U_ERFCINV: if constexpr (op_in_group(DPX_U_ERFCINV)) f(tag<ErfFamilyOp<3>>{}); return true;
    case DPX_U_I0: if constexpr (op_in_group(DPX_U_I0)) f(tag<I0Op>{}); return true;
    default: return false;
    }
}

} // namespace dpx
