// where, divide_by_scalar, fill and the fused chains.
#include "ew_dispatch.hpp"
#include "black_scholes.hpp"

namespace dpx {

// ---- where: libtensor/include/kernels/where.hpp:72-262, host libtensor/source/where.cpp:74-247.
// The select moves bit patterns, so x1/x2/dst are instantiated per element size;
// the condition is any dtype, true when non-zero (type_utils.hpp:64-93).
template <class C, class S> struct WhereFn {
    DPX_D S operator()(V<C> c, S a, S b) const { return convert<bool_t, C>(to_storage<C>(c)).v ? a : b; }
};

template <class S> struct rows2_enabled<WhereFn<bool_t, S>> : std::true_type {};

template <class F> static bool for_size_class(int bytes, F &&f)
{
    switch (bytes) {
    case 1: f(tag<uint8_t>{}); return true;
    case 2: f(tag<uint16_t>{}); return true;
    case 4: f(tag<uint32_t>{}); return true;
    case 8: f(tag<uint64_t>{}); return true;
    case 16: f(tag<c128>{}); return true;
    default: return false;
    }
}

static int where_call(const dpx_array_view *cond, const dpx_array_view *x1, const dpx_array_view *x2,
                      const dpx_array_view *dst, void *stream, dpx_plan *plan_out)
{
    if (!view_ok(cond) || !view_ok(x1) || !view_ok(x2) || !view_ok(dst))
        return fail(DPX_ERR_BAD_ARGUMENT, "malformed array descriptor");
    if (x1->dtype != x2->dtype || x1->dtype != dst->dtype)
        return fail(DPX_ERR_BAD_DTYPE, "Value arrays must have the same data type");
    const dpx_array_view *views[4] = {cond, x1, x2, dst};
    int64_t n = 0;
    if (int rc = ew_validate(4, views, n)) return rc;
    int rc = DPX_ERR_NOT_IMPLEMENTED;
    for_dtype(cond->dtype, [&](auto ct) {
        using C = typename decltype(ct)::type;
        for_size_class(itemsize_of(dst->dtype), [&](auto st) {
            using S = typename decltype(st)::type;
            rc = run_ew<WhereFn<C, S>, S, C, S, S>({}, views, (hipStream_t)stream, plan_out);
        });
    });
    return rc;
}

// ---- fused compare + select: dst = (lhs CMP rhs) ? x1 : x2 --------------------------------
template <class Cmp, class T, class S> struct WhereCmpFn {
    DPX_D S operator()(V<T> l, V<T> r, S a, S b) const { return Cmp::template apply<T>(l, r) ? a : b; }
};
// where(x CMP r, x, b): the compared array is also the first choice, read once
template <class Cmp, class T> struct WhereCmpSelfFn {
    DPX_D T operator()(T x, T r, T b) const { return Cmp::template apply<T>(x, r) ? x : b; }
};

template <class Cmp, class T> struct rows2_enabled<WhereCmpSelfFn<Cmp, T>> : std::true_type {};

static int where_compare_call(int cmp_op, const dpx_array_view *lhs, const dpx_array_view *rhs,
                              const dpx_array_view *x1, const dpx_array_view *x2,
                              const dpx_array_view *dst, void *stream)
{
    if (!view_ok(lhs) || !view_ok(rhs) || !view_ok(x1) || !view_ok(x2) || !view_ok(dst))
        return fail(DPX_ERR_BAD_ARGUMENT, "malformed array descriptor");
    if (cmp_op < DPX_B_EQUAL || cmp_op > DPX_B_GREATER_EQUAL)
        return fail(DPX_ERR_BAD_ARGUMENT, "cmp_op is not a comparison");
    if (lhs->dtype != rhs->dtype) return fail(DPX_ERR_BAD_DTYPE, "compared arrays must have the same data type");
    if (x1->dtype != x2->dtype || x1->dtype != dst->dtype)
        return fail(DPX_ERR_BAD_DTYPE, "Value arrays must have the same data type");
    // only the 4- and 8-byte real types: the fused form exists for the hot cases
    const int dt = lhs->dtype;
    if (!(dt == DPX_FLOAT || dt == DPX_DOUBLE || dt == DPX_INT32 || dt == DPX_INT64))
        return fail(DPX_ERR_NOT_IMPLEMENTED, "fused where-compare: unsupported comparison dtype");
    const int vs = itemsize_of(dst->dtype);
    if (vs != 4 && vs != 8) return fail(DPX_ERR_NOT_IMPLEMENTED, "fused where-compare: unsupported value dtype");
    const dpx_array_view *views[5] = {lhs, rhs, x1, x2, dst};
    int64_t n = 0;
    if (int rc = ew_validate(5, views, n)) return rc;
    int rc = DPX_ERR_NOT_IMPLEMENTED;
    const bool self = views_same_logical(lhs, x1);
    const dpx_array_view *views3[4] = {lhs, rhs, x2, dst};
    auto with_cmp = [&](auto cmptag) {
        using Cmp = typename decltype(cmptag)::type;
        auto with_t = [&](auto ttag) {
            using T = typename decltype(ttag)::type;
            if (self) rc = run_ew<WhereCmpSelfFn<Cmp, T>, T, T, T, T>({}, views3, (hipStream_t)stream, nullptr);
            else if (vs == 4) rc = run_ew<WhereCmpFn<Cmp, T, uint32_t>, uint32_t, T, T, uint32_t, uint32_t>({}, views, (hipStream_t)stream, nullptr);
            else rc = run_ew<WhereCmpFn<Cmp, T, uint64_t>, uint64_t, T, T, uint64_t, uint64_t>({}, views, (hipStream_t)stream, nullptr);
        };
        if (dt == DPX_FLOAT) with_t(tag<float>{});
        else if (dt == DPX_DOUBLE) with_t(tag<double>{});
        else if (dt == DPX_INT32) with_t(tag<int32_t>{});
        else with_t(tag<int64_t>{});
    };
    switch (cmp_op) {
    case DPX_B_EQUAL: with_cmp(tag<CmpOp<0>>{}); break;
    case DPX_B_NOT_EQUAL: with_cmp(tag<CmpOp<1>>{}); break;
    case DPX_B_LESS: with_cmp(tag<CmpOp<2>>{}); break;
    case DPX_B_LESS_EQUAL: with_cmp(tag<CmpOp<3>>{}); break;
    case DPX_B_GREATER: with_cmp(tag<CmpOp<4>>{}); break;
    default: with_cmp(tag<CmpOp<5>>{}); break;
    }
    return rc;
}

// ---- divide by scalar: libtensor/source/elementwise_functions/true_divide.cpp:204-430 -------------
template <class T> struct DivScalarFn {
    real_of_t<T> s;
    DPX_D T operator()(T x) const
    {
        if constexpr (is_cplx_v<T>) return T{x.re / s, x.im / s};
        else return x / s;
    }
};

static int divide_by_scalar_call(const dpx_array_view *src, double scalar, const dpx_array_view *dst,
                                 void *stream)
{
    if (!view_ok(src) || !view_ok(dst)) return fail(DPX_ERR_BAD_ARGUMENT, "malformed array descriptor");
    if (src->dtype != dst->dtype)
        return fail(DPX_ERR_BAD_DTYPE, "Destination array has unexpected elemental data type.");
    const dpx_array_view *views[2] = {src, dst};
    int64_t n = 0;
    if (int rc = ew_validate(2, views, n)) return rc;
    hipStream_t s = (hipStream_t)stream;
    switch (src->dtype) {
    case DPX_HALF: return run_ew<DivScalarFn<half_t>, half_t, half_t>({(half_t)scalar}, views, s, nullptr);
    case DPX_FLOAT: return run_ew<DivScalarFn<float>, float, float>({(float)scalar}, views, s, nullptr);
    case DPX_DOUBLE: return run_ew<DivScalarFn<double>, double, double>({scalar}, views, s, nullptr);
    case DPX_CFLOAT: return run_ew<DivScalarFn<c64>, c64, c64>({(float)scalar}, views, s, nullptr);
    case DPX_CDOUBLE: return run_ew<DivScalarFn<c128>, c128, c128>({scalar}, views, s, nullptr);
    default: return fail(DPX_ERR_NOT_IMPLEMENTED, "divide_by_scalar: only floating and complex types");
    }
}

// ---- nan_to_num: dpnp/backend/kernels/elementwise_functions/nan_to_num.hpp:44-104 (scalar
// replacement values; complex elements are treated part by part) ---------------------------------
template <class T> struct NanToNumFn {
    using R = real_of_t<T>;
    R nan, posinf, neginf;
    DPX_D R one(R v) const { return (v != v) ? nan : (m_isinf(v) ? (v > R(0) ? posinf : neginf) : v); }
    DPX_D T operator()(T x) const
    {
        if constexpr (is_cplx_v<T>) return T{one(x.re), one(x.im)};
        else return one(x);
    }
};

static int nan_to_num_call(const dpx_array_view *src, double nan, double posinf, double neginf,
                           const dpx_array_view *dst, void *stream)
{
    if (!view_ok(src) || !view_ok(dst)) return fail(DPX_ERR_BAD_ARGUMENT, "malformed array descriptor");
    if (src->dtype != dst->dtype)
        return fail(DPX_ERR_BAD_DTYPE, "Destination array has unexpected elemental data type.");
    const dpx_array_view *views[2] = {src, dst};
    int64_t n = 0;
    if (int rc = ew_validate(2, views, n)) return rc;
    hipStream_t s = (hipStream_t)stream;
    switch (src->dtype) {
    case DPX_HALF:
        return run_ew<NanToNumFn<half_t>, half_t, half_t>({(half_t)nan, (half_t)posinf, (half_t)neginf}, views, s, nullptr);
    case DPX_FLOAT:
        return run_ew<NanToNumFn<float>, float, float>({(float)nan, (float)posinf, (float)neginf}, views, s, nullptr);
    case DPX_DOUBLE: return run_ew<NanToNumFn<double>, double, double>({nan, posinf, neginf}, views, s, nullptr);
    case DPX_CFLOAT:
        return run_ew<NanToNumFn<c64>, c64, c64>({(float)nan, (float)posinf, (float)neginf}, views, s, nullptr);
    case DPX_CDOUBLE: return run_ew<NanToNumFn<c128>, c128, c128>({nan, posinf, neginf}, views, s, nullptr);
    default: return fail(DPX_ERR_NOT_IMPLEMENTED, "nan_to_num: only floating and complex types");
    }
}

// ---- isclose: dpnp/backend/kernels/elementwise_functions/isclose.hpp:47-92 (scalar tolerances) ---
template <class T> struct IsCloseFn {
    using R = real_of_t<T>;
    R rtol, atol;
    bool equal_nan;
    DPX_D static bool finite(R v) { return v == v && !m_isinf(v); }
    DPX_D bool operator()(T a, T b) const
    {
        if constexpr (is_cplx_v<T>) {
            if (finite(a.re) && finite(a.im) && finite(b.re) && finite(b.im))
                return m_hypot(a.re - b.re, a.im - b.im) <= atol + rtol * m_hypot(b.re, b.im);
            if (a.re != a.re && a.im != a.im && b.re != b.re && b.im != b.im) return equal_nan;
            return a == b;
        }
        else {
            if (finite(a) && finite(b)) {
                const R d = a - b;
                return (d < R(0) ? -d : d) <= atol + rtol * (b < R(0) ? -b : b);
            }
            if (a != a && b != b) return equal_nan;
            return a == b;
        }
    }
};

static int isclose_call(const dpx_array_view *a, const dpx_array_view *b, double rtol, double atol, int equal_nan,
                        const dpx_array_view *dst, void *stream)
{
    if (!view_ok(a) || !view_ok(b) || !view_ok(dst)) return fail(DPX_ERR_BAD_ARGUMENT, "malformed array descriptor");
    if (a->dtype != b->dtype) return fail(DPX_ERR_BAD_DTYPE, "Input arrays must have the same data type");
    if (dst->dtype != DPX_BOOL) return fail(DPX_ERR_BAD_DTYPE, "Destination array has unexpected elemental data type.");
    const dpx_array_view *views[3] = {a, b, dst};
    int64_t n = 0;
    if (int rc = ew_validate(3, views, n)) return rc;
    hipStream_t s = (hipStream_t)stream;
    const bool en = equal_nan != 0;
    switch (a->dtype) {
    case DPX_HALF:
        return run_ew<IsCloseFn<half_t>, bool_t, half_t, half_t>({(half_t)rtol, (half_t)atol, en}, views, s, nullptr);
    case DPX_FLOAT:
        return run_ew<IsCloseFn<float>, bool_t, float, float>({(float)rtol, (float)atol, en}, views, s, nullptr);
    case DPX_DOUBLE: return run_ew<IsCloseFn<double>, bool_t, double, double>({rtol, atol, en}, views, s, nullptr);
    case DPX_CFLOAT: return run_ew<IsCloseFn<c64>, bool_t, c64, c64>({(float)rtol, (float)atol, en}, views, s, nullptr);
    case DPX_CDOUBLE: return run_ew<IsCloseFn<c128>, bool_t, c128, c128>({rtol, atol, en}, views, s, nullptr);
    default: return fail(DPX_ERR_NOT_IMPLEMENTED, "isclose: only floating and complex types");
    }
}

// ---- clip: libtensor/include/kernels/clip.hpp:66-86 (contiguous 89-200, strided 232-290) ------------
// max(x, lo) then min(.., hi); a NaN in x stays, a NaN bound wins; bool: (x || lo) && hi; complex
// through the NaN-propagating lexicographic extrema.
template <class T> struct ClipFn {
    DPX_D V<T> operator()(V<T> x, V<T> lo, V<T> hi) const
    {
        if constexpr (is_cplx_v<T>) return min_nan(max_nan(x, lo), hi);
        else if constexpr (is_bool_v<T>) return (x || lo) && hi;
        else if constexpr (is_fp_v<V<T>>) {
            const V<T> t = (x != x || x > lo) ? x : lo;
            return (t != t || t < hi) ? t : hi;
        }
        else {
            const V<T> t = (x > lo) ? x : lo;
            return (t < hi) ? t : hi;
        }
    }
};

static int clip_call(const dpx_array_view *x, const dpx_array_view *lo, const dpx_array_view *hi,
                     const dpx_array_view *dst, void *stream)
{
    if (!view_ok(x) || !view_ok(lo) || !view_ok(hi) || !view_ok(dst))
        return fail(DPX_ERR_BAD_ARGUMENT, "malformed array descriptor");
    if (x->dtype != lo->dtype || x->dtype != hi->dtype) return fail(DPX_ERR_BAD_DTYPE, "Input arrays must have the same data type");
    if (x->dtype != dst->dtype) return fail(DPX_ERR_BAD_DTYPE, "Destination array has unexpected elemental data type.");
    const dpx_array_view *views[4] = {x, lo, hi, dst};
    int64_t n = 0;
    if (int rc = ew_validate(4, views, n)) return rc;
    int rc = DPX_ERR_NOT_IMPLEMENTED;
    for_dtype(x->dtype, [&](auto tt) {
        using T = typename decltype(tt)::type;
        rc = run_ew<ClipFn<T>, T, T, T, T>({}, views, (hipStream_t)stream, nullptr);
    });
    return rc;
}

// ---- ldexp: dpnp/backend/kernels/elementwise_functions/ldexp.hpp:39-58 -------------------------------
// x1 * 2^x2; an exponent outside the int range gives +inf when positive and 0 otherwise, whatever x1 is
// (as the reference's functor does).
template <class T, class I> struct LdexpFn {
    DPX_D V<T> operator()(V<T> x, I n) const
    {
        if ((I)(int)n == n) {
            if constexpr (std::is_same_v<V<T>, double>) return ::ldexp(x, (int)n);
            else return ::ldexpf(x, (int)n);
        }
        if (n > 0) return (V<T>)__builtin_inff();
        return V<T>(0);
    }
};

static int ldexp_call(const dpx_array_view *a, const dpx_array_view *b, const dpx_array_view *dst, void *stream)
{
    if (!view_ok(a) || !view_ok(b) || !view_ok(dst)) return fail(DPX_ERR_BAD_ARGUMENT, "malformed array descriptor");
    if (dpx_ldexp_result_type(a->dtype, b->dtype) < 0)
        return fail(DPX_ERR_BAD_DTYPE, "ldexp: needs a floating first and a signed integer second operand");
    if (dst->dtype != a->dtype) return fail(DPX_ERR_BAD_DTYPE, "Destination array has unexpected elemental data type.");
    const dpx_array_view *views[3] = {a, b, dst};
    int64_t n = 0;
    if (int rc = ew_validate(3, views, n)) return rc;
    hipStream_t s = (hipStream_t)stream;
    int rc = DPX_ERR_NOT_IMPLEMENTED;
    auto with_int = [&](auto ft) {
        using T = typename decltype(ft)::type;
        switch (b->dtype) {
        case DPX_INT8: rc = run_ew<LdexpFn<T, int8_t>, T, T, int8_t>({}, views, s, nullptr); break;
        case DPX_INT16: rc = run_ew<LdexpFn<T, int16_t>, T, T, int16_t>({}, views, s, nullptr); break;
        case DPX_INT32: rc = run_ew<LdexpFn<T, int32_t>, T, T, int32_t>({}, views, s, nullptr); break;
        case DPX_INT64: rc = run_ew<LdexpFn<T, int64_t>, T, T, int64_t>({}, views, s, nullptr); break;
        default: break;
        }
    };
    switch (a->dtype) {
    case DPX_HALF: with_int(tag<half_t>{}); break;
    case DPX_FLOAT: with_int(tag<float>{}); break;
    case DPX_DOUBLE: with_int(tag<double>{}); break;
    default: break;
    }
    return rc;
}

// ---- frexp: dpnp/backend/kernels/elementwise_functions/frexp.hpp:36-56 ------------------------------
// x = mantissa * 2^exponent with |mantissa| in [0.5, 1); zeros, infinities and NaN come back
// unchanged with exponent 0.  PART 0: the mantissa (type of x), PART 1: the exponent (int32).
template <class T, int PART> struct FrexpFn {
    DPX_D auto operator()(V<T> x) const
    {
        constexpr bool dbl = std::is_same_v<V<T>, double>;
        if constexpr (PART == 0) {
            if constexpr (dbl) return __builtin_amdgcn_frexp_mant(x);
            else return __builtin_amdgcn_frexp_mantf(x);
        }
        else {
            const bool special = !(x == x) || m_isinf(x) || x == V<T>(0);
            int32_t e;
            if constexpr (dbl) e = __builtin_amdgcn_frexp_exp(x);
            else e = __builtin_amdgcn_frexp_expf(x);
            return special ? (int32_t)0 : e;
        }
    }
};

static int frexp_call(const dpx_array_view *x, const dpx_array_view *mant, const dpx_array_view *ex, void *stream)
{
    if (!view_ok(x) || !view_ok(mant) || !view_ok(ex)) return fail(DPX_ERR_BAD_ARGUMENT, "malformed array descriptor");
    if (x->dtype != DPX_HALF && x->dtype != DPX_FLOAT && x->dtype != DPX_DOUBLE)
        return fail(DPX_ERR_BAD_DTYPE, "frexp: only floating types");
    if (mant->dtype != x->dtype || ex->dtype != DPX_INT32)
        return fail(DPX_ERR_BAD_DTYPE, "Destination array has unexpected elemental data type.");
    if (views_overlap(mant, ex)) return fail(DPX_ERR_OVERLAP, "frexp: the two outputs overlap");
    const dpx_array_view *v1[2] = {x, mant}, *v2[2] = {x, ex};
    int64_t n = 0;
    if (int rc = ew_validate(2, v2, n)) return rc; // before anything is written
    if (int rc = ew_validate(2, v1, n)) return rc;
    hipStream_t s = (hipStream_t)stream;
    auto both = [&](auto ft) {
        using T = typename decltype(ft)::type;
        // the exponent first: x may be the mantissa's destination
        if (int rc = run_ew<FrexpFn<T, 1>, int32_t, T>({}, v2, s, nullptr)) return rc;
        return run_ew<FrexpFn<T, 0>, T, T>({}, v1, s, nullptr);
    };
    switch (x->dtype) {
    case DPX_HALF: return both(tag<half_t>{});
    case DPX_FLOAT: return both(tag<float>{});
    default: return both(tag<double>{});
    }
}

// ---- fill ----------------------------------------------------------------------------------------------
template <class T> struct FillFn {
    T v;
    DPX_D V<T> operator()() const { return to_value(v); }
};

static int fill_call(const dpx_array_view *dst, double re, double im, int64_t iv, int use_int, void *stream)
{
    if (!view_ok(dst)) return fail(DPX_ERR_BAD_ARGUMENT, "malformed array descriptor");
    const dpx_array_view *views[1] = {dst};
    int64_t n = 0;
    if (int rc = ew_validate(1, views, n)) return rc;
    int rc = DPX_ERR_NOT_IMPLEMENTED;
    for_dtype(dst->dtype, [&](auto tt) {
        using T = typename decltype(tt)::type;
        T v;
        if constexpr (is_cplx_v<T>) v = T{(real_of_t<T>)(use_int ? (double)iv : re), (real_of_t<T>)(use_int ? 0.0 : im)};
        else if constexpr (is_bool_v<T>) v = bool_t{(uint8_t)(use_int ? iv != 0 : (re != 0.0 || im != 0.0))};
        else if constexpr (is_int_v<T>) v = use_int ? (T)iv : convert<T, double>(re);
        else v = use_int ? (T)iv : (T)re;
        rc = run_ew<FillFn<T>, T>(FillFn<T>{v}, views, (hipStream_t)stream, nullptr);
    });
    return rc;
}

template <class T>
static int black_scholes_call(const void *price, const void *strike, const void *t, double rate, double vol,
                              void *call, void *put, int64_t n, hipStream_t stream)
{
    constexpr int E = 16 / sizeof(T);
    const uintptr_t all = (uintptr_t)price | (uintptr_t)strike | (uintptr_t)t | (uintptr_t)call | (uintptr_t)put;
    if (all % 16 != 0) return fail(DPX_ERR_BAD_ARGUMENT, "black_scholes: arrays must be 16-byte aligned");
    BlackScholesFn<T> fn{(T)(-rate), (T)(vol * vol * 2), (T)0.25, (T)0.5, (T)1};
    if constexpr (std::is_same_v<T, double>) {
        const int64_t nfull = n / ((int64_t)BS_BLOCK * E * BS_PACKS);
        if (nfull + 1 > 0x7fffffff) return fail(DPX_ERR_BAD_ARGUMENT, "black_scholes: too many options for one launch");
        hipLaunchKernelGGL(black_scholes_f64_kernel<BS_WHOLE>, dim3((unsigned)(nfull + 1)), dim3(BS_BLOCK), 0, stream, fn,
                           (const double *)price, (const double *)strike, (const double *)t, (double *)call, (double *)put,
                           n, nfull);
    }
    else {
        const int block = 128;
        const int64_t grid = (n + (int64_t)block * E - 1) / ((int64_t)block * E);
        hipLaunchKernelGGL(black_scholes_kernel<T>, dim3((unsigned)grid), dim3(block), 0, stream, fn, (const T *)price,
                           (const T *)strike, (const T *)t, (T *)call, (T *)put, n);
    }
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? DPX_OK : fail_hip(e, "black_scholes launch");
}

} // namespace dpx

using namespace dpx;
extern "C" {
int dpx_where(const dpx_array_view *cond, const dpx_array_view *x1, const dpx_array_view *x2,
              const dpx_array_view *dst, void *stream)
{
    return where_call(cond, x1, x2, dst, stream, nullptr);
}
int dpx_where_plan(const dpx_array_view *cond, const dpx_array_view *x1, const dpx_array_view *x2,
                   const dpx_array_view *dst, dpx_plan *plan)
{
    if (!plan) return fail(DPX_ERR_BAD_ARGUMENT, "plan is null");
    return where_call(cond, x1, x2, dst, nullptr, plan);
}
int dpx_where_compare(int cmp_op, const dpx_array_view *lhs, const dpx_array_view *rhs, const dpx_array_view *x1,
                      const dpx_array_view *x2, const dpx_array_view *dst, void *stream)
{
    return where_compare_call(cmp_op, lhs, rhs, x1, x2, dst, stream);
}
int dpx_divide_by_scalar(const dpx_array_view *src, double scalar, const dpx_array_view *dst, void *stream)
{
    return divide_by_scalar_call(src, scalar, dst, stream);
}
int dpx_nan_to_num(const dpx_array_view *src, double nan, double posinf, double neginf, const dpx_array_view *dst,
                   void *stream)
{
    return nan_to_num_call(src, nan, posinf, neginf, dst, stream);
}
int dpx_isclose(const dpx_array_view *a, const dpx_array_view *b, double rtol, double atol, int equal_nan,
                const dpx_array_view *dst, void *stream)
{
    return isclose_call(a, b, rtol, atol, equal_nan, dst, stream);
}
int dpx_clip(const dpx_array_view *x, const dpx_array_view *lo, const dpx_array_view *hi, const dpx_array_view *dst,
             void *stream)
{
    return clip_call(x, lo, hi, dst, stream);
}
int dpx_ldexp_result_type(int dt1, int dt2)
{
    const bool fp = dt1 == DPX_HALF || dt1 == DPX_FLOAT || dt1 == DPX_DOUBLE;
    const bool in = dt2 == DPX_INT8 || dt2 == DPX_INT16 || dt2 == DPX_INT32 || dt2 == DPX_INT64;
    return (fp && in) ? dt1 : -1;
}
int dpx_ldexp(const dpx_array_view *x1, const dpx_array_view *x2, const dpx_array_view *dst, void *stream)
{
    return ldexp_call(x1, x2, dst, stream);
}
int dpx_frexp(const dpx_array_view *x, const dpx_array_view *mantissa, const dpx_array_view *exponent, void *stream)
{
    return frexp_call(x, mantissa, exponent, stream);
}
int dpx_fill(const dpx_array_view *dst, double value_re, double value_im, int64_t value_int, int use_int,
             void *stream)
{
    return fill_call(dst, value_re, value_im, value_int, use_int, stream);
}
int dpx_black_scholes(const void *price, const void *strike, const void *t, double rate, double vol, void *call,
                      void *put, int64_t n, int dtype, void *stream)
{
    if (n < 0) return fail(DPX_ERR_BAD_ARGUMENT, "black_scholes: negative length");
    if (n == 0) return DPX_OK;
    if (!price || !strike || !t || !call || !put) return fail(DPX_ERR_BAD_ARGUMENT, "black_scholes: null pointer");
    if (dtype == DPX_DOUBLE)
        return black_scholes_call<double>(price, strike, t, rate, vol, call, put, n, (hipStream_t)stream);
    if (dtype == DPX_FLOAT)
        return black_scholes_call<float>(price, strike, t, rate, vol, call, put, n, (hipStream_t)stream);
    return fail(DPX_ERR_NOT_IMPLEMENTED, "black_scholes: float32 or float64 only");
}
}
