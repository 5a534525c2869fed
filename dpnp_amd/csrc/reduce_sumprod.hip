// Sum-like reductions: tri._sum_over_axis / _prod_over_axis
// (libtensor/source/reductions/sum.cpp, prod.cpp) and the squared-deviation pass of var.
// Built twice: -DDPX_KIND_PROD=0 (sum, sumsqdev) and -DDPX_KIND_PROD=1 (prod).
#include "reduce_dispatch.hpp"

#ifndef DPX_KIND_PROD
#define DPX_KIND_PROD 0
#endif

namespace dpx {

// (input, result) pairs with a kernel.  Everything else is reached by the Python layer
// through a cast of the input or of the result (dpnp/tensor/_reduction.py:236-281), which
// gives the same value for integers and a more accurate one for floats.
template <class F> static bool for_sum_pair(int in_dt, int out_dt, F &&f)
{
    bool hit = false;
#define DPX_PAIR(I, O)                                                      \
    if (!hit && in_dt == id_of_v<I> && out_dt == id_of_v<O>) {              \
        f(tag<I>{}, tag<O>{});                                              \
        hit = true;                                                         \
    }
    DPX_PAIR(bool_t, bool_t) DPX_PAIR(int8_t, int8_t) DPX_PAIR(uint8_t, uint8_t) DPX_PAIR(int16_t, int16_t)
    DPX_PAIR(uint16_t, uint16_t) DPX_PAIR(int32_t, int32_t) DPX_PAIR(uint32_t, uint32_t)
    DPX_PAIR(int64_t, int64_t) DPX_PAIR(uint64_t, uint64_t) DPX_PAIR(half_t, half_t) DPX_PAIR(float, float)
    DPX_PAIR(double, double) DPX_PAIR(c64, c64) DPX_PAIR(c128, c128)
    // default accumulation types (_default_accumulation_dtype, dpnp/tensor/_type_utils.py:932-952)
    DPX_PAIR(bool_t, int64_t) DPX_PAIR(int8_t, int64_t) DPX_PAIR(int16_t, int64_t) DPX_PAIR(int32_t, int64_t)
    DPX_PAIR(uint8_t, uint64_t) DPX_PAIR(uint16_t, uint64_t) DPX_PAIR(uint32_t, uint64_t)
    // wider floating accumulation (sum.cpp:130-241 lists these among others)
    DPX_PAIR(half_t, float) DPX_PAIR(half_t, double) DPX_PAIR(float, double) DPX_PAIR(c64, c128)
    // integers and bool summed in floating point: what mean() of an integer array asks for
    // (dpnp/tensor/_statistical_functions.py:166-270 sums with dtype float64), in one pass
    DPX_PAIR(bool_t, double) DPX_PAIR(int8_t, double) DPX_PAIR(uint8_t, double) DPX_PAIR(int16_t, double)
    DPX_PAIR(uint16_t, double) DPX_PAIR(int32_t, double) DPX_PAIR(uint32_t, double) DPX_PAIR(int64_t, double)
    DPX_PAIR(uint64_t, double) DPX_PAIR(bool_t, float) DPX_PAIR(int8_t, float) DPX_PAIR(uint8_t, float)
    DPX_PAIR(int16_t, float) DPX_PAIR(uint16_t, float) DPX_PAIR(int32_t, float) DPX_PAIR(uint32_t, float)
    DPX_PAIR(int64_t, float) DPX_PAIR(uint64_t, float)
    // the remaining pairs of the reference's tables (sum.cpp:87-241, prod.cpp alike): narrower
    // integer results (the input is converted to the result type, which then wraps), unsigned
    // into signed, real into complex
    DPX_PAIR(bool_t, int8_t) DPX_PAIR(bool_t, uint8_t) DPX_PAIR(bool_t, int16_t) DPX_PAIR(bool_t, uint16_t)
    DPX_PAIR(bool_t, int32_t) DPX_PAIR(bool_t, uint32_t) DPX_PAIR(bool_t, uint64_t)
    DPX_PAIR(int8_t, int16_t) DPX_PAIR(int8_t, int32_t)
    DPX_PAIR(uint8_t, int16_t) DPX_PAIR(uint8_t, uint16_t) DPX_PAIR(uint8_t, int32_t) DPX_PAIR(uint8_t, uint32_t)
    DPX_PAIR(uint8_t, int64_t)
    DPX_PAIR(int16_t, int32_t)
    DPX_PAIR(uint16_t, int32_t) DPX_PAIR(uint16_t, uint32_t) DPX_PAIR(uint16_t, int64_t)
    DPX_PAIR(uint32_t, int64_t)
    DPX_PAIR(half_t, c64) DPX_PAIR(half_t, c128) DPX_PAIR(float, c64) DPX_PAIR(float, c128) DPX_PAIR(double, c128)
#undef DPX_PAIR
    return hit;
}

#if DPX_KIND_PROD
bool prod_pair_supported(int in_dt, int out_dt)
{
    return for_sum_pair(in_dt, out_dt, [](auto, auto) {});
}
int prod_run(RedPlan &pl, const dpx_array_view *src, const dpx_array_view *dst, hipStream_t stream)
{
    int rc = DPX_ERR_NOT_IMPLEMENTED;
    for_sum_pair(src->dtype, dst->dtype, [&](auto it, auto ot) {
        using I = typename decltype(it)::type;
        using O = typename decltype(ot)::type;
        rc = red_run<K_PROD, I, O>(pl, src, dst, nullptr, stream);
    });
    return rc;
}
int prod_acc_size(int in_dt, int out_dt)
{
    int sz = 0;
    for_sum_pair(in_dt, out_dt, [&](auto it, auto ot) {
        sz = (int)sizeof(typename RedPolicy<K_PROD, typename decltype(it)::type, typename decltype(ot)::type>::Acc);
    });
    return sz;
}
#else
bool sum_pair_supported(int in_dt, int out_dt)
{
    return for_sum_pair(in_dt, out_dt, [](auto, auto) {});
}
int sum_run(RedPlan &pl, const dpx_array_view *src, const dpx_array_view *dst, hipStream_t stream)
{
    int rc = DPX_ERR_NOT_IMPLEMENTED;
    for_sum_pair(src->dtype, dst->dtype, [&](auto it, auto ot) {
        using I = typename decltype(it)::type;
        using O = typename decltype(ot)::type;
        rc = red_run<K_SUM, I, O>(pl, src, dst, nullptr, stream);
    });
    return rc;
}
int sum_acc_size(int in_dt, int out_dt)
{
    int sz = 0;
    for_sum_pair(in_dt, out_dt, [&](auto it, auto ot) {
        sz = (int)sizeof(typename RedPolicy<K_SUM, typename decltype(it)::type, typename decltype(ot)::type>::Acc);
    });
    return sz;
}
// sum((x - aux)^2): real floating types, and integers / bool accumulated in double (var of an
// integer array)
template <class F> static bool for_sqdev_pair(int in_dt, int out_dt, F &&f)
{
    bool hit = false;
#define DPX_PAIR(I, O)                                         \
    if (!hit && in_dt == id_of_v<I> && out_dt == id_of_v<O>) { \
        f(tag<I>{}, tag<O>{});                                 \
        hit = true;                                            \
    }
    DPX_PAIR(half_t, half_t) DPX_PAIR(half_t, float) DPX_PAIR(float, float) DPX_PAIR(float, double)
    DPX_PAIR(double, double) DPX_PAIR(bool_t, double) DPX_PAIR(int8_t, double) DPX_PAIR(uint8_t, double)
    DPX_PAIR(int16_t, double) DPX_PAIR(uint16_t, double) DPX_PAIR(int32_t, double) DPX_PAIR(uint32_t, double)
    DPX_PAIR(int64_t, double) DPX_PAIR(uint64_t, double)
    // complex input, complex aux: sum(|z - aux|^2), a real result
    DPX_PAIR(c64, float) DPX_PAIR(c64, double) DPX_PAIR(c128, double)
#undef DPX_PAIR
    return hit;
}
bool sqdev_pair_supported(int in_dt, int out_dt)
{
    return for_sqdev_pair(in_dt, out_dt, [](auto, auto) {});
}
int sqdev_acc_size(int in_dt, int out_dt)
{
    int sz = 0;
    for_sqdev_pair(in_dt, out_dt, [&](auto it, auto ot) {
        sz = (int)sizeof(typename RedPolicy<K_SUMSQDEV, typename decltype(it)::type, typename decltype(ot)::type>::Acc);
    });
    return sz;
}
int sqdev_run(RedPlan &pl, const dpx_array_view *src, const dpx_array_view *dst, const dpx_array_view *aux,
              hipStream_t stream)
{
    int rc = DPX_ERR_NOT_IMPLEMENTED;
    for_sqdev_pair(src->dtype, dst->dtype, [&](auto it, auto ot) {
        using I = typename decltype(it)::type;
        using O = typename decltype(ot)::type;
        rc = red_run<K_SUMSQDEV, I, O>(pl, src, dst, aux, stream);
    });
    return rc;
}
#endif

} // namespace dpx
