// NaN-ignoring reductions and searches in one pass over the input.  The reference builds
// nansum / nanprod / nanmax / nanmin / nanmean / nanvar / nanargmax / nanargmin from a masked
// copy of the input followed by the plain reduction (dpnp/dpnp_iface_nanfunctions.py:48-116,
// 195-200, 509-518, 600-636, 1318-1390); here the replacement happens as elements are read.
// Floating inputs only: other types hold no NaN and take the plain kernels.
#include "reduce_dispatch.hpp"

namespace dpx {

template <class F> static bool for_nan_pair(int op, int in_dt, int out_dt, F &&f)
{
    bool hit = false;
#define DPX_PAIR(I, O)                                         \
    if (!hit && in_dt == id_of_v<I> && out_dt == id_of_v<O>) { \
        f(tag<I>{}, tag<O>{});                                 \
        hit = true;                                            \
    }
    if (op == DPX_R_NANSUM || op == DPX_R_NANPROD || op == DPX_R_NANMEAN) {
        DPX_PAIR(half_t, half_t) DPX_PAIR(float, float) DPX_PAIR(double, double) DPX_PAIR(c64, c64)
        DPX_PAIR(c128, c128) DPX_PAIR(half_t, float) DPX_PAIR(float, double) DPX_PAIR(c64, c128)
    }
    else if (op == DPX_R_NANMAX || op == DPX_R_NANMIN) {
        DPX_PAIR(half_t, half_t) DPX_PAIR(float, float) DPX_PAIR(double, double)
    }
    else if (op == DPX_R_NANCOUNT) {
        DPX_PAIR(half_t, int64_t) DPX_PAIR(float, int64_t) DPX_PAIR(double, int64_t) DPX_PAIR(c64, int64_t)
        DPX_PAIR(c128, int64_t)
    }
    else if (op == DPX_R_NANSUMSQDEV || op == DPX_R_NANVAR) {
        DPX_PAIR(half_t, half_t) DPX_PAIR(float, float) DPX_PAIR(double, double) DPX_PAIR(half_t, float)
        DPX_PAIR(float, double)
    }
    else if (op == DPX_R_SQDEV_ONEPASS) { // (no NaN handling: it shares this file's plumbing)
        DPX_PAIR(float, double) DPX_PAIR(double, double) DPX_PAIR(half_t, double)
        // integers: var of an integer array is float64 (the reference casts the array first)
        DPX_PAIR(int8_t, double) DPX_PAIR(uint8_t, double) DPX_PAIR(int16_t, double) DPX_PAIR(uint16_t, double)
        DPX_PAIR(int32_t, double) DPX_PAIR(uint32_t, double) DPX_PAIR(int64_t, double) DPX_PAIR(uint64_t, double)
    }
#undef DPX_PAIR
    return hit;
}

bool nan_pair_supported(int op, int in_dt, int out_dt)
{
    return for_nan_pair(op, in_dt, out_dt, [](auto, auto) {});
}

template <int KIND> static int nan_run_kind(int op, RedPlan &pl, const dpx_array_view *src, const dpx_array_view *dst,
                                            const dpx_array_view *aux, hipStream_t stream, int *acc_size)
{
    int rc = DPX_ERR_NOT_IMPLEMENTED;
    for_nan_pair(op, src->dtype, dst->dtype, [&](auto it, auto ot) {
        using I = typename decltype(it)::type;
        using O = typename decltype(ot)::type;
        // the pair lists above keep complex inputs away from the ordered and the squared-deviation kinds
        constexpr bool ok = !(is_cplx_v<I> && (kind_is_minmax(KIND) || KIND == K_NANSUMSQDEV || KIND == K_NANVAR)) &&
                            (KIND == K_NANCOUNT) == std::is_same_v<O, int64_t> &&
                            (KIND == K_SQDEV1 ? (std::is_same_v<O, double> && !is_cplx_v<I>)
                                              : !std::is_integral_v<I>);
        if constexpr (ok) {
            if (acc_size) {
                *acc_size = (int)sizeof(typename RedPolicy<KIND, I, O>::Acc);
                rc = DPX_OK;
            }
            else rc = red_run<KIND, I, O>(pl, src, dst, aux, stream);
        }
    });
    return rc;
}

static int nan_dispatch(int op, RedPlan &pl, const dpx_array_view *src, const dpx_array_view *dst,
                        const dpx_array_view *aux, hipStream_t stream, int *acc_size)
{
    switch (op) {
    case DPX_R_NANSUM: return nan_run_kind<K_NANSUM>(op, pl, src, dst, aux, stream, acc_size);
    case DPX_R_NANPROD: return nan_run_kind<K_NANPROD>(op, pl, src, dst, aux, stream, acc_size);
    case DPX_R_NANMAX: return nan_run_kind<K_NANMAX>(op, pl, src, dst, aux, stream, acc_size);
    case DPX_R_NANMIN: return nan_run_kind<K_NANMIN>(op, pl, src, dst, aux, stream, acc_size);
    case DPX_R_NANCOUNT: return nan_run_kind<K_NANCOUNT>(op, pl, src, dst, aux, stream, acc_size);
    case DPX_R_NANSUMSQDEV: return nan_run_kind<K_NANSUMSQDEV>(op, pl, src, dst, aux, stream, acc_size);
    case DPX_R_NANMEAN: return nan_run_kind<K_NANMEAN>(op, pl, src, dst, aux, stream, acc_size);
    case DPX_R_NANVAR: return nan_run_kind<K_NANVAR>(op, pl, src, dst, aux, stream, acc_size);
    case DPX_R_SQDEV_ONEPASS: return nan_run_kind<K_SQDEV1>(op, pl, src, dst, aux, stream, acc_size);
    default: return DPX_ERR_NOT_IMPLEMENTED;
    }
}

int nan_run(int op, RedPlan &pl, const dpx_array_view *src, const dpx_array_view *dst, const dpx_array_view *aux,
            hipStream_t stream)
{
    return nan_dispatch(op, pl, src, dst, aux, stream, nullptr);
}
int nan_acc_size(int op, const dpx_array_view *src, const dpx_array_view *dst)
{
    RedPlan unused{};
    int sz = 0;
    nan_dispatch(op, unused, src, dst, nullptr, nullptr, &sz);
    return sz;
}

// nanargmax / nanargmin: real floating types
int nanarg_run(bool is_max, RedPlan &pl, const dpx_array_view *src, const dpx_array_view *dst, hipStream_t stream)
{
    switch (src->dtype) {
    case DPX_HALF:
        return is_max ? arg_run<nanskip<half_t, true>, true>(pl, src, dst, stream)
                      : arg_run<nanskip<half_t, false>, false>(pl, src, dst, stream);
    case DPX_FLOAT:
        return is_max ? arg_run<nanskip<float, true>, true>(pl, src, dst, stream)
                      : arg_run<nanskip<float, false>, false>(pl, src, dst, stream);
    case DPX_DOUBLE:
        return is_max ? arg_run<nanskip<double, true>, true>(pl, src, dst, stream)
                      : arg_run<nanskip<double, false>, false>(pl, src, dst, stream);
    default: return DPX_ERR_NOT_IMPLEMENTED;
    }
}

} // namespace dpx
