// tri._max_over_axis / _min_over_axis (libtensor/source/reductions/max.cpp:88-157, min.cpp):
// same-dtype pairs for all 14 types, NaN propagates.
#include "reduce_dispatch.hpp"

namespace dpx {

int minmax_run(bool is_max, RedPlan &pl, const dpx_array_view *src, const dpx_array_view *dst,
               hipStream_t stream)
{
    int rc = DPX_ERR_NOT_IMPLEMENTED;
    for_dtype(src->dtype, [&](auto tt) {
        using T = typename decltype(tt)::type;
        rc = is_max ? red_run<K_MAX, T, T>(pl, src, dst, nullptr, stream)
                    : red_run<K_MIN, T, T>(pl, src, dst, nullptr, stream);
    });
    return rc;
}

// tri._logsumexp_over_axis / _hypot_over_axis (libtensor/source/reductions/logsumexp.cpp,
// reduce_hypot.cpp): real floating types, same-dtype (half accumulates in float)
int fpred_run(bool is_lse, RedPlan &pl, const dpx_array_view *src, const dpx_array_view *dst, hipStream_t stream)
{
    const int i = src->dtype, o = dst->dtype;
#define DPX_FPRED(I, O)                                                                       \
    if (i == id_of_v<I> && o == id_of_v<O>)                                                   \
        return is_lse ? red_run<K_LOGSUMEXP, I, O>(pl, src, dst, nullptr, stream)              \
                      : red_run<K_HYPOT, I, O>(pl, src, dst, nullptr, stream);
    DPX_FPRED(half_t, half_t) DPX_FPRED(float, float) DPX_FPRED(double, double) DPX_FPRED(half_t, float)
    DPX_FPRED(float, double)
#undef DPX_FPRED
    return DPX_ERR_NOT_IMPLEMENTED;
}
bool fpred_pair_supported(int i, int o)
{
    return (i == DPX_HALF && (o == DPX_HALF || o == DPX_FLOAT)) || (i == DPX_FLOAT && (o == DPX_FLOAT || o == DPX_DOUBLE)) ||
           (i == DPX_DOUBLE && o == DPX_DOUBLE);
}

} // namespace dpx
