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

} // namespace dpx
