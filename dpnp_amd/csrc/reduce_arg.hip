// tri._argmax_over_axis / _argmin_over_axis (libtensor/source/reductions/argmax.cpp:77-160,
// argmin.cpp): any dtype -> int64 position.
#include "reduce_dispatch.hpp"

namespace dpx {

int arg_run_any(bool is_max, RedPlan &pl, const dpx_array_view *src, const dpx_array_view *dst,
                hipStream_t stream)
{
    int rc = DPX_ERR_NOT_IMPLEMENTED;
    for_dtype(src->dtype, [&](auto tt) {
        using T = typename decltype(tt)::type;
        rc = is_max ? arg_run<T, true>(pl, src, dst, stream) : arg_run<T, false>(pl, src, dst, stream);
    });
    return rc;
}

} // namespace dpx
