// Truth-value reductions over any input type in one pass: all, any (py_boolean_reduction,
// libtensor/source/reductions/reduction_over_axis.hpp:1057-1303, tri._all / tri._any) and
// count_nonzero (dpnp/tensor/_reduction.py:472-512, which casts to bool and sums).  An element
// is true when it is not zero (NaN is true, complex: either part).
#include "reduce_dispatch.hpp"

namespace dpx {

bool truth_pair_supported(int op, int in_dt, int out_dt)
{
    if (in_dt < 0 || in_dt >= DPX_NUM_DTYPES) return false;
    return (op == DPX_R_COUNT_NONZERO) ? out_dt == DPX_INT64 : out_dt == DPX_BOOL;
}

int truth_run(int op, RedPlan &pl, const dpx_array_view *src, const dpx_array_view *dst, hipStream_t stream)
{
    int rc = DPX_ERR_NOT_IMPLEMENTED;
    for_dtype(src->dtype, [&](auto tt) {
        using T = typename decltype(tt)::type;
        if (op == DPX_R_ANY) rc = red_run<K_ANY, T, bool_t>(pl, src, dst, nullptr, stream);
        else if (op == DPX_R_ALL) rc = red_run<K_ALL, T, bool_t>(pl, src, dst, nullptr, stream);
        else rc = red_run<K_COUNT_NONZERO, T, int64_t>(pl, src, dst, nullptr, stream);
    });
    return rc;
}

} // namespace dpx
