// dpx_unary: py_unary_ufunc (libtensor/source/elementwise_functions/elementwise_functions.hpp:77-251).
// Compiled once per op group (-DDPX_GROUP=g -DDPX_NGROUPS=n): ops with id % n == g.
#include "ew_dispatch.hpp"

#ifndef DPX_GROUP
#define DPX_GROUP 0
#define DPX_NGROUPS 1
#endif
#define DPX_CAT2(a, b) a##b
#define DPX_CAT(a, b) DPX_CAT2(a, b)

namespace dpx {

// returns -1 when `op` does not belong to this group
int DPX_CAT(unary_group_, DPX_GROUP)(int op, const dpx_array_view *src, const dpx_array_view *dst,
                                      hipStream_t stream, dpx_plan *plan_out)
{
    if (op % DPX_NGROUPS != DPX_GROUP) return -1;
    int rc = DPX_ERR_NOT_IMPLEMENTED;
    const dpx_array_view *views[2] = {src, dst};
    for_unary_op(op, [&](auto otag) {
        using Op = typename decltype(otag)::type;
        for_dtype(src->dtype, [&](auto ttag) {
            using T = typename decltype(ttag)::type;
            if constexpr (Op::template ok<T>) {
                using O = typename Op::template out<T>;
                rc = run_ew<UnaryFn<Op, T>, O, T>(UnaryFn<Op, T>{}, views, stream, plan_out);
            }
        });
    });
    if (rc == DPX_ERR_NOT_IMPLEMENTED) return fail(rc, "no kernel for this unary op and dtype");
    return rc;
}

} // namespace dpx
