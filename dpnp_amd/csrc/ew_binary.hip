// dpx_binary / dpx_binary_inplace kernels: py_binary_ufunc and py_binary_inplace_ufunc
// (libtensor/source/elementwise_functions/elementwise_functions.hpp:305-563,612-804).
// Compiled once per op group (-DDPX_GROUP=g -DDPX_NGROUPS=n): ops with id % n == g.
#include "ew_dispatch.hpp"

#ifndef DPX_GROUP
#define DPX_GROUP 0
#define DPX_NGROUPS 1
#endif
#define DPX_CAT2(a, b) a##b
#define DPX_CAT(a, b) DPX_CAT2(a, b)

namespace dpx {

template <class Op, bool IU> struct MixedCmpFn {
    DPX_D bool operator()(std::conditional_t<IU, int64_t, uint64_t> a,
                          std::conditional_t<IU, uint64_t, int64_t> b) const
    {
        if constexpr (IU) return Op::apply_iu(a, b);
        else return Op::apply_ui(a, b);
    }
};

// views = src1, src2, dst; returns -1 when `op` does not belong to this group
int DPX_CAT(binary_group_, DPX_GROUP)(int op, const dpx_array_view *const *views, hipStream_t stream,
                                       dpx_plan *plan_out)
{
    if (op % DPX_NGROUPS != DPX_GROUP) return -1;
    int rc = DPX_ERR_NOT_IMPLEMENTED;
    const int dt1 = views[0]->dtype, dt2 = views[1]->dtype;
    if (dt1 != dt2) {
        // mixed pairs: int64 <-> uint64 comparisons (greater.hpp:62-146) and arithmetic with the
        // conversion of one operand folded in
        for_binary_op(op, [&](auto otag) {
            using Op = typename decltype(otag)::type;
            if constexpr (std::is_same_v<Op, AddOp> || std::is_same_v<Op, SubOp> || std::is_same_v<Op, MulOp> ||
                          std::is_same_v<Op, DivOp>) {
                for_mixed_pair(dt1, dt2, [&](auto tt, auto at, auto bt) {
                    using T = typename decltype(tt)::type;
                    using A = typename decltype(at)::type;
                    using B = typename decltype(bt)::type;
                    rc = run_ew<MixedFn<Op, T, A, B>, T, A, B>({}, views, stream, plan_out);
                });
            }
            if constexpr (std::is_same_v<Op, CmpOp<0>> || std::is_same_v<Op, CmpOp<1>> ||
                          std::is_same_v<Op, CmpOp<2>> || std::is_same_v<Op, CmpOp<3>> ||
                          std::is_same_v<Op, CmpOp<4>> || std::is_same_v<Op, CmpOp<5>>) {
                if (dt1 == DPX_INT64 && dt2 == DPX_UINT64)
                    rc = run_ew<MixedCmpFn<Op, true>, bool_t, int64_t, uint64_t>({}, views, stream, plan_out);
                else if (dt1 == DPX_UINT64 && dt2 == DPX_INT64)
                    rc = run_ew<MixedCmpFn<Op, false>, bool_t, uint64_t, int64_t>({}, views, stream, plan_out);
            }
        });
    }
    else {
        for_binary_op(op, [&](auto otag) {
            using Op = typename decltype(otag)::type;
            for_dtype(dt1, [&](auto ttag) {
                using T = typename decltype(ttag)::type;
                if constexpr (Op::template ok<T>) {
                    using O = typename Op::template out<T>;
                    rc = run_ew<BinaryFn<Op, T>, O, T, T>(BinaryFn<Op, T>{}, views, stream, plan_out);
                }
            });
        });
    }
    if (rc == DPX_ERR_NOT_IMPLEMENTED) return fail(rc, "no kernel for this binary op and dtype pair");
    return rc;
}

} // namespace dpx
