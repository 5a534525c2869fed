// extern "C" elementwise entry points: dtype tables, validation, group dispatch.
#include "ew_dispatch.hpp"

namespace dpx {
#define DPX_DECL_U(g) \
    int unary_group_##g(int, const dpx_array_view *, const dpx_array_view *, hipStream_t, dpx_plan *);
#define DPX_DECL_B(g) int binary_group_##g(int, const dpx_array_view *const *, hipStream_t, dpx_plan *);
DPX_DECL_U(0) DPX_DECL_U(1) DPX_DECL_U(2) DPX_DECL_U(3)
DPX_DECL_B(0) DPX_DECL_B(1) DPX_DECL_B(2) DPX_DECL_B(3) DPX_DECL_B(4) DPX_DECL_B(5)

static int unary_result_type(int op, int dt)
{
    int r = -1;
    for_unary_op(op, [&](auto otag) {
        using Op = typename decltype(otag)::type;
        for_dtype(dt, [&](auto ttag) {
            using T = typename decltype(ttag)::type;
            if constexpr (Op::template ok<T>) r = id_of_v<typename Op::template out<T>>;
        });
    });
    return r;
}
static bool is_compare(int op) { return op >= DPX_B_EQUAL && op <= DPX_B_GREATER_EQUAL; }
static int mixed_result_type(int op, int dt1, int dt2)
{
    int r = -1;
    if (dt1 != dt2 && is_mixed_arith(op))
        for_mixed_pair(dt1, dt2, [&](auto tt, auto, auto) { r = id_of_v<typename decltype(tt)::type>; });
    return r;
}
// with_fused: also the pairs whose conversion is folded into the kernel.  The exported type table
// leaves them out: the caller's promotion search must see the same table as the reference's.
static int binary_result_type(int op, int dt1, int dt2, bool with_fused = false)
{
    int r = -1;
    if (dt1 != dt2) {
        if (is_compare(op) && ((dt1 == DPX_INT64 && dt2 == DPX_UINT64) || (dt1 == DPX_UINT64 && dt2 == DPX_INT64)))
            r = DPX_BOOL;
        else if (with_fused)
            r = mixed_result_type(op, dt1, dt2);
        return r;
    }
    for_binary_op(op, [&](auto otag) {
        using Op = typename decltype(otag)::type;
        for_dtype(dt1, [&](auto ttag) {
            using T = typename decltype(ttag)::type;
            if constexpr (Op::template ok<T>) r = id_of_v<typename Op::template out<T>>;
        });
    });
    return r;
}

static int unary_call(int op, const dpx_array_view *src, const dpx_array_view *dst, void *stream,
                      dpx_plan *plan_out)
{
    if (!view_ok(src) || !view_ok(dst)) return fail(DPX_ERR_BAD_ARGUMENT, "malformed array descriptor");
    const int rt = unary_result_type(op, src->dtype);
    if (op < 0 || op >= DPX_U_NUM_OPS) return fail(DPX_ERR_BAD_ARGUMENT, "unknown unary op id");
    if (rt < 0 || rt != dst->dtype)
        return fail(DPX_ERR_BAD_DTYPE, "Destination array has unexpected elemental data type.");
    const dpx_array_view *views[2] = {src, dst};
    int64_t n = 0;
    if (int rc = ew_validate(2, views, n)) return rc;
    int rc = -1;
    hipStream_t s = (hipStream_t)stream;
    if ((rc = unary_group_0(op, src, dst, s, plan_out)) != -1) return rc;
    if ((rc = unary_group_1(op, src, dst, s, plan_out)) != -1) return rc;
    if ((rc = unary_group_2(op, src, dst, s, plan_out)) != -1) return rc;
    if ((rc = unary_group_3(op, src, dst, s, plan_out)) != -1) return rc;
    return fail(DPX_ERR_NOT_IMPLEMENTED, "unary op not built");
}

static int binary_call(int op, const dpx_array_view *a, const dpx_array_view *b, const dpx_array_view *dst,
                       void *stream, dpx_plan *plan_out)
{
    if (!view_ok(a) || !view_ok(b) || !view_ok(dst))
        return fail(DPX_ERR_BAD_ARGUMENT, "malformed array descriptor");
    if (op < 0 || op >= DPX_B_NUM_OPS) return fail(DPX_ERR_BAD_ARGUMENT, "unknown binary op id");
    const int rt = binary_result_type(op, a->dtype, b->dtype, true);
    if (rt < 0 || rt != dst->dtype)
        return fail(DPX_ERR_BAD_DTYPE, "Output array of type " + std::string(dtype_name(dst->dtype)) +
                                           " does not match the result type of the operation.");
    const dpx_array_view *views[3] = {a, b, dst};
    int64_t n = 0;
    if (int rc = ew_validate(3, views, n)) return rc;
    hipStream_t s = (hipStream_t)stream;
    int rc = -1;
    if ((rc = binary_group_0(op, views, s, plan_out)) != -1) return rc;
    if ((rc = binary_group_1(op, views, s, plan_out)) != -1) return rc;
    if ((rc = binary_group_2(op, views, s, plan_out)) != -1) return rc;
    if ((rc = binary_group_3(op, views, s, plan_out)) != -1) return rc;
    if ((rc = binary_group_4(op, views, s, plan_out)) != -1) return rc;
    if ((rc = binary_group_5(op, views, s, plan_out)) != -1) return rc;
    return fail(DPX_ERR_NOT_IMPLEMENTED, "binary op not built");
}

} // namespace dpx

using namespace dpx;

extern "C" {

int dpx_unary_result_type(int op, int dt) { return unary_result_type(op, dt); }
int dpx_binary_result_type(int op, int dt1, int dt2) { return binary_result_type(op, dt1, dt2); }
int dpx_binary_fused_cast_result_type(int op, int dt1, int dt2) { return mixed_result_type(op, dt1, dt2); }
int dpx_binary_inplace_supported(int op, int lhs_dt, int rhs_dt)
{
    // lhs op= rhs needs a kernel whose result type is lhs's type
    return binary_result_type(op, lhs_dt, rhs_dt) == lhs_dt ? 1 : 0;
}

int dpx_unary(int op, const dpx_array_view *src, const dpx_array_view *dst, void *stream)
{
    return unary_call(op, src, dst, stream, nullptr);
}
int dpx_unary_plan(int op, const dpx_array_view *src, const dpx_array_view *dst, dpx_plan *plan)
{
    if (!plan) return fail(DPX_ERR_BAD_ARGUMENT, "plan is null");
    return unary_call(op, src, dst, nullptr, plan);
}
int dpx_binary(int op, const dpx_array_view *src1, const dpx_array_view *src2, const dpx_array_view *dst,
               void *stream)
{
    return binary_call(op, src1, src2, dst, stream, nullptr);
}
int dpx_binary_plan(int op, const dpx_array_view *src1, const dpx_array_view *src2,
                    const dpx_array_view *dst, dpx_plan *plan)
{
    if (!plan) return fail(DPX_ERR_BAD_ARGUMENT, "plan is null");
    return binary_call(op, src1, src2, dst, nullptr, plan);
}
int dpx_binary_inplace(int op, const dpx_array_view *lhs, const dpx_array_view *rhs, void *stream)
{
    if (!view_ok(lhs) || !view_ok(rhs)) return fail(DPX_ERR_BAD_ARGUMENT, "malformed array descriptor");
    if (!dpx_binary_inplace_supported(op, lhs->dtype, rhs->dtype) &&
        mixed_result_type(op, lhs->dtype, rhs->dtype) != lhs->dtype)
        return fail(DPX_ERR_BAD_DTYPE, "Left-hand side array has unexpected elemental data type for the "
                                       "in-place operation.");
    return binary_call(op, lhs, rhs, lhs, stream, nullptr);
}

} // extern "C"
