// dpx_unary: py_unary_ufunc (libtensor/source/elementwise_functions/elementwise_functions.hpp:77-251).
// Compiled once per op group (-DDPX_GROUP=g -DDPX_NGROUPS=n): ops with id % n == g.
#include "ew_dispatch.hpp"
#include "ew_half_table.hpp"

#ifndef DPX_GROUP
#define DPX_GROUP 0
#define DPX_NGROUPS 1
#endif
#define DPX_CAT2(a, b) a##b
#define DPX_CAT(a, b) DPX_CAT2(a, b)

namespace dpx {

// float16 functions that take more vector instructions per element than 4 bytes of traffic hide (measured at
// 2^27 elements: 30 to 72 % of the HBM rate with the plain kernel, 76 % through the table): large contiguous
// arrays go through the function's table of all 65536 results (ew_half_table.hpp)
template <class Op> struct op_half_table : std::false_type {};
#define DPX_HALF_TABLE(OP) \
    template <> struct op_half_table<OP> : std::true_type {};
DPX_HALF_TABLE(SinOp) DPX_HALF_TABLE(CosOp) DPX_HALF_TABLE(TanOp) DPX_HALF_TABLE(TanhOp) DPX_HALF_TABLE(Expm1Op)
DPX_HALF_TABLE(Log1pOp) DPX_HALF_TABLE(SinhOp) DPX_HALF_TABLE(AsinhOp) DPX_HALF_TABLE(AcoshOp) DPX_HALF_TABLE(AtanhOp)
DPX_HALF_TABLE(SincOp)
#undef DPX_HALF_TABLE

template <class Fn> __global__ __launch_bounds__(256) void half_table_build_kernel(Fn fn, uint16_t *table)
{
    const uint32_t i = blockIdx.x * 256 + threadIdx.x; // 256 blocks: every float16 bit pattern
    union {
        uint16_t u;
        half_t h;
    } a, r;
    a.u = (uint16_t)i;
    r.h = to_storage<half_t>(fn(to_value(a.h)));
    table[i] = r.u;
}
template <class Op> hipError_t half_table_build(uint16_t *table, hipStream_t stream)
{
    using Fn = UnaryFn<Op, half_t>;
    hipLaunchKernelGGL((half_table_build_kernel<Fn>), dim3(HALF_TABLE_ENTRIES / 256), dim3(256), 0, stream, Fn{}, table);
    return hipGetLastError();
}
// DPX_OK or an error when the call went through the table; -1 when it is one for the plain kernel
template <class Op> int half_table_call(int op, const dpx_array_view *const *views, hipStream_t stream)
{
    EwPlan pl;
    ew_make_plan(pl, 2, views);
    if (pl.path != DPX_PATH_EW_CONTIG || pl.flat2d || pl.n < HALF_TABLE_MIN || pl.strides[0][0] != 1) return -1;
    const uint16_t *table = half_table_for(op, stream, &half_table_build<Op>);
    if (!table) return -1;
    const hipError_t e = half_table_apply(table, (const char *)views[0]->data + pl.offsets[0] * 2,
                                          (char *)views[1]->data + pl.offsets[1] * 2, pl.n, stream);
    return e == hipSuccess ? DPX_OK : fail_hip(e, "float16 table kernel launch");
}

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
                if constexpr (std::is_same_v<T, half_t> && std::is_same_v<O, half_t> && op_half_table<Op>::value) {
                    if (!plan_out) {
                        const int t = half_table_call<Op>(op, views, stream);
                        if (t >= 0) {
                            rc = t;
                            return;
                        }
                    }
                }
                rc = run_ew<UnaryFn<Op, T>, O, T>(UnaryFn<Op, T>{}, views, stream, plan_out);
            }
        });
    });
    if (rc == DPX_ERR_NOT_IMPLEMENTED) return fail(rc, "no kernel for this unary op and dtype");
    return rc;
}

} // namespace dpx
