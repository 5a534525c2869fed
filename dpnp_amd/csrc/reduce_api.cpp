// extern "C" reduction entry points.
#include <mutex>
#include "reduce_dispatch.hpp"

// Scratch of dpx_reduce_noalloc: device memory that exists from the moment the library's code
// object is loaded on a GPU, so the entry point never allocates.  Each GPU holds its own copy
// until the process ends.  In host code the name below is only a handle for
// hipGetSymbolAddress; kernels and fills get the per-device address it returns.
static __device__ __align__(256) unsigned char scratch[DPX_NOALLOC_SCRATCH_BYTES];

namespace dpx {
namespace {
constexpr int NOALLOC_MAX_DEVICES = 64;
std::mutex g_noalloc_mu;
char *g_noalloc_ptr[NOALLOC_MAX_DEVICES]; // address of `scratch` on each device, looked up once
} // namespace

// Address of the static scratch on the current device (first call on a device: one symbol lookup).
static int noalloc_scratch(char **out)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail_hip(e, "hipGetDevice");
    if (dev < 0 || dev >= NOALLOC_MAX_DEVICES) return fail(DPX_ERR_BAD_ARGUMENT, "device index out of range");
    std::lock_guard<std::mutex> lk(g_noalloc_mu);
    if (!g_noalloc_ptr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) return fail_hip(e, "hipGetSymbolAddress(static reduction scratch)");
        g_noalloc_ptr[dev] = (char *)p;
    }
    *out = g_noalloc_ptr[dev];
    return DPX_OK;
}

bool sum_pair_supported(int, int);
bool prod_pair_supported(int, int);
bool sqdev_pair_supported(int, int);
int sum_run(RedPlan &, const dpx_array_view *, const dpx_array_view *, hipStream_t);
int prod_run(RedPlan &, const dpx_array_view *, const dpx_array_view *, hipStream_t);
int sqdev_run(RedPlan &, const dpx_array_view *, const dpx_array_view *, const dpx_array_view *, hipStream_t);
int sum_acc_size(int, int);
int sqdev_acc_size(int, int);
int prod_acc_size(int, int);
int minmax_run(bool, RedPlan &, const dpx_array_view *, const dpx_array_view *, hipStream_t);
int arg_run_any(bool, RedPlan &, const dpx_array_view *, const dpx_array_view *, hipStream_t);
int fpred_run(bool, RedPlan &, const dpx_array_view *, const dpx_array_view *, hipStream_t);
bool fpred_pair_supported(int, int);
bool nan_pair_supported(int, int, int);
int nan_run(int, RedPlan &, const dpx_array_view *, const dpx_array_view *, const dpx_array_view *, hipStream_t);
int nan_acc_size(int, const dpx_array_view *, const dpx_array_view *);
int nanarg_run(bool, RedPlan &, const dpx_array_view *, const dpx_array_view *, hipStream_t);

bool truth_pair_supported(int, int, int);
int truth_run(int, RedPlan &, const dpx_array_view *, const dpx_array_view *, hipStream_t);
static bool is_truth_op(int op) { return op == DPX_R_ANY || op == DPX_R_ALL || op == DPX_R_COUNT_NONZERO; }
static bool is_nan_op(int op)
{
    // (the one-pass squared deviations are typed in the same file)
    return (op >= DPX_R_NANSUM && op <= DPX_R_NANSUMSQDEV) || op == DPX_R_NANMEAN || op == DPX_R_NANVAR ||
           op == DPX_R_SQDEV_ONEPASS;
}
static bool takes_aux(int op) { return op == DPX_R_SUMSQDEV || op == DPX_R_NANSUMSQDEV || op == DPX_R_NANVAR; }

static bool reduce_supported(int op, int s, int d)
{
    if (s < 0 || s >= DPX_NUM_DTYPES || d < 0 || d >= DPX_NUM_DTYPES) return false;
    switch (op) {
    case DPX_R_SUM: return sum_pair_supported(s, d);
    case DPX_R_PROD: return prod_pair_supported(s, d);
    case DPX_R_MAX:
    case DPX_R_MIN: return s == d;
    case DPX_R_SUMSQDEV: return sqdev_pair_supported(s, d);
    case DPX_R_LOGSUMEXP:
    case DPX_R_HYPOT: return fpred_pair_supported(s, d);
    default:
        if (is_truth_op(op)) return truth_pair_supported(op, s, d);
        return is_nan_op(op) && nan_pair_supported(op, s, d);
    }
}

static int reduce_call(int op, const dpx_array_view *src, int trailing, const dpx_array_view *dst,
                       const dpx_array_view *aux, void *stream, dpx_plan *plan_out, double param = 0.0,
                       bool noalloc = false)
{
    if (op < 0 || op >= DPX_R_NUM_OPS) return fail(DPX_ERR_BAD_ARGUMENT, "unknown reduction op id");
    if (!view_ok(src) || !view_ok(dst)) return fail(DPX_ERR_BAD_ARGUMENT, "malformed array descriptor");
    if (!plan_out && takes_aux(op) != (aux != nullptr))
        return fail(DPX_ERR_BAD_ARGUMENT, "aux must be given for the squared-deviation ops and only for them");
    if (!reduce_supported(op, src->dtype, dst->dtype))
        return fail(DPX_ERR_NOT_IMPLEMENTED, "Datatypes are not supported");
    const bool empty_ok = op != DPX_R_MAX && op != DPX_R_MIN && op != DPX_R_NANMAX && op != DPX_R_NANMIN;
    // deviations of complex input from a complex mean, squared magnitudes summed into a real result
    const int aux_dt = (op == DPX_R_SUMSQDEV && (src->dtype == DPX_CFLOAT || src->dtype == DPX_CDOUBLE))
                           ? (dst->dtype == DPX_FLOAT ? DPX_CFLOAT : DPX_CDOUBLE)
                           : -1;
    if (int rc = red_validate(src, trailing, dst, aux, empty_ok, aux_dt)) return rc;
    RedPlan pl;
    red_make_plan(pl, src, trailing, dst, aux, false, itemsize_of(src->dtype), false, op == DPX_R_SQDEV_ONEPASS);
    // (one-pass squared deviations: every layout has a kernel; the plan above keeps away from the flat stream and
    // the staged short rows, whose lanes do not know the reference the means are kept relative to)
    // bytes of one partial result (the accumulator type of the typed kernel)
    auto acc_bytes = [&]() {
        int acc = itemsize_of(dst->dtype);
        if (op == DPX_R_SUM) acc = sum_acc_size(src->dtype, dst->dtype);
        if (op == DPX_R_SUMSQDEV) acc = sqdev_acc_size(src->dtype, dst->dtype);
        if (op == DPX_R_PROD) acc = prod_acc_size(src->dtype, dst->dtype);
        if ((op == DPX_R_MAX || op == DPX_R_MIN) && dst->dtype == DPX_BOOL) acc = 4;
        if ((op == DPX_R_LOGSUMEXP || op == DPX_R_HYPOT) && dst->dtype == DPX_HALF) acc = 4;
        if (op == DPX_R_LOGSUMEXP) acc *= 2; // (largest element, sum of exponentials relative to it)
        if (is_nan_op(op)) acc = nan_acc_size(op, src, dst);
        if (is_truth_op(op)) acc = op == DPX_R_COUNT_NONZERO ? 8 : 4;
        return acc;
    };
    if (plan_out) {
        red_export_plan(pl, plan_out, acc_bytes());
        return DPX_OK;
    }
    hipStream_t s = (hipStream_t)stream;
    pl.L.param = param;
    if (noalloc && pl.L.splits > 1) {
        const size_t need = RED_COUNTER_BYTES + (size_t)pl.scratch_elems * (size_t)((acc_bytes() + 3) / 4 * 4);
        if (need > DPX_NOALLOC_SCRATCH_BYTES)
            return fail(DPX_ERR_BAD_ARGUMENT,
                        "dpx_reduce_noalloc: the partial results of this reduction need " + std::to_string(need) +
                            " bytes of scratch, the static scratch holds " +
                            std::to_string((size_t)DPX_NOALLOC_SCRATCH_BYTES) + "; use dpx_reduce");
        // the static block instead of the pool's (red_scratch checks the typed kernel's own slot size against it
        // once more and clears the ticket counters, in that order)
        if (int rc = noalloc_scratch(&pl.ext_scratch)) return rc;
        pl.ext_scratch_bytes = DPX_NOALLOC_SCRATCH_BYTES;
    }
    if (is_nan_op(op)) return nan_run(op, pl, src, dst, aux, s);
    if (is_truth_op(op)) return truth_run(op, pl, src, dst, s);
    switch (op) {
    case DPX_R_SUM: return sum_run(pl, src, dst, s);
    case DPX_R_PROD: return prod_run(pl, src, dst, s);
    case DPX_R_MAX: return minmax_run(true, pl, src, dst, s);
    case DPX_R_MIN: return minmax_run(false, pl, src, dst, s);
    case DPX_R_LOGSUMEXP: return fpred_run(true, pl, src, dst, s);
    case DPX_R_HYPOT: return fpred_run(false, pl, src, dst, s);
    default: return sqdev_run(pl, src, dst, aux, s);
    }
}

static bool search_supported(int op, int s, int d)
{
    if (s < 0 || s >= DPX_NUM_DTYPES || d != DPX_INT64) return false;
    if (op == DPX_S_ARGMAX || op == DPX_S_ARGMIN) return true;
    if (op >= DPX_S_NANARGMAX && op <= DPX_S_NANARGMIN_MARKED) return s == DPX_HALF || s == DPX_FLOAT || s == DPX_DOUBLE;
    return false;
}

static int argreduce_call(int op, const dpx_array_view *src, int trailing, const dpx_array_view *dst,
                          void *stream, dpx_plan *plan_out)
{
    if (op < 0 || op > DPX_S_NANARGMIN_MARKED) return fail(DPX_ERR_BAD_ARGUMENT, "unknown search op id");
    if (!view_ok(src) || !view_ok(dst)) return fail(DPX_ERR_BAD_ARGUMENT, "malformed array descriptor");
    if (!search_supported(op, src->dtype, dst->dtype)) return fail(DPX_ERR_NOT_IMPLEMENTED, "Datatypes are not supported");
    if (int rc = red_validate(src, trailing, dst, nullptr, false)) return rc;
    RedPlan pl;
    red_make_plan(pl, src, trailing, dst, nullptr, true, itemsize_of(src->dtype), true);
    if (plan_out) {
        red_export_plan(pl, plan_out, itemsize_of(src->dtype) + 8);
        return DPX_OK;
    }
    if (op >= DPX_S_NANARGMAX) {
        pl.L.mark_fill = (op == DPX_S_NANARGMAX_MARKED || op == DPX_S_NANARGMIN_MARKED) ? 1 : 0;
        return nanarg_run(op == DPX_S_NANARGMAX || op == DPX_S_NANARGMAX_MARKED, pl, src, dst, (hipStream_t)stream);
    }
    return arg_run_any(op == DPX_S_ARGMAX, pl, src, dst, (hipStream_t)stream);
}

} // namespace dpx

using namespace dpx;
extern "C" {
int dpx_reduce_dtype_supported(int op, int src_dt, int dst_dt) { return reduce_supported(op, src_dt, dst_dt) ? 1 : 0; }
int dpx_search_dtype_supported(int op, int src_dt, int dst_dt) { return search_supported(op, src_dt, dst_dt) ? 1 : 0; }
int dpx_reduce(int op, const dpx_array_view *src, int trailing_dims_to_reduce, const dpx_array_view *dst,
               const dpx_array_view *aux, void *stream)
{
    return reduce_call(op, src, trailing_dims_to_reduce, dst, aux, stream, nullptr);
}
int dpx_reduce_noalloc(int op, const dpx_array_view *src, int trailing_dims_to_reduce, const dpx_array_view *dst,
                       const dpx_array_view *aux, void *stream)
{
    return reduce_call(op, src, trailing_dims_to_reduce, dst, aux, stream, nullptr, 0.0, true);
}
int dpx_reduce_plan(int op, const dpx_array_view *src, int trailing_dims_to_reduce, const dpx_array_view *dst,
                    dpx_plan *plan)
{
    if (!plan) return fail(DPX_ERR_BAD_ARGUMENT, "plan is null");
    // (the ops with a side input are planned without it: its layout follows the destination's)
    return reduce_call(op, src, trailing_dims_to_reduce, dst, nullptr, nullptr, plan);
}
int dpx_nan_variance(const dpx_array_view *src, int trailing_dims_to_reduce, const dpx_array_view *mean, double ddof,
                     const dpx_array_view *dst, void *stream)
{
    return reduce_call(DPX_R_NANVAR, src, trailing_dims_to_reduce, dst, mean, stream, nullptr, ddof);
}
int dpx_argreduce(int op, const dpx_array_view *src, int trailing_dims_to_reduce, const dpx_array_view *dst,
                  void *stream)
{
    return argreduce_call(op, src, trailing_dims_to_reduce, dst, stream, nullptr);
}
int dpx_argreduce_plan(int op, const dpx_array_view *src, int trailing_dims_to_reduce,
                       const dpx_array_view *dst, dpx_plan *plan)
{
    if (!plan) return fail(DPX_ERR_BAD_ARGUMENT, "plan is null");
    return argreduce_call(op, src, trailing_dims_to_reduce, dst, nullptr, plan);
}
}
