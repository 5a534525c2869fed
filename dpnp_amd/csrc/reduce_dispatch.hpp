// Host side of the reductions: plan (type independent) + templated launch sequence.
#pragma once
#include <algorithm>
#include "host.hpp"
#include "reduce.hpp"

namespace dpx {

struct RedPlan {
    int path; // dpx_path
    RedIndex ix;
    RedLaunch L;
    int64_t src_off, dst_off, aux_off; // element displacements from collapsing
    int block;                          // threads per block of the first pass
    int64_t grid;
    // fold pass (splits > 1)
    RedIndex fix;
    RedLaunch fL;
    int fblock;
    int64_t fgrid;
    bool fold_cols;
    int64_t scratch_elems; // m * splits
};

// Validation shared by reductions and searches, in the order of py_reduction_over_axis
// (libtensor/source/reductions/reduction_over_axis.hpp:188-238).
int red_validate(const dpx_array_view *src, int trailing, const dpx_array_view *dst,
                 const dpx_array_view *aux, bool empty_ok);
// keep_order: reduced dims may only be merged, not reordered (searches).
// in_size / acc_size: bytes of the input element and of a partial.
void red_make_plan(RedPlan &pl, const dpx_array_view *src, int trailing, const dpx_array_view *dst,
                   const dpx_array_view *aux, bool keep_order, int in_size, bool arg);
void red_finish_fold(RedPlan &pl, int acc_size, bool arg);
void red_export_plan(const RedPlan &pl, dpx_plan *out, int acc_size);

template <int KIND, class In, class Out>
inline int red_run(RedPlan &pl, const dpx_array_view *src, const dpx_array_view *dst,
                   const dpx_array_view *aux, hipStream_t stream)
{
    using P = RedPolicy<KIND, In, Out>;
    using Acc = typename P::Acc;
    // the fold pass of a squared-deviation sum is a plain sum of partials
    using F = RedPolicy<(KIND == K_SUMSQDEV ? K_SUM : KIND), Acc, Out, true>;
    const In *sp = (const In *)src->data + pl.src_off;
    Out *dp = (Out *)dst->data + pl.dst_off;
    const Out *ap = aux ? (const Out *)aux->data + pl.aux_off : nullptr;
    if (pl.path == DPX_PATH_NOOP) return DPX_OK;
    if (pl.L.n == 0) {
        hipLaunchKernelGGL((red_fill_kernel<P>), dim3((unsigned)((pl.L.m + 255) / 256)), dim3(256), 0, stream,
                           pl.ix, pl.L.m, dp);
        hipError_t e = hipGetLastError();
        return e == hipSuccess ? DPX_OK : fail_hip(e, "reduction identity fill");
    }
    Acc *partial = nullptr;
    red_finish_fold(pl, (int)sizeof(Acc), false);
    if (pl.L.splits > 1) {
        partial = (Acc *)scratch_get(stream, (size_t)pl.scratch_elems * sizeof(Acc));
        if (!partial) return fail(DPX_ERR_HIP, "cannot allocate reduction scratch");
    }
    const bool cols = pl.path == DPX_PATH_RED_COLS || pl.path == DPX_PATH_RED_COLS_SPLIT;
    if (cols)
        hipLaunchKernelGGL((red_cols_kernel<P>), dim3((unsigned)pl.grid), dim3(256), 0, stream, pl.ix, pl.L, sp,
                           dp, partial, ap);
    else if (pl.path == DPX_PATH_RED_GENERIC)
        hipLaunchKernelGGL((red_rows_kernel<P, false>), dim3((unsigned)pl.grid), dim3(pl.block), 0, stream,
                           pl.ix, pl.L, sp, dp, partial, ap);
    else
        hipLaunchKernelGGL((red_rows_kernel<P, true>), dim3((unsigned)pl.grid), dim3(pl.block), 0, stream, pl.ix,
                           pl.L, sp, dp, partial, ap);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail_hip(e, "reduction launch");
    if (pl.L.splits > 1) {
        if (pl.fold_cols)
            hipLaunchKernelGGL((red_cols_kernel<F>), dim3((unsigned)pl.fgrid), dim3(256), 0, stream, pl.fix,
                               pl.fL, (const Acc *)partial, dp, (Acc *)nullptr, (const Out *)nullptr);
        else
            hipLaunchKernelGGL((red_rows_kernel<F, true>), dim3((unsigned)pl.fgrid), dim3(pl.fblock), 0, stream,
                               pl.fix, pl.fL, (const Acc *)partial, dp, (Acc *)nullptr, (const Out *)nullptr);
        e = hipGetLastError();
        if (e != hipSuccess) return fail_hip(e, "reduction fold launch");
    }
    return DPX_OK;
}

template <class T, bool IS_MAX>
inline int arg_run(RedPlan &pl, const dpx_array_view *src, const dpx_array_view *dst, hipStream_t stream)
{
    const T *sp = (const T *)src->data + pl.src_off;
    int64_t *dp = (int64_t *)dst->data + pl.dst_off;
    if (pl.path == DPX_PATH_NOOP) return DPX_OK;
    T *pval = nullptr;
    int64_t *pidx = nullptr;
    red_finish_fold(pl, (int)sizeof(T), true);
    if (pl.L.splits > 1) {
        // [indices | values]
        char *s = (char *)scratch_get(stream, (size_t)pl.scratch_elems * (sizeof(int64_t) + sizeof(T)));
        if (!s) return fail(DPX_ERR_HIP, "cannot allocate reduction scratch");
        pidx = (int64_t *)s;
        pval = (T *)(s + (size_t)pl.scratch_elems * sizeof(int64_t));
    }
    const bool cols = pl.path == DPX_PATH_RED_COLS || pl.path == DPX_PATH_RED_COLS_SPLIT;
    if (cols)
        hipLaunchKernelGGL((arg_cols_kernel<T, IS_MAX, true>), dim3((unsigned)pl.grid), dim3(256), 0, stream,
                           pl.ix, pl.L, sp, (const int64_t *)nullptr, dp, pval, pidx);
    else if (pl.path == DPX_PATH_RED_GENERIC)
        hipLaunchKernelGGL((arg_rows_kernel<T, IS_MAX, false, true>), dim3((unsigned)pl.grid), dim3(pl.block), 0,
                           stream, pl.ix, pl.L, sp, (const int64_t *)nullptr, dp, pval, pidx);
    else
        hipLaunchKernelGGL((arg_rows_kernel<T, IS_MAX, true, true>), dim3((unsigned)pl.grid), dim3(pl.block), 0,
                           stream, pl.ix, pl.L, sp, (const int64_t *)nullptr, dp, pval, pidx);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail_hip(e, "search launch");
    if (pl.L.splits > 1) {
        if (pl.fold_cols)
            hipLaunchKernelGGL((arg_cols_kernel<T, IS_MAX, false>), dim3((unsigned)pl.fgrid), dim3(256), 0, stream,
                               pl.fix, pl.fL, (const T *)pval, (const int64_t *)pidx, dp, (T *)nullptr,
                               (int64_t *)nullptr);
        else
            hipLaunchKernelGGL((arg_rows_kernel<T, IS_MAX, true, false>), dim3((unsigned)pl.fgrid),
                               dim3(pl.fblock), 0, stream, pl.fix, pl.fL, (const T *)pval, (const int64_t *)pidx,
                               dp, (T *)nullptr, (int64_t *)nullptr);
        e = hipGetLastError();
        if (e != hipSuccess) return fail_hip(e, "search fold launch");
    }
    return DPX_OK;
}

} // namespace dpx
