// Host side of the reductions: plan (type independent) + templated launch sequence.
#pragma once
#include <algorithm>
#include <string>
#include "host.hpp"
#include "reduce.hpp"

namespace dpx {


struct RedPlan {
    int path; // dpx_path
    RedIndex ix;
    RedLaunch L;
    int64_t src_off, dst_off, aux_off; // element displacements from collapsing
    int block;                          // threads per block
    int64_t grid;
    int64_t scratch_elems; // partials: m * splits
    // scratch block brought by the caller instead of the stream's pool block (the entry point that
    // allocates nothing): [counters | partials], counters zero; nullptr: take the pool's
    char *ext_scratch;
    size_t ext_scratch_bytes;
};

// Scratch for a split launch: `need` bytes laid out [counters | partials].  DPX_OK and *out set, or
// the failure recorded.
inline int red_scratch(const RedPlan &pl, hipStream_t stream, size_t need, char **out)
{
    if (pl.ext_scratch) {
        if (need > pl.ext_scratch_bytes)
            return fail(DPX_ERR_BAD_ARGUMENT,
                        "this reduction needs " + std::to_string(need) + " bytes of scratch for its partial results; "
                        "the static scratch of the entry point that allocates nothing holds " +
                        std::to_string(pl.ext_scratch_bytes) + ": use dpx_reduce");
        // the size is known to fit (from the typed kernel's own slot size): only now is anything launched.
        // The ticket counters must be zero when the kernel starts, whatever an earlier call left
        // (a fill kernel: legal under stream capture)
        const hipError_t e = zero_fill_async(pl.ext_scratch, RED_COUNTER_BYTES / 16, stream);
        if (e != hipSuccess) return fail_hip(e, "clearing the static scratch counters");
        *out = pl.ext_scratch;
        return DPX_OK;
    }
    *out = (char *)scratch_get(stream, need, RED_COUNTER_BYTES);
    return *out ? DPX_OK : fail(DPX_ERR_HIP, "cannot allocate reduction scratch");
}
// after a launch that used scratch: an error leaves the ticket counters in doubt
inline int red_launch_status(const RedPlan &pl, hipStream_t stream, const char *what)
{
    const hipError_t e = hipGetLastError();
    if (e == hipSuccess) return DPX_OK;
    if (pl.L.splits > 1 && !pl.ext_scratch) scratch_mark_dirty(stream);
    return fail_hip(e, what);
}

// Validation shared by reductions and searches, in the order of py_reduction_over_axis
// (libtensor/source/reductions/reduction_over_axis.hpp:188-238).
// aux_dt: the dtype aux must have (-1: the destination's)
int red_validate(const dpx_array_view *src, int trailing, const dpx_array_view *dst,
                 const dpx_array_view *aux, bool empty_ok, int aux_dt = -1);
// keep_order: reduced dims may only be merged, not reordered (searches).
// rows_only: the kernels for short rows (staged in LDS, or read as one flat stream) are not to be chosen: such
// matrices then take the plain row or column kernel (the caller checks the path for the other layouts)
void red_make_plan(RedPlan &pl, const dpx_array_view *src, int trailing, const dpx_array_view *dst,
                   const dpx_array_view *aux, bool keep_order, int in_size, bool arg, bool rows_only = false);
void red_export_plan(const RedPlan &pl, dpx_plan *out, int acc_size);

inline bool red_is_cols(const RedPlan &pl)
{
    return pl.path == DPX_PATH_RED_COLS || pl.path == DPX_PATH_RED_COLS_SPLIT;
}

template <int KIND, class In, class Out>
inline int red_run(RedPlan &pl, const dpx_array_view *src, const dpx_array_view *dst,
                   const dpx_array_view *aux, hipStream_t stream)
{
    using P = RedPolicy<KIND, In, Out>;
    using Acc = typename P::Acc;
    const In *sp = (const In *)src->data + pl.src_off;
    Out *dp = (Out *)dst->data + pl.dst_off;
    const typename P::Aux *ap = aux ? (const typename P::Aux *)aux->data + pl.aux_off : nullptr;
    if (pl.path == DPX_PATH_NOOP) return DPX_OK;
    if (pl.L.n == 0) {
        hipLaunchKernelGGL((red_fill_kernel<P>), dim3((unsigned)((pl.L.m + 255) / 256)), dim3(256), 0, stream,
                           pl.ix, pl.L.m, dp);
        hipError_t e = hipGetLastError();
        return e == hipSuccess ? DPX_OK : fail_hip(e, "reduction identity fill");
    }
    Slot<Acc> *partial = nullptr;
    unsigned *counters = nullptr;
    if (pl.L.splits > 1) {
        char *s = nullptr;
        if (int rc = red_scratch(pl, stream, RED_COUNTER_BYTES + (size_t)pl.scratch_elems * sizeof(Slot<Acc>), &s))
            return rc;
        counters = (unsigned *)s;
        partial = (Slot<Acc> *)(s + RED_COUNTER_BYTES);
    }
    if (red_is_cols(pl)) {
        constexpr int E = cols_cfg<In>::E;
        int block = pl.block; // LDS: one accumulator pack per thread, at most 64 KiB
        while ((size_t)block * E * sizeof(Acc) > 65536) block /= 2;
        if (block < (1 << pl.L.g_log2)) return fail(DPX_ERR_NOT_IMPLEMENTED, "column reduction: accumulator too wide");
        const size_t smem = (size_t)block * E * sizeof(Acc);
        if (pl.L.walk)
            hipLaunchKernelGGL((red_cols_kernel<P, true>), dim3((unsigned)pl.grid), dim3(block), smem, stream, pl.ix,
                               pl.L, sp, dp, partial, ap, counters);
        else
            hipLaunchKernelGGL((red_cols_kernel<P, false>), dim3((unsigned)pl.grid), dim3(block), smem, stream, pl.ix,
                               pl.L, sp, dp, partial, ap, counters);
    }
    else if (pl.path == DPX_PATH_RED_SHORT_ROWS) {
        const size_t smem = (size_t)pl.L.chunk * srow_pitch<In>((int)pl.L.n) * sizeof(In); // at most 32 KiB
        hipLaunchKernelGGL((red_short_rows_kernel<P>), dim3((unsigned)pl.grid), dim3(256), smem, stream, pl.ix, pl.L,
                           sp, dp, ap);
    }
    else if (pl.path == DPX_PATH_RED_FLAT) {
        const size_t smem = (size_t)pl.block * cols_cfg<In>::E * sizeof(Acc); // at most 32 KiB
        hipLaunchKernelGGL((red_flat_kernel<P>), dim3((unsigned)pl.grid), dim3(pl.block), smem, stream, pl.ix, pl.L,
                           sp, dp, partial, ap, counters);
    }
    else if (pl.path == DPX_PATH_RED_GENERIC)
        hipLaunchKernelGGL((red_rows_kernel<P, false>), dim3((unsigned)pl.grid), dim3(pl.block), 0, stream,
                           pl.L, sp, dp, partial, ap, counters, pl.ix);
    else
        hipLaunchKernelGGL((red_rows_kernel<P, true>), dim3((unsigned)pl.grid), dim3(pl.block), 0, stream, pl.L,
                           sp, dp, partial, ap, counters, pl.ix);
    return red_launch_status(pl, stream, "reduction launch");
}

template <class T, bool IS_MAX>
inline int arg_run(RedPlan &pl, const dpx_array_view *src, const dpx_array_view *dst, hipStream_t stream)
{
    const T *sp = (const T *)src->data + pl.src_off;
    int64_t *dp = (int64_t *)dst->data + pl.dst_off;
    if (pl.path == DPX_PATH_NOOP) return DPX_OK;
    Slot<T> *pval = nullptr;
    Slot<int64_t> *pidx = nullptr;
    unsigned *counters = nullptr;
    if (pl.L.splits > 1) {
        // [counters | positions | values]
        char *s = nullptr;
        if (int rc = red_scratch(pl, stream,
                                 RED_COUNTER_BYTES + (size_t)pl.scratch_elems * (sizeof(Slot<int64_t>) + sizeof(Slot<T>)), &s))
            return rc;
        counters = (unsigned *)s;
        pidx = (Slot<int64_t> *)(s + RED_COUNTER_BYTES);
        pval = (Slot<T> *)(s + RED_COUNTER_BYTES + (size_t)pl.scratch_elems * sizeof(Slot<int64_t>));
    }
    if (pl.path == DPX_PATH_RED_SHORT_ROWS) {
        const size_t smem = (size_t)pl.L.chunk * srow_pitch<T>((int)pl.L.n) * sizeof(T);
        hipLaunchKernelGGL((arg_short_rows_kernel<T, IS_MAX>), dim3((unsigned)pl.grid), dim3(256), smem, stream, pl.ix,
                           pl.L, sp, dp);
    }
    else if (pl.path == DPX_PATH_RED_FLAT) {
        // (row, value) pairs of every thread: at most 256 x 16 x 9 bytes
        const size_t smem = (size_t)pl.block * (16 / sizeof(T)) * (sizeof(int64_t) + sizeof(value_of_t<T>));
        hipLaunchKernelGGL((arg_flat_kernel<T, IS_MAX>), dim3((unsigned)pl.grid), dim3(pl.block), smem, stream, pl.ix,
                           pl.L, sp, dp, pval, pidx, counters);
    }
    else if (red_is_cols(pl)) {
        const size_t smem = (size_t)pl.block * (16 / sizeof(T)) * (sizeof(int64_t) + sizeof(value_of_t<T>));
        hipLaunchKernelGGL((arg_cols_kernel<T, IS_MAX>), dim3((unsigned)pl.grid), dim3(pl.block), smem, stream, pl.ix,
                           pl.L, sp, dp, pval, pidx, counters);
    }
    else if (pl.path == DPX_PATH_RED_GENERIC)
        hipLaunchKernelGGL((arg_rows_kernel<T, IS_MAX, false>), dim3((unsigned)pl.grid), dim3(pl.block), 0, stream,
                           pl.L, sp, dp, pval, pidx, counters, pl.ix);
    else
        hipLaunchKernelGGL((arg_rows_kernel<T, IS_MAX, true>), dim3((unsigned)pl.grid), dim3(pl.block), 0, stream,
                           pl.L, sp, dp, pval, pidx, counters, pl.ix);
    return red_launch_status(pl, stream, "search launch");
}

} // namespace dpx
