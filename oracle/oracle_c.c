/*
 * C restatement of the reference's algorithms for the three headline kernels, used as
 * the CPU baseline of bench.py and cross-checked against oracle.py in tests/.
 * TEST INFRASTRUCTURE ONLY: nothing under dpnp_amd/ links or loads this file.
 *
 * Paths are relative to the reference tree, libtensor = dpnp/tensor/libtensor.
 *
 *  - oc_add_f32: BinaryContigFunctor with AddFunctor
 *    (libtensor/include/kernels/elementwise_functions/common.hpp:398-521, add.hpp:63-114):
 *    out[i] = a[i] + b[i].
 *  - oc_sum_f32: reduction_axis1_over_group_temps_contig_impl with one output
 *    (libtensor/include/kernels/reductions.hpp:1397-1624): work-groups of wg work-items,
 *    work-item `lid` of group `g` folds elements g*rpw*wg + m*wg + lid (m < rpw, rpw = 8),
 *    the group combines its work-items' values, one partial per group goes to a
 *    temporary; levels repeat while more than 8*max_wg partials remain; a last group of
 *    max_wg work-items finishes (reductions.hpp:451-516,1496-1623).  n < wg: one
 *    work-item walks the whole run (SequentialReduction, :98-152).
 *  - oc_argmax_f32 / oc_argmin_f32: search_axis1_over_group_temps_contig_impl
 *    (reductions.hpp:2786-3041) with the per-work-item update rule of
 *    CustomSearchReduction (:2187-2363): equal values keep the smaller index, a NaN always
 *    replaces the running value; inside a group only work-items whose value equals the
 *    group's value (or is NaN) offer their index and the smallest offered index wins.
 *    As in the reference, with several NaNs the result depends on the partition.
 *
 * Work-groups run as OpenMP loop iterations; the work-items of a group are a vector loop.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define WG 256
#define RPW 8
#define MAX_WG 2048

int oc_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

__attribute__((target_clones("avx2", "default")))
void oc_add_f32(const float *a, const float *b, float *out, int64_t n)
{
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) out[i] = a[i] + b[i];
}

/* one level: groups of `wg` work-items, `rpw` elements per work-item */
__attribute__((target_clones("avx2", "default")))
static void sum_level(const float *x, int64_t n, int wg, int64_t rpw, float *partials, int64_t ngroups)
{
#pragma omp parallel for schedule(static)
    for (int64_t g = 0; g < ngroups; ++g) {
        float acc[MAX_WG];
        for (int l = 0; l < wg; ++l) acc[l] = 0.0f;
        const int64_t base = g * rpw * wg;
        for (int64_t m = 0; m < rpw; ++m) {
            const int64_t off = base + m * wg;
            if (off >= n) break;
            const int lim = (n - off < wg) ? (int)(n - off) : wg;
            for (int l = 0; l < lim; ++l) acc[l] += x[off + l];
        }
        for (int half = wg / 2; half > 0; half /= 2) /* group combine: halving tree */
            for (int l = 0; l < half; ++l) acc[l] += acc[l + half];
        partials[g] = acc[0];
    }
}

float oc_sum_f32(const float *x, int64_t n)
{
    if (n == 0) return 0.0f;
    if (n < WG) {
        float s = 0.0f;
        for (int64_t i = 0; i < n; ++i) s += x[i];
        return s;
    }
    const float *cur = x;
    float *tmp[2] = {NULL, NULL};
    int which = 0;
    int64_t remaining = n;
    while (remaining > (int64_t)RPW * MAX_WG) {
        const int64_t groups = (remaining + (int64_t)RPW * WG - 1) / ((int64_t)RPW * WG);
        tmp[which] = (float *)realloc(tmp[which], (size_t)groups * sizeof(float));
        sum_level(cur, remaining, WG, RPW, tmp[which], groups);
        cur = tmp[which];
        which ^= 1;
        remaining = groups;
    }
    float res;
    sum_level(cur, remaining, MAX_WG, (remaining + MAX_WG - 1) / MAX_WG, &res, 1);
    free(tmp[0]);
    free(tmp[1]);
    return res;
}

static inline int better(int is_max, float v, float cur) { return is_max ? (v > cur) : (v < cur); }
/* Maximum / Minimum of libtensor/include/utils/sycl_utils.hpp:332-376 */
static inline float pick(int is_max, float x, float y)
{
    return (isnan(x) || (is_max ? x > y : x < y)) ? x : y;
}

static void search_level(int is_max, int first, const float *vals, const int64_t *inds, int64_t n, int wg,
                         int64_t rpw, float *out_vals, int64_t *out_inds, int64_t ngroups)
{
    const float identity = is_max ? -INFINITY : INFINITY;
#pragma omp parallel for schedule(static)
    for (int64_t g = 0; g < ngroups; ++g) {
        float lv[MAX_WG];
        int64_t li[MAX_WG];
        for (int l = 0; l < wg; ++l) {
            lv[l] = identity;
            li[l] = INT64_MAX;
        }
        const int64_t base = g * rpw * wg;
        for (int64_t m = 0; m < rpw; ++m) {
            const int64_t off = base + m * wg;
            if (off >= n) break;
            const int lim = (n - off < wg) ? (int)(n - off) : wg;
            for (int l = 0; l < lim; ++l) {
                const float v = vals[off + l];
                const int64_t idx = first ? off + l : inds[off + l];
                if (v == lv[l]) {
                    if (idx < li[l]) li[l] = idx;
                }
                else if (better(is_max, v, lv[l]) || isnan(v)) {
                    lv[l] = v;
                    li[l] = idx;
                }
            }
        }
        float gv = lv[0];
        for (int l = 1; l < wg; ++l) gv = pick(is_max, gv, lv[l]);
        int64_t gi = INT64_MAX;
        for (int l = 0; l < wg; ++l)
            if ((gv == lv[l] || isnan(lv[l])) && li[l] < gi) gi = li[l];
        out_vals[g] = gv;
        out_inds[g] = gi;
    }
}

static int64_t search_f32(int is_max, const float *x, int64_t n)
{
    if (n <= 0) return -1;
    if (n < WG) { /* SequentialSearchReduction, reductions.hpp:1868-1976 */
        float cur = is_max ? -INFINITY : INFINITY;
        int64_t idx = INT64_MAX;
        for (int64_t i = 0; i < n; ++i) {
            const float v = x[i];
            if (v == cur) {
                if (i < idx) idx = i;
            }
            else if (better(is_max, v, cur) || isnan(v)) {
                cur = v;
                idx = i;
            }
        }
        return idx;
    }
    const float *cv = x;
    const int64_t *ci = NULL;
    float *tv[2] = {NULL, NULL};
    int64_t *ti[2] = {NULL, NULL};
    int which = 0, first = 1;
    int64_t remaining = n;
    while (remaining > (int64_t)RPW * MAX_WG) {
        const int64_t groups = (remaining + (int64_t)RPW * WG - 1) / ((int64_t)RPW * WG);
        tv[which] = (float *)realloc(tv[which], (size_t)groups * sizeof(float));
        ti[which] = (int64_t *)realloc(ti[which], (size_t)groups * sizeof(int64_t));
        search_level(is_max, first, cv, ci, remaining, WG, RPW, tv[which], ti[which], groups);
        cv = tv[which];
        ci = ti[which];
        which ^= 1;
        first = 0;
        remaining = groups;
    }
    float rv;
    int64_t ri;
    search_level(is_max, first, cv, ci, remaining, MAX_WG, (remaining + MAX_WG - 1) / MAX_WG, &rv, &ri, 1);
    free(tv[0]);
    free(tv[1]);
    free(ti[0]);
    free(ti[1]);
    return ri;
}

int64_t oc_argmax_f32(const float *x, int64_t n) { return search_f32(1, x, n); }
int64_t oc_argmin_f32(const float *x, int64_t n) { return search_f32(0, x, n); }
