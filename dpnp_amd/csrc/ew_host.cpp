// Elementwise calls: validation and the choice of kernel, independent of element types.
#include <cstdlib>
#include "ew.hpp"
#include "host.hpp"

namespace dpx {

// Checks shared by unary / binary / where / copy calls, in the order of
// py_binary_ufunc (libtensor/source/elementwise_functions/elementwise_functions.hpp:338-381).
// views = inputs..., dst.  Returns DPX_OK with n == 0 for empty iteration spaces.
int ew_validate(int nops, const dpx_array_view *const *views, int64_t &n)
{
    for (int k = 0; k < nops; ++k)
        if (!view_ok(views[k])) return fail(DPX_ERR_BAD_ARGUMENT, "malformed array descriptor");
    const dpx_array_view *dst = views[nops - 1];
    if (!(dst->flags & DPX_WRITABLE)) return fail(DPX_ERR_NOT_WRITABLE, "output array is read-only.");
    for (int k = 0; k + 1 < nops; ++k)
        if (views[k]->nd != dst->nd)
            return fail(DPX_ERR_RANK_MISMATCH, "Array dimensions are not the same.");
    for (int k = 0; k + 1 < nops; ++k)
        if (!same_shape(views[k], dst)) return fail(DPX_ERR_SHAPE_MISMATCH, "Array shapes are not the same.");
    n = view_size(dst);
    if (n == 0) return DPX_OK;
    for (int k = 0; k < nops; ++k)
        if (views[k]->data == nullptr) return fail(DPX_ERR_BAD_ARGUMENT, "null data pointer");
    int64_t lo, hi;
    view_minmax(dst, lo, hi);
    if (hi - lo + 1 < n)
        return fail(DPX_ERR_NOT_AMPLE, "Memory addressed by the output array is not sufficiently ample.");
    for (int k = 0; k + 1 < nops; ++k)
        if (views_overlap(views[k], dst) && !views_same_logical(views[k], dst))
            return fail(DPX_ERR_OVERLAP, "Arrays index overlapping segments of memory");
    return DPX_OK;
}

// block-size override for sweeps (a power of two in [64, 256], else the default); the product
// build compiles tune_int() down to its default
static int env_block(const char *name, int dflt)
{
    const int v = tune_int(name, dflt);
    return (v == 64 || v == 128 || v == 256) ? v : dflt;
}

void ew_make_plan(EwPlan &pl, int nops, const dpx_array_view *const *views)
{
    const dpx_array_view *dst = views[nops - 1];
    pl.nops = nops;
    pl.n = view_size(dst);
    pl.vec = false;
    pl.flat2d = false;
    pl.period = 1;
    pl.bcast = pl.modes = 0;
    pl.tx_log2 = 0;
    pl.rows2_pat = -1;
    pl.outer = pl.outer_fit = 0;
    pl.rows2_scalar = pl.rows2_waves = 0;
    pl.rows2_pairs = 0;
    pl.rows2_wpb = 1;
    pl.block = EW_CONTIG_BLOCK;
    pl.nrows = pl.col_blocks = pl.grid = 0;
    for (int k = 0; k < 5; ++k) pl.offsets[k] = 0;
    if (pl.n == 0) {
        pl.path = DPX_PATH_NOOP;
        pl.nd = 0;
        return;
    }
    for (int d = 0; d < dst->nd; ++d) {
        pl.shape[d] = dst->shape[d];
        for (int k = 0; k < nops; ++k) pl.strides[k][d] = views[k]->strides[d];
    }
    pl.nd = collapse(dst->nd, nops, pl.shape, pl.strides, pl.offsets, false);
    if (pl.nd == 0) { // a single element
        pl.nd = 1;
        pl.shape[0] = 1;
        for (int k = 0; k < nops; ++k) pl.strides[k][0] = 1;
    }
    bool contig = pl.nd == 1 && pl.strides[nops - 1][0] == 1;
    for (int k = 0; k + 1 < nops && contig; ++k)
        contig = pl.strides[k][0] == 1 || pl.strides[k][0] == 0;
    pl.path = contig ? DPX_PATH_EW_CONTIG : DPX_PATH_EW_ROWS;
    pl.tmask = 0;
    pl.dT = -1;
    if (contig || pl.nd < 2 || nops < 2) return;
    // (Rows of 2 MiB and more take the same path: measured on MI355X, fp32 matrix plus a row, 64 x 1000003:
    // 53 -> 63 % of peak, 3 x 2^26: 58 -> 72 %; between 512 bytes and 2 MiB the row kernel is as fast or faster.)
    // A row-major matrix with rows shorter than 512 bytes combined with a row and/or a column
    // (x - mean(x, axis=0), x / norm(x, axis=1)[:, None]): the row kernel would leave most lanes of a
    // wave without a pack; the contiguous kernel walks the matrix flat and indexes the small
    // operands by position modulo / divided by the row length.
    if (pl.nd == 2 && pl.n < ((int64_t)1 << 32) && pl.strides[nops - 1][1] == 1 &&
        pl.strides[nops - 1][0] == pl.shape[1] &&
        (pl.shape[1] * itemsize_of(dst->dtype) < 512 ||
         pl.shape[1] * itemsize_of(dst->dtype) >= (int64_t)tune_int("DPX_EW_FLAT_LONG", 2 << 20))) {
        const bool long_rows = pl.shape[1] * itemsize_of(dst->dtype) >= 512;
        bool ok = true, has_row = false;
        for (int k = 0; k + 1 < nops && ok; ++k) {
            const int64_t s0 = pl.strides[k][0], s1 = pl.strides[k][1];
            ok = (s0 == pl.shape[1] && s1 == 1) || (s0 == 0 && s1 == 1) || (s0 == 1 && s1 == 0) || (s0 == 0 && s1 == 0);
            has_row = has_row || (s0 == 0 && s1 == 1);
            if (long_rows && s0 == 1 && s1 == 0) ok = false; // a column over long rows: one value per row in the row kernel
        }
        if (long_rows && !has_row) ok = false;
        // rows of 8, 16 or 32 whole packs fill the lanes of the row kernel, which then is a little
        // faster (fp32, 10^6 x 64 minus a row: 76 % against 72 % of peak)
        int widest = 1;
        for (int k = 0; k < nops; ++k) widest = std::max(widest, itemsize_of(views[k]->dtype));
        const int64_t row_bytes = pl.shape[1] * widest;
        if (row_bytes == 128 || row_bytes == 256 || row_bytes == 512) ok = false;
        if (ok) {
            pl.path = DPX_PATH_EW_CONTIG;
            pl.flat2d = true;
            return;
        }
    }
    // Transposed operands: the output runs along the inner dim, some input runs along another
    // dim dT (stride 1 there, a long stride along the inner dim).  All such inputs must agree
    // on dT; the others are read in output orientation.
    const int inner = pl.nd - 1;
    if (pl.strides[nops - 1][inner] != 1 || pl.shape[inner] < 16) return;
    int dT = -1;
    uint32_t tmask = 0;
    for (int k = 0; k + 1 < nops; ++k) {
        const int64_t si = pl.strides[k][inner];
        if (si == 0 || si == 1 || si == -1 || si == 2) continue; // row oriented (or a cheap stride)
        int d1 = -1;
        for (int d = 0; d < inner; ++d)
            if (pl.strides[k][d] == 1 && pl.shape[d] >= 16) d1 = d;
        if (d1 < 0) continue;         // strided both ways: nothing to gain from staging
        if (dT >= 0 && d1 != dT) return; // two different orientations: keep the generic kernel
        dT = d1;
        tmask |= 1u << k;
    }
    if (tmask) {
        pl.path = DPX_PATH_EW_TILE;
        pl.tmask = tmask;
        pl.dT = dT;
    }
}

// bits MODE_KEEP_SHIFT + k for inputs with a broadcast (stride 0, extent > 1) dim
static uint32_t keep_bits(const EwPlan &pl)
{
    uint32_t bits = 0;
    for (int k = 0; k + 1 < pl.nops; ++k)
        for (int d = 0; d < pl.nd; ++d)
            if (pl.strides[k][d] == 0 && pl.shape[d] > 1) bits |= 1u << (MODE_KEEP_SHIFT + k);
    return bits;
}

void ew_finish_plan(EwPlan &pl, int E, int U, const int *itemsize, const void *const *ptrs)
{
    if (pl.path == DPX_PATH_NOOP) return;
    const int nops = pl.nops;
    // (packs need no alignment: any operand whose inner stride is 1 is read in packs)
    if (pl.path == DPX_PATH_EW_CONTIG) {
        pl.vec = true;
        pl.bcast = 0;
        for (int k = 0; k + 1 < nops; ++k) {
            uint32_t mode = BC_FULL;
            if (pl.flat2d) {
                const int64_t s0 = pl.strides[k][0], s1 = pl.strides[k][1];
                mode = (s0 == 0 && s1 == 0) ? BC_SCALAR : (s0 == 0 ? BC_PERIODIC : (s1 == 0 ? BC_REPEAT : BC_FULL));
            }
            else if (pl.strides[k][0] == 0 && pl.n > 1) mode = BC_SCALAR;
            pl.bcast |= mode << (2 * k);
        }
        pl.period = pl.flat2d ? (uint32_t)pl.shape[1] : 1u;
        pl.block = env_block("DPX_EW_CONTIG_BLOCK", EW_CONTIG_BLOCK);
        // a kernel that only stores (fill) is one instruction per wave: one-wave blocks are then bound by the
        // rate waves are launched at (2^28 floats: 59 % of the HBM rate, with four waves per block 81 %)
        if (nops == 1) pl.block = 256;
        pl.grid = (pl.n + (int64_t)pl.block * E * U - 1) / ((int64_t)pl.block * E * U);
        return;
    }
    // A one-dimensional call with a stride-2 input (A[:, ::2] of a contiguous matrix with rows of
    // even length collapses to one): cut it into rows of one wave of packs, which is what
    // ew_rows2_kernel works on.
    if (pl.path == DPX_PATH_EW_ROWS && pl.nd == 1 && E >= 2 && pl.strides[nops - 1][0] == 1) {
        const int64_t C = 64 * (int64_t)E;
        bool s2 = false, ok = pl.n % (2 * C) == 0;
        for (int k = 0; k + 1 < nops && ok; ++k) {
            const int64_t st = pl.strides[k][0];
            if (st == 2 && itemsize[k] * E == 16) s2 = true;
            else ok = st == 0 || st == 1;
        }
        if (ok && s2) {
            pl.nd = 2;
            pl.shape[0] = pl.n / C;
            pl.shape[1] = C;
            for (int k = 0; k < nops; ++k) {
                pl.strides[k][1] = pl.strides[k][0];
                pl.strides[k][0] = C * pl.strides[k][1];
            }
        }
    }
    const int inner = pl.nd - 1;
    if (pl.path == DPX_PATH_EW_TILE) {
        // tile = 128 (64 for 16-byte elements) positions along dT x (512 bytes / widest itemsize)
        // positions along the inner dim
        const int64_t TI = ew_tile_ti(16 / E), TJ = 32 * E;
        pl.modes = 0;
        for (int k = 0; k < nops; ++k) {
            uint32_t mode = MODE_STRIDED;
            const bool staged = k + 1 < nops && ((pl.tmask >> k) & 1u);
            // the dim this operand's 16-byte accesses run along
            const int run = staged ? pl.dT : inner;
            if (pl.strides[k][run] == 0 && !staged && k + 1 < nops) mode = MODE_BCAST;
            else if (pl.strides[k][run] == 1) mode = MODE_VEC;
            pl.modes |= mode << (2 * k);
        }
        pl.modes |= keep_bits(pl);
        pl.block = EW_TILE_BLOCK;
        pl.tiles_t = (pl.shape[pl.dT] + TI - 1) / TI;
        pl.tiles_i = (pl.shape[inner] + TJ - 1) / TJ;
        int64_t batch = 1;
        for (int d = 0; d < inner; ++d)
            if (d != pl.dT) batch *= pl.shape[d];
        pl.grid = batch * pl.tiles_t * pl.tiles_i;
        return;
    }
    const int64_t ncols = pl.shape[inner];
    pl.nrows = pl.n / ncols;
    pl.modes = 0;
    for (int k = 0; k < nops; ++k) {
        uint32_t mode = MODE_STRIDED;
        const int64_t s = pl.strides[k][inner];
        if (s == 0 && k + 1 < nops) mode = MODE_BCAST;
        else if (s == 1) mode = MODE_VEC;
        else if (s == 2 && E >= 2 && k + 1 < nops) mode = MODE_VEC2;
        pl.modes |= mode << (2 * k);
    }
    pl.modes |= keep_bits(pl);
    // threads wanted along a row (every operand contiguous along the inner dim and read once: the straight-line
    // form of the rows kernel may move a row's packs back by up to E - 1 columns, which takes one thread more)
    bool all_vec = !(pl.modes >> MODE_KEEP_SHIFT);
    for (int k = 0; k < nops; ++k) all_vec = all_vec && ((pl.modes >> (2 * k)) & 3u) == MODE_VEC;
    {
        // (... unless every row of the output starts on a pack boundary)
        const int64_t pack_bytes = (int64_t)E * itemsize[nops - 1];
        bool rows_aligned = (uintptr_t)ptrs[nops - 1] % (uintptr_t)pack_bytes == 0;
        for (int d = 0; d < inner; ++d)
            rows_aligned = rows_aligned && (pl.shape[d] == 1 || (pl.strides[nops - 1][d] * itemsize[nops - 1]) % pack_bytes == 0);
        all_vec = all_vec && !rows_aligned;
    }
    const int64_t per_row = (ncols + (all_vec ? E - 1 : 0) + E - 1) / E;
    pl.block = env_block("DPX_EW_ROWS_BLOCK", EW_ROWS_BLOCK);
    {
        // One full-size input and the output, both in aligned packs, every other input broadcast along some dim
        // (a matrix plus a row, times a column, minus a per-channel constant): one-wave blocks, like the contiguous
        // kernel's (fp32 16384 x 16384 plus a row or a column: 74 -> 80 % of the HBM rate).  Calls that only write
        // (an outer sum) keep four waves per block (and, for two-operand functions, take ew_outer_kernel); two full-size
        // inputs gain nothing, and lose 7 points when their rows do not start on 16-byte boundaries.
        int streaming = 0;
        bool aligned = ((pl.modes >> (2 * (nops - 1))) & 3u) == MODE_VEC;
        for (int k = 0; k < nops; ++k) {
            const bool out_k = k + 1 == nops;
            bool bcast = false;
            for (int d = 0; d < pl.nd && !out_k; ++d) bcast = bcast || (pl.strides[k][d] == 0 && pl.shape[d] > 1);
            if (bcast) continue;
            if (!out_k) {
                ++streaming;
                aligned = aligned && ((pl.modes >> (2 * k)) & 3u) == MODE_VEC;
            }
            aligned = aligned && (uintptr_t)ptrs[k] % 16 == 0;
            for (int d = 0; d < inner; ++d) aligned = aligned && (pl.strides[k][d] * itemsize[k]) % 16 == 0;
        }
        if (streaming == 1 && aligned && per_row >= 64 && tune_int("DPX_EW_ROWS_ONE_WAVE", 1) != 0) pl.block = 64;
    }
    int lg = 0, lg_max = 0;
    while ((1 << lg_max) < pl.block) ++lg_max;
    while (lg < lg_max && ((int64_t)1 << lg) < per_row) ++lg;
    pl.tx_log2 = lg;
    const int64_t tx = (int64_t)1 << lg, ty = pl.block / tx;
    pl.col_blocks = (per_row + tx - 1) / tx;
    pl.grid = pl.col_blocks * ((pl.nrows + ty - 1) / ty);
    // Does the call fit ew_outer_kernel?  Two inputs, a contiguous output, and every input one value per row, or a
    // row vector (contiguous along the inner dim) that is the same for all rows of dim inner - 1 or for all indices
    // of an earlier dim: nothing of the output's size is read.  Enough rows and columns for its blocks.
    pl.outer_fit = 0;
    if (pl.nd >= 2 && nops == 3 && pl.strides[nops - 1][inner] == 1 && pl.shape[inner - 1] >= 16 && per_row >= 16 &&
        tune_int("DPX_EW_OUTER", 1) != 0) {
        bool ok = true;
        uint32_t mask = 0;
        for (int k = 0; k + 1 < nops; ++k) {
            const int64_t si = pl.strides[k][inner], sm = pl.strides[k][inner - 1];
            if (si == 0) mask |= 1u << k;
            else if (si != 1) ok = false;
            else if (sm != 0) {
                // a vector per row: only one that is the same for every index of some earlier dim (a small operand)
                bool repeats = false;
                for (int d = 0; d < inner - 1; ++d) repeats = repeats || (pl.strides[k][d] == 0 && pl.shape[d] > 1);
                ok = ok && repeats;
            }
        }
        int64_t before = 1;
        for (int d = 0; d < inner - 1; ++d) before *= pl.shape[d];
        const int block = (int)std::min<int64_t>(256, (per_row + 63) / 64 * 64);
        const int64_t cbs = (per_row + block - 1) / block, mbs = (pl.shape[inner - 1] + EW_OUTER_ROWS - 1) / EW_OUTER_ROWS;
        if (ok && before <= 0x7fffffff && cbs * mbs <= 0x7fffffff / std::max<int64_t>(before, 1)) {
            pl.outer_fit = 1;
            pl.outer_per_row = mask;
            pl.outer_mid_blocks = (uint32_t)mbs;
            pl.outer_block = block;
            pl.outer_col_blocks = cbs;
            pl.outer_grid = cbs * mbs * before;
        }
    }
    // Does the call fit ew_rows2_kernel?  Rows of whole waves of packs, an even number of them along
    // dim inner - 1, a contiguous output, and every input one of: stride 2 along the inner dim
    // (elements as wide as a pack allows), contiguous and moving with the rows, or the same for
    // every row (a row vector or a scalar).
    pl.rows2_pat = -1;
    if (E >= 2 && pl.nd >= 2 && pl.strides[nops - 1][inner] == 1 && pl.shape[inner - 1] % 2 == 0 &&
        ncols % (64 * (int64_t)E) == 0 && nops - 1 <= 3 && tune_int("DPX_EW_ROWS2", 1) != 0) {
        int pat = 0;
        uint32_t scalar = 0;
        bool any_s2 = false;
        for (int k = 0; k + 1 < nops && pat >= 0; ++k) {
            const int64_t si = pl.strides[k][inner], sr = pl.strides[k][inner - 1];
            int rc = -1;
            if (si == 2 && itemsize[k] * E == 16) {
                rc = RC_S2;
                any_s2 = true;
                // the wave-wide reads go one element past a row's last: only the row at the highest
                // address may not, and that is the last row when no stride is negative and rows do not
                // interleave (every other row then begins at or beyond the element after its predecessor's
                // last; views with explicit strides smaller than a row's extent take the general kernel)
                for (int d = 0; d < inner; ++d)
                    if (pl.strides[k][d] < 0 || (pl.shape[d] > 1 && pl.strides[k][d] < 2 * ncols - 1)) rc = -1;
            }
            else if (si == 1 && sr != 0) rc = RC_ROWS;
            else if ((si == 1 || si == 0) && sr == 0) {
                rc = RC_ONCE;
                if (si == 0) scalar |= 1u << k;
            }
            pat = rc < 0 ? -1 : (pat | rc << (2 * k));
        }
        if (pat >= 0 && any_s2) {
            pl.rows2_pat = pat;
            pl.rows2_scalar = scalar;
            pl.rows2_waves = (uint32_t)(ncols / (64 * (int64_t)E));
            pl.rows2_pairs = pl.nrows / 2;
            pl.rows2_wpb = tune_int("DPX_EW_ROWS2_WAVES", 1) == 4 ? 4 : 1; // sweep override, product build: 1
        }
    }
}

void ew_export_plan(const EwPlan &pl, dpx_plan *out)
{
    *out = dpx_plan{};
    out->path = pl.path;
    out->nd = pl.nd;
    for (int d = 0; d < pl.nd && pl.path != DPX_PATH_NOOP; ++d) {
        out->shape[d] = pl.shape[d];
        for (int k = 0; k < pl.nops && k < 4; ++k) out->strides[k][d] = pl.strides[k][d];
    }
    for (int k = 0; k < pl.nops && k < 4; ++k) out->offsets[k] = pl.offsets[k];
    out->grid[0] = pl.grid;
    out->grid[1] = out->grid[2] = 1;
    out->block = pl.block;
}

} // namespace dpx
