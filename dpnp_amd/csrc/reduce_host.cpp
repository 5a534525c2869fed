// Reductions: validation and launch planning (no element types here).
#include <algorithm>
#include <cstdint>
#include <cstdlib>
#include "reduce_dispatch.hpp"

namespace dpx {

int red_validate(const dpx_array_view *src, int trailing, const dpx_array_view *dst,
                 const dpx_array_view *aux, bool empty_ok, int aux_dt)
{
    if (!view_ok(src) || !view_ok(dst) || (aux && !view_ok(aux)))
        return fail(DPX_ERR_BAD_ARGUMENT, "malformed array descriptor");
    if (trailing <= 0 || trailing > src->nd)
        return fail(DPX_ERR_BAD_ARGUMENT, "Trailing_dim_to_reduce must be positive, but no greater than rank "
                                          "of the array being reduced");
    const int ndi = src->nd - trailing;
    if (dst->nd != ndi)
        return fail(DPX_ERR_RANK_MISMATCH, "Destination array rank does not match input array rank and number "
                                           "of reduced dimensions");
    for (int d = 0; d < ndi; ++d)
        if (src->shape[d] != dst->shape[d])
            return fail(DPX_ERR_SHAPE_MISMATCH, "Destination shape does not match unreduced dimensions of the input shape");
    if (!(dst->flags & DPX_WRITABLE)) return fail(DPX_ERR_NOT_WRITABLE, "output array is read-only.");
    if (aux) {
        if (!same_shape(aux, dst)) return fail(DPX_ERR_SHAPE_MISMATCH, "aux shape does not match destination shape");
        if (aux_dt < 0 && aux->dtype != dst->dtype)
            return fail(DPX_ERR_BAD_DTYPE, "aux dtype does not match destination dtype");
        if (aux_dt >= 0 && aux->dtype != aux_dt)
            return fail(DPX_ERR_BAD_DTYPE, "aux of complex input must be complex, of the destination's precision");
    }
    const int64_t m = view_size(dst);
    int64_t n = 1;
    for (int d = ndi; d < src->nd; ++d) n *= src->shape[d];
    if (m == 0) return DPX_OK;
    if (n == 0 && !empty_ok) return fail(DPX_ERR_BAD_ARGUMENT, "reduction cannot be performed over zero-size axes");
    if (dst->data == nullptr || (n > 0 && src->data == nullptr) || (aux && aux->data == nullptr))
        return fail(DPX_ERR_BAD_ARGUMENT, "null data pointer");
    if (views_overlap(src, dst) || (aux && views_overlap(aux, dst)))
        return fail(DPX_ERR_OVERLAP, "Arrays index overlapping segments of memory");
    int64_t lo, hi;
    view_minmax(dst, lo, hi);
    if (hi - lo + 1 < m)
        return fail(DPX_ERR_NOT_AMPLE, "Memory addressed by the output array is not sufficiently ample.");
    return DPX_OK;
}

static int ceil_log2(int64_t v)
{
    int lg = 0;
    while (((int64_t)1 << lg) < v) ++lg;
    return lg;
}
static int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Measured on MI355X (2^28 floats): HBM streams best when each CU runs about 8 waves with
// 4 x 16-byte loads in flight per lane (85-87 % of peak); 16 or 32 waves per CU, or
// 1024-thread blocks, lose 5-10 points, and a grid that is not a multiple of the CU count
// loses as much to the tail.  Hence: 256-thread blocks, two per CU when a reduction has to
// be split.
// (the override is clamped so that outputs x splits stays within the ticket table)
static int64_t red_target_blocks()
{
    return std::min<int64_t>(std::max(tune_int("DPX_RED_TARGET_BLOCKS", 2 * device_cus()), 1), RED_MAX_TICKETS);
}

// lanes cooperating on one output of `n` elements read `e` at a time: aim at ~8 accesses
// per lane; more than a wave means a whole 256-thread block
static void rows_geometry(int64_t n, int e, int &g_log2, int &block)
{
    int64_t lanes = cdiv(n, (int64_t)e * 8);
    const int forced = tune_int("DPX_ROWS_G_LOG2", -1); // sweep override, product build: default
    if (forced >= 0) lanes = (int64_t)1 << forced;
    if (lanes <= 64) {
        g_log2 = ceil_log2(lanes);
        block = 256;
    }
    else if (forced >= 7 && forced <= 10) {
        g_log2 = forced;
        block = 1 << forced;
    }
    else {
        g_log2 = 8;
        block = 256;
    }
}

void red_make_plan(RedPlan &pl, const dpx_array_view *src, int trailing, const dpx_array_view *dst,
                   const dpx_array_view *aux, bool keep_order, int in_size, bool arg, bool rows_only)
{
    pl = RedPlan{};
    const int nd = src->nd, ndi = nd - trailing;
    int64_t m = 1, n = 1;
    for (int d = 0; d < ndi; ++d) m *= src->shape[d];
    for (int d = ndi; d < nd; ++d) n *= src->shape[d];
    pl.L.m = m;
    pl.L.n = n;
    pl.L.splits = 1;
    if (m == 0) {
        pl.path = DPX_PATH_NOOP;
        return;
    }
    // iteration space: src (leading dims), aux, dst collapse together
    int64_t ishape[DPX_MAX_ND], istr[3][DPX_MAX_ND], ioff[3];
    for (int d = 0; d < ndi; ++d) {
        ishape[d] = src->shape[d];
        istr[0][d] = src->strides[d];
        istr[1][d] = aux ? aux->strides[d] : 0;
        istr[2][d] = dst->strides[d];
    }
    int nd_i = collapse(ndi, 3, ishape, istr, ioff, false);
    if (nd_i == 0) {
        nd_i = 1;
        ishape[0] = 1;
        istr[0][0] = istr[1][0] = istr[2][0] = 0;
    }
    int64_t rshape[DPX_MAX_ND], rstr[1][DPX_MAX_ND], roff[1] = {0};
    int nd_r = 0;
    if (n > 0) {
        for (int d = 0; d < trailing; ++d) {
            rshape[d] = src->shape[ndi + d];
            rstr[0][d] = src->strides[ndi + d];
        }
        nd_r = collapse(trailing, 1, rshape, rstr, roff, keep_order);
    }
    if (nd_r == 0) {
        nd_r = 1;
        rshape[0] = n > 0 ? 1 : 0;
        rstr[0][0] = 1;
    }
    RedIndex &ix = pl.ix;
    ix.nd_i = nd_i;
    ix.nd_r = nd_r;
    for (int d = 0; d < DPX_MAX_ND; ++d) {
        ix.shape_i[d] = d < nd_i ? ishape[d] : 1;
        ix.src_istr[d] = d < nd_i ? istr[0][d] : 0;
        ix.aux_str[d] = d < nd_i ? istr[1][d] : 0;
        ix.dst_str[d] = d < nd_i ? istr[2][d] : 0;
        ix.shape_r[d] = d < nd_r ? rshape[d] : 1;
        ix.src_rstr[d] = d < nd_r ? rstr[0][d] : 0;
    }
    pl.L.nd_i1 = nd_i == 1 ? 1 : 0;
    pl.L.istr0 = istr[0][0];
    pl.L.astr0 = istr[1][0];
    pl.L.dstr0 = istr[2][0];
    pl.src_off = ioff[0] + roff[0];
    pl.aux_off = ioff[1];
    pl.dst_off = ioff[2];
    if (n == 0) {
        pl.path = DPX_PATH_RED_SMALL; // identity fill
        pl.block = 256;
        pl.grid = cdiv(m, 256);
        return;
    }

    const int E = 16 / in_size;
    const int64_t target = red_target_blocks();
    const int last = nd_i - 1;
    const int64_t inner = ishape[last];
    const bool contig_red = nd_r == 1 && (rstr[0][0] == 1 || n == 1);
    const bool cols_plain = !contig_red && nd_r == 1 && istr[0][last] == 1 && inner > 1;
    // the same arrangement (threads side by side along the inner iteration dim, rows of the reduced space walked
    // by offset) when that dim is the one src moves least along, whatever its stride and however many reduced
    // dims stay apart: axes (0, 2) of a 4-d array, columns of a matrix view that takes every other column
    bool cols_walk = false;
    if (!contig_red && !cols_plain && !arg && nd_r <= 3 && inner > 1 && istr[0][last] != 0 &&
        rshape[nd_r - 1] < ((int64_t)1 << 31) && (nd_r < 2 || rshape[nd_r - 2] < ((int64_t)1 << 31))) {
        int64_t smin = INT64_MAX;
        for (int d = 0; d < nd_r; ++d) smin = std::min(smin, rstr[0][d] < 0 ? -rstr[0][d] : rstr[0][d]);
        const int64_t si = istr[0][last] < 0 ? -istr[0][last] : istr[0][last];
        cols_walk = si < smin;
    }
    const bool cols_ok = cols_plain || cols_walk;
    RedLaunch &L = pl.L;

    if (!rows_only && contig_red && nd_i == 1 && istr[0][0] == n && n >= 2 && n * in_size <= 256 && m >= 64 &&
        tune_int("DPX_RED_SHORT_ROWS", 1) != 0) { // (sweep override: 0 keeps the rows kernel)
        // ---- short rows: a block stages R whole rows in LDS (see red_short_rows_kernel) ----
        const int64_t pitch_bytes = (int64_t)srow_pitch_for((int)n, in_size) * in_size;
        const int64_t R = std::min<int64_t>(2048, SROW_LDS_BYTES / pitch_bytes);
        L.vec = 1;
        L.g_log2 = 0;
        L.chunk = R;
        L.splits = 1;
        L.tgroup = 0;
        pl.block = 256;
        pl.grid = cdiv(m, R);
        pl.path = DPX_PATH_RED_SHORT_ROWS;
        return;
    }
    if (!cols_ok) {
        // ---- rows / generic -------------------------------------------------------
        bool vec = contig_red; // packs need no alignment
        int e = vec ? E : 1;
        int64_t work = n; // what lanes and splits share out: elements, or the units of a walked space
        // (the kernels keep the two inner digits of a walked space and a run's length in 32 bits)
        const int64_t lim32 = (int64_t)1 << 31;
        if (!contig_red && nd_r <= 3 && rshape[nd_r - 1] < lim32 && (nd_r < 2 || rshape[nd_r - 2] < lim32)) {
            // reduced dims that stay apart (a sliced matrix summed whole, axes (0, 2) of a 3-d array, a
            // strided run): lanes walk the reduced space in units of its last dim, 16-byte packs when that
            // dim has unit stride and holds at least one
            int64_t c = rshape[nd_r - 1];
            const int64_t s_in = rstr[0][nd_r - 1];
            vec = s_in == 1 && c >= E;
            L.walk = 1;
            if (s_in == 2 && E >= 4 && c >= E && 2 * c < lim32) {
                // every other element of a run: the lines it touches are read as packs, half of each is used
                vec = true;
                c = 2 * c - 1;
                L.walk = 2;
            }
            const int64_t per_run = vec ? cdiv(c, E) : c;
            for (int j = 0; j < 3; ++j) {
                const int d = nd_r - 3 + j; // digit j is reduced dim d, or missing
                L.wd[j] = d < 0 ? 1 : rshape[d];
                L.ws[j] = d < 0 ? 0 : rstr[0][d];
            }
            L.wd[2] = per_run;
            L.ws[2] = vec ? E : s_in;
            L.inner = c;
            L.units = work = (n / rshape[nd_r - 1]) * per_run;
            e = 1;
        }
        L.vec = vec ? 1 : 0;
        rows_geometry(work, e, L.g_log2, pl.block);
        if (L.walk && vec && pl.block == 256 && L.g_log2 == 8 && m > target && m <= 8 * target &&
            tune_int("DPX_ROWS_G_LOG2", -1) < 0) {
            // A walked space with more outputs than split plans have blocks: a wave's loads of one round go to
            // runs that lie far apart, and with every output on a whole 256-thread block four times as many waves
            // as a split plan runs stream from that many places at once (256 x 1024 x 1024 floats summed over
            // axes 0 and 2: 74 % of the HBM rate; 128 x 2048 x 1024: 71 %).  Fewer lanes per output, for as many
            // waves as a split plan has (4 per block, `target` blocks): 86 % and 90 %; half as many waves again
            // lose 20 points.
            L.g_log2 = ceil_log2(cdiv(64 * 4 * target, m));
            pl.block = L.g_log2 >= 7 ? 1 << L.g_log2 : 256;
        }
        const int64_t G = (int64_t)1 << L.g_log2;
        const int64_t opb = (G <= 64) ? 256 / G : 1;
        const int64_t oblocks = cdiv(m, opb);
        int64_t splits = 1;
        const int64_t per_pass = G * e * 8; // elements one group covers with 8 accesses per lane
        // splitting needs a whole block per output (G > 64) and one ticket counter per output
        // (the largest split count whose grid stays within the target: a grid a little above it
        // runs a second, nearly empty round of blocks and loses 10-15 points of bandwidth)
        // (single elements in flight instead of packs: more blocks per CU make up for the bytes)
        const int64_t tgt = (L.walk && !vec) ? target * (in_size >= 16 ? 1 : (in_size == 8 ? 2 : 4)) : target;
        if (G > 64 && 2 * oblocks <= tgt && oblocks <= RED_MAX_TICKETS && work >= 2 * per_pass)
            splits = std::min(tgt / oblocks, cdiv(work, per_pass));
        // 32-bit positions inside a chunk (a walked space counts the whole last pack of every run: below 2 n)
        if (arg && G > 64 && oblocks <= RED_MAX_TICKETS)
            splits = std::max(splits, cdiv(n, (int64_t)1 << (L.walk ? 30 : 31)));
        int64_t chunk = cdiv(work, splits);
        chunk = cdiv(chunk, G * e) * (G * e);
        splits = cdiv(work, chunk);
        L.chunk = chunk;
        L.splits = (int32_t)splits;
        // many blocks per output: two levels of tickets (groups of 32 blocks), while the group
        // counters of all outputs fit their table
        L.tgroup = (splits >= 128 && m * cdiv(splits, 32) <= RED_MAX_GROUPS) ? 32 : 0;
        pl.grid = oblocks * splits;
        pl.path = !contig_red ? DPX_PATH_RED_GENERIC
                              : (splits > 1 ? DPX_PATH_RED_ROWS_SPLIT
                                            : (G == 1 ? DPX_PATH_RED_SMALL : DPX_PATH_RED_ROWS));
        if (splits > 1) pl.scratch_elems = m * splits;
        return;
    }
    // ---- cols -----------------------------------------------------------------------
    const int64_t rstride = rstr[0][0];
    if (!rows_only && !cols_walk && nd_i == 1 && rstride == inner && inner * in_size < 512 && n >= 16 &&
        tune_int("DPX_RED_FLAT", 1) != 0) { // (sweep override: 0 keeps the column kernel)
        // a row-major matrix with rows shorter than 512 bytes: one flat stream of packs, a block of
        // T threads with T * E a multiple of the row length (see red_flat_kernel)
        int64_t g = inner, b = E;
        while (b) {
            const int64_t r = g % b;
            g = b;
            b = r;
        }
        const int64_t period = inner / g; // threads after which the columns of a pack repeat
        if (period <= 256) {
            const int64_t T = period * (256 / period);
            const int64_t per_block = T * E * 8; // at least 8 packs per thread
            int64_t blocks = std::max<int64_t>(1, std::min<int64_t>(target, (n * inner) / per_block));
            if (arg) blocks = std::max(blocks, cdiv(n, (int64_t)1 << 31)); // 32-bit rows inside a block
            {
                const int64_t chunk = cdiv(n, blocks);
                blocks = cdiv(n, chunk);
                L.vec = 1;
                L.g_log2 = 0;
                L.rstride = rstride;
                L.inner = inner;
                L.col_blocks = 1;
                L.chunk = chunk;
                L.splits = (int32_t)blocks;
                L.tgroup = 0;
                pl.block = (int)T;
                pl.grid = blocks;
                pl.path = DPX_PATH_RED_FLAT;
                if (blocks > 1) pl.scratch_elems = blocks * inner;
                return;
            }
        }
    }
    // packs need no alignment; the kernels read a row's last pack by element
    // every other column of a matrix (src stride 2 along the inner iteration dim): the lines are read whole, as
    // packs, and the places in between are dropped: the geometry below is that of the lines (`width` elements)
    const bool half = cols_walk && istr[0][last] == 2 && E >= 4 && 2 * inner - 1 >= E;
    const bool vec = !cols_walk || istr[0][last] == 1 || half;
    const int e = vec ? E : 1;
    const int64_t width = half ? 2 * inner - 1 : inner;
    L.vec = vec ? 1 : 0;
    L.rstride = rstride;
    L.inner = width;
    if (cols_walk) {
        for (int j = 0; j < 3; ++j) {
            const int d = nd_r - 3 + j; // digit j is reduced dim d, or missing
            L.wd[j] = d < 0 ? 1 : rshape[d];
            L.ws[j] = d < 0 ? 0 : rstr[0][d];
        }
        L.walk = half ? 2 : 1;
        L.units = n;
        L.istep = istr[0][last];
    }
    // TX threads side by side cover 512 contiguous bytes of a row (32 x 16 B); up to 16 thread
    // rows walk down the reduced axis: 512-thread blocks, one per CU when splitting
    // thread rows wanted for n reduced rows (4 or more rows per thread)
    // (rounded down: with fewer than 4 rows a thread never has its 4 loads in flight together)
    int64_t ty = 1;
    while (ty < 16 && 8 * ty <= n) ty *= 2;
    // with a single thread row a whole wave lies side by side and nothing is combined in LDS
    // (single elements at a stride: a whole wave side by side as well, 64 elements are the least it should span)
    // rows that do not start on 16-byte boundaries (an odd row length): a thread row's run touches one line more
    // than it fills, which is a quarter more lines for 512 bytes and an eighth for the 1024 bytes of a whole
    // wave side by side (16385 x 16385 floats summed down the columns: 60 -> 76 % of the HBM rate; 2-byte
    // elements and searches of 4-byte ones gain nothing or lose)
    const bool misaligned = !cols_walk && (rstride * in_size) % 16 != 0 && in_size >= (arg ? 8 : 4);
    int lg = std::min((ty == 1 || !vec || misaligned) ? 6 : 5, ceil_log2(cdiv(width, e)));
    const int forced = tune_int("DPX_COLS_TX_LOG2", -1); // sweep override, product build: default
    if (forced >= 0 && forced <= 8) lg = std::min(ceil_log2(cdiv(width, e)), forced);
    L.g_log2 = lg;
    const int64_t TX = (int64_t)1 << lg;
    int block = (int)std::min<int64_t>(arg ? 256 : 512, std::max<int64_t>(64, TX * ty));
    if (!arg) {
        const int fb = tune_int("DPX_COLS_BLOCK", 0); // sweep override, product build: default
        if (fb == 256 || fb == 512) block = fb;
    }
    if (block < TX) block = (int)TX;
    const int64_t TY = block / TX;
    L.col_blocks = cdiv(width, TX * e);
    const int64_t outer = m / inner;
    const int64_t base_blocks = L.col_blocks * outer;
    const int64_t want = std::max<int64_t>(target * 256 / block, 1); // same number of threads in flight
    int64_t splits = 1;
    // the largest split count that still gives every block a CU of its own at once: a grid a little
    // above a multiple of the CU count runs up to a third slower than one a little below it
    if (2 * base_blocks <= want && base_blocks <= RED_MAX_TICKETS && n >= 2 * TY * 8)
        splits = std::min(want / base_blocks, cdiv(n, TY * 8));
    if (arg) splits = std::max(splits, cdiv(n, (int64_t)1 << 31)); // 32-bit positions inside a chunk
    int64_t chunk = cdiv(n, splits);
    splits = cdiv(n, chunk);
    L.chunk = chunk;
    L.splits = (int32_t)splits;
    // searches over few columns (many blocks per column block): the partial pairs are folded in two levels
    L.tgroup = (arg && splits >= 64 && base_blocks * cdiv(splits, 32) <= RED_MAX_GROUPS) ? 32 : 0;
    if (arg && splits == 1 && TY > 1 && n >= 24 && n <= 96 && outer >= 2 * (256 / TX)) {
        // searches down short columns under many outer indices (argmax along the middle axis of batch x 32 x
        // features): the thread rows of a 256-thread block are outer indices, a thread walks its whole column
        // (65536 x 32 x 128 floats: 61 -> 76 % of the HBM rate, 65536 x 64 x 64: 44 -> 73 %; columns of 8 and 16
        // rows are better off with two thread rows that meet in LDS: 82 and 80 % against 74 and 77 %)
        L.obatch = 1;
        pl.block = 256;
        pl.grid = L.col_blocks * cdiv(outer, 256 / TX);
        pl.path = DPX_PATH_RED_COLS;
        return;
    }
    pl.block = block;
    pl.grid = base_blocks * splits;
    pl.path = splits > 1 ? DPX_PATH_RED_COLS_SPLIT : DPX_PATH_RED_COLS;
    if (splits > 1) pl.scratch_elems = m * splits;
}

void red_export_plan(const RedPlan &pl, dpx_plan *out, int acc_size)
{
    *out = dpx_plan{};
    out->path = pl.path;
    if (pl.path == DPX_PATH_NOOP) return;
    out->nd = pl.ix.nd_i;
    out->red_nd = pl.ix.nd_r;
    for (int d = 0; d < pl.ix.nd_i; ++d) {
        out->shape[d] = pl.ix.shape_i[d];
        out->strides[0][d] = pl.ix.src_istr[d];
        out->strides[1][d] = pl.ix.dst_str[d];
    }
    for (int d = 0; d < pl.ix.nd_r; ++d) {
        out->strides[2][d] = pl.ix.shape_r[d];
        out->strides[3][d] = pl.ix.src_rstr[d];
    }
    out->offsets[0] = pl.src_off;
    out->offsets[1] = pl.dst_off;
    out->vec = pl.L.vec;
    out->grid[0] = pl.grid;
    out->grid[1] = out->grid[2] = 1;
    out->block = pl.block;
    out->splits = pl.L.splits;
    out->scratch_bytes = pl.scratch_elems ? (int64_t)RED_COUNTER_BYTES + pl.scratch_elems * ((acc_size + 3) / 4 * 4) : 0;
}

} // namespace dpx
