// Elementwise kernel engine: one N-ary kernel pair (contiguous / row-vectorised
// strided) instantiated for every functor and element-type combination.
//
// Replaces the Unary/Binary{Contig,Strided,RowBroadcast}Functor kernels and
// their launchers (libtensor/include/kernels/elementwise_functions/common.hpp:70-689,
// common_inplace.hpp:69-273, libtensor/include/kernels/where.hpp:72-262).
//
// Layout choices for MI355X:
//   * every thread moves 16 bytes of the widest operand per access
//     (global_load_dwordx4 / global_store_dwordx4, non-temporal) and makes exactly
//     one access per operand; contiguous kernels run one wave (64 threads) per
//     block: many short-lived waves keep the HBM queues full and the hardware
//     dispatcher walks the arrays front to back.  Measured on MI355X for
//     c = a + b over 2^28 floats: 64-thread blocks 6.6-6.8 TB/s, 256-thread
//     blocks 6.3-6.5 TB/s, grid-stride loops 5.3-6.0 TB/s, no NT hint -5 %;
//   * shape and strides of the collapsed iteration space travel in the kernel
//     argument segment (no device-side metadata buffers to allocate or free);
//   * strided kernels keep threads adjacent along the innermost output
//     dimension and pay one div/mod chain per thread, not per element.
#pragma once
#include <array>
#include <atomic>
#include <tuple>
#include <utility>
#include "types.hpp"

namespace dpx {

constexpr int EW_BLOCK = 256;       // upper bound of threads per block
constexpr int EW_CONTIG_BLOCK = 64; // default for contiguous kernels: one wave
constexpr int EW_ROWS_BLOCK = 256;  // default for strided kernels

// operand access mode along the inner dimension (2 bits per operand)
enum : uint32_t { MODE_STRIDED = 0, MODE_VEC = 1, MODE_BCAST = 2, MODE_VEC2 = 3 };
// bit MODE_KEEP_SHIFT + k of `modes`: input k is read more than once (a broadcast dim), so its
// loads are ordinary cached ones instead of non-temporal
constexpr int MODE_KEEP_SHIFT = 16;

template <int NOPS> struct NdIndex {
    int32_t nd; // >= 1; the last dim is the inner one
    int32_t pad;
    int64_t shape[DPX_MAX_ND];
    int64_t strides[NOPS][DPX_MAX_ND];
};

template <int N> struct InPtrs {
    const void *p[N];
};

template <class Out, class... Ins> struct ew_traits {
    static constexpr int width = max_sizeof<Out, Ins...>();
    static constexpr int E = 16 / width; // elements per pack: the widest operand moves 16 bytes
    // Contiguous kernels: packs per thread.  A thread that moves 20 bytes or less per pack (a cast
    // from a wide to a narrow type, a predicate) takes two.  Measured on MI355X over 1 GiB of
    // input: f8 -> i1 0.224 -> 0.193 ms, isnan(f4) 0.227 -> 0.198 ms; at 24 bytes per pack
    // (f4 -> f8) two packs are slower than one, 0.476 -> 0.521 ms.
    static constexpr int pack_bytes = E * (int)(sizeof(Out) + (size_t(0) + ... + sizeof(Ins)));
    // a kernel without inputs (fill) stores one pack per thread, in blocks of four waves
    static constexpr int U = (sizeof...(Ins) > 0 && pack_bytes <= 20) ? 2 : 1;
};

// Packs per thread of the contiguous kernel for functor Fn.  A functor may ask for two with a member
// `static constexpr bool two_packs = true` (some fp64 routines: the 64-bit constants a thread
// materialises then serve four elements instead of two.  Measured on 2^26 doubles: expm1 67 -> 80 %,
// log2 63 -> 66-73 % of HBM peak; light functions lose 2-3 points with two packs and most heavy ones
// gain nothing, so it is not the rule).
template <class Fn, class = void> struct fn_two_packs : std::false_type {};
template <class Fn> struct fn_two_packs<Fn, std::enable_if_t<Fn::two_packs>> : std::true_type {};
template <class Fn, class = void> struct fn_two_phase : std::false_type {};
template <class Fn> struct fn_two_phase<Fn, std::enable_if_t<Fn::two_phase>> : std::true_type {};
template <class Fn, class Out, class... Ins> constexpr int ew_packs_per_thread()
{
    return (fn_two_packs<Fn>::value && ew_traits<Out, Ins...>::U == 1) ? 2 : ew_traits<Out, Ins...>::U;
}

template <class T, int E> DPX_D pack<T, E> splat(T v)
{
    pack<T, E> p;
#pragma unroll
    for (int e = 0; e < E; ++e) p.v[e] = v;
    return p;
}

// ---- contiguous ---------------------------------------------------------------
// grid.x * blockDim.x * E * U >= n.  Pack u of thread t in block b covers elements
// ((b * U + u) * blockDim.x + t) * E ... + E of the output.  `bcast` holds 2 bits per input:
// BC_FULL the input has an element per output element; BC_SCALAR it is a single element;
// BC_PERIODIC it has `period` elements and output element i takes element i mod period (a row
// added to every row of a row-major matrix with short rows); BC_REPEAT output element i takes
// element i / period (a column, one element per row).  The last two need n < 2^32.
enum : uint32_t { BC_FULL = 0, BC_SCALAR = 1, BC_PERIODIC = 2, BC_REPEAT = 3 };

template <class T> DPX_D T load_bcast_one(const T *p, uint32_t mode, int64_t i, uint32_t period)
{
    switch (mode) {
    case BC_FULL: return load_one(p + i);
    case BC_SCALAR: return load_one(p);
    case BC_PERIODIC: return load_one(p + (uint32_t)i % period);
    default: return load_one(p + (uint32_t)i / period);
    }
}
template <class T, int E> DPX_D pack<T, E> load_bcast_pack(const T *p, uint32_t mode, int64_t base, uint32_t period)
{
    if (mode == BC_FULL) return load_pack<T, E>(p + base);
    if (mode == BC_SCALAR) return splat<T, E>(load_one(p));
    // a small vector that stays in cache: element-wise reads, one division per pack
    uint32_t r = (uint32_t)base / period, c = (uint32_t)base - r * period;
    pack<T, E> v;
#pragma unroll
    for (int e = 0; e < E; ++e) {
        v.v[e] = load_one(p + (mode == BC_PERIODIC ? c : r));
        if (++c == period) {
            c = 0;
            ++r;
        }
    }
    return v;
}

template <class Fn, class Out, class... Ins, size_t... I>
DPX_D void ew_contig_pack(const Fn &fn, Out *out, int64_t base,
                          std::tuple<pack<Ins, ew_traits<Out, Ins...>::E>...> &v, std::index_sequence<I...>)
{
    constexpr int E = ew_traits<Out, Ins...>::E;
    (keep_whole(std::get<I>(v)), ...);
    pack<Out, E> r;
    if constexpr (fn_two_phase<Fn>::value) {
        if constexpr (Fn::has_cheap) {
            // a whole wave of arguments the functor has a cheap form for (x ** 2) takes only that
            bool cheap = true;
#pragma unroll
            for (int e = 0; e < E; ++e) cheap = cheap && fn.cheap_applies(to_value(std::get<I>(v).v[e])...);
            if (__builtin_amdgcn_ballot_w64(!cheap) == 0) {
#pragma unroll
                for (int e = 0; e < E; ++e) r.v[e] = to_storage<Out>(fn.cheap(to_value(std::get<I>(v).v[e])...));
                store_pack<Out, E>(out + base, r);
                return;
            }
        }
        // the straight-line part for every element first, then the rare branches
        decltype(fn.fast(to_value(std::get<I>(v).v[0])...)) t[E];
#pragma unroll
        for (int e = 0; e < E; ++e) t[e] = fn.fast(to_value(std::get<I>(v).v[e])...);
        // the results exist here: without this the compiler moves each element's chain down to its branch
#pragma unroll
        for (int e = 0; e < E; ++e) asm volatile("" : "+v"(t[e]));
#pragma unroll
        for (int e = 0; e < E; ++e) r.v[e] = to_storage<Out>(fn.fixup(t[e], to_value(std::get<I>(v).v[e])...));
    }
    else {
#pragma unroll
        for (int e = 0; e < E; ++e) r.v[e] = to_storage<Out>(fn(to_value(std::get<I>(v).v[e])...));
    }
    store_pack<Out, E>(out + base, r);
}

template <class Fn, class Out, class... Ins, size_t... I>
DPX_D void ew_contig_body(const Fn &fn, int64_t n, uint32_t bcast, uint32_t period, Out *out,
                          const InPtrs<sizeof...(Ins)> &in, std::index_sequence<I...> seq)
{
    constexpr int E = ew_traits<Out, Ins...>::E;
    constexpr int U = ew_packs_per_thread<Fn, Out, Ins...>();
    const int64_t block_base = (int64_t)blockIdx.x * ((int)blockDim.x * E * U);
    auto load = [&](int64_t base, std::tuple<pack<Ins, E>...> &v) {
        ((std::get<I>(v) = load_bcast_pack<Ins, E>((const Ins *)in.p[I], (bcast >> (2 * I)) & 3u, base, period)), ...);
    };
    if (block_base + (int64_t)blockDim.x * E * U <= n) { // the usual case: every load first
        std::tuple<pack<Ins, E>...> v[U];
        if (bcast == 0) {
            // every input has an element per output element: a path of its own, because with one element
            // per pack (16-byte elements) the compiler folds the loads of all modes into one instruction
            // and the streaming hint of this one is lost (complex128 add: 77 % of the HBM rate)
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int64_t base = block_base + ((int64_t)u * (int)blockDim.x + threadIdx.x) * E;
                ((std::get<I>(v[u]) = load_pack<Ins, E>((const Ins *)in.p[I] + base)), ...);
            }
            // nothing to execute; it ends the run of instructions this path has in common with the other one,
            // which the compiler would otherwise move behind the point where the two meet, the last load included
            asm volatile("" ::: "memory");
#pragma unroll
            for (int u = 0; u < U; ++u)
                ew_contig_pack<Fn, Out, Ins...>(fn, out, block_base + ((int64_t)u * (int)blockDim.x + threadIdx.x) * E,
                                                v[u], seq);
            return; // (a path to the end: loads that met the other modes' loads again would be folded with them)
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
            load(block_base + ((int64_t)u * (int)blockDim.x + threadIdx.x) * E, v[u]);
#pragma unroll
        for (int u = 0; u < U; ++u)
            ew_contig_pack<Fn, Out, Ins...>(fn, out, block_base + ((int64_t)u * (int)blockDim.x + threadIdx.x) * E,
                                            v[u], seq);
        return;
    }
    for (int u = 0; u < U; ++u) { // the block that holds the end of the array
        const int64_t base = block_base + ((int64_t)u * (int)blockDim.x + threadIdx.x) * E;
        if (base + E <= n) {
            std::tuple<pack<Ins, E>...> v;
            load(base, v);
            ew_contig_pack<Fn, Out, Ins...>(fn, out, base, v, seq);
        }
        else
            for (int64_t i = base; i < n; ++i)
                out[i] = to_storage<Out>(fn(to_value(
                    load_bcast_one((const Ins *)in.p[I], (bcast >> (2 * I)) & 3u, i, period))...));
    }
}

template <class Fn, class Out, class... Ins>
__global__ __launch_bounds__(EW_BLOCK) void ew_contig_kernel(Fn fn, int64_t n, uint32_t bcast, uint32_t period,
                                                            Out *out, InPtrs<sizeof...(Ins)> in)
{
    ew_contig_body<Fn, Out, Ins...>(fn, n, bcast, period, out, in, std::index_sequence_for<Ins...>{});
}

// Stride-2 operand (x[:, ::2], real or imaginary parts) read by a whole wave: the lane's E
// elements x[0], x[2], ..., x[2E-2] start at `lane_ptr`; lanes are 2E elements apart.  The wave
// reads its 2 KiB run with two lane-interleaved 16-byte loads (each instruction covers 1 KiB
// without holes) and the lanes then pull the two packs that hold their elements from their
// neighbours' registers.  All 64 lanes of the wave must make the call.  Measured on MI355X
// against two loads at a 32-byte lane pitch: 6.4 vs 5.9 TB/s of physical traffic.
template <class T, int E> DPX_D void stride2_wave_issue(const T *lane_ptr, u32x4 &a, u32x4 &b)
{
    const int lane = threadIdx.x & 63;
    const T *wp = lane_ptr - (int64_t)lane * 2 * E;
    a = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(wp + lane * E));
    b = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(wp + (64 + lane) * E));
}
template <class T, int E> DPX_D pack<T, E> stride2_wave_regroup(const u32x4 &a, const u32x4 &b)
{
    static_assert(E >= 2 && sizeof(T) * E == 16);
    const int lane = threadIdx.x & 63;
    const int s = (2 * lane) & 63;
    const bool first = lane < 32;
    union {
        u32x4 r;
        pack<T, E> p;
    } lo, hi;
    lo.r = u32x4{0, 0, 0, 0};
    hi.r = u32x4{0, 0, 0, 0};
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        // dwords that hold an element of even index
        if (sizeof(T) >= 4 && ((d * 4 / (int)sizeof(T)) & 1)) continue;
        const uint32_t a0 = __shfl(a[d], s), b0 = __shfl(b[d], s);
        const uint32_t a1 = __shfl(a[d], s + 1), b1 = __shfl(b[d], s + 1);
        lo.r[d] = first ? a0 : b0;
        hi.r[d] = first ? a1 : b1;
    }
    pack<T, E> r;
#pragma unroll
    for (int e = 0; e < E; ++e) r.v[e] = (2 * e < E) ? lo.p.v[(2 * e) % E] : hi.p.v[(2 * e) % E];
    return r;
}
// issue and regroup are separate so that a thread can have the loads of several rows in flight
// before the first shuffle waits for data
template <class T, int E> DPX_D pack<T, E> load_stride2_wave(const T *lane_ptr)
{
    u32x4 a, b;
    stride2_wave_issue<T, E>(lane_ptr, a, b);
    return stride2_wave_regroup<T, E>(a, b);
}

// ---- strided, vectorised along the inner dimension -----------------------------
// Block = TY rows x TX threads (TX = 1 << tx_log2, TX * TY = blockDim.x); a thread owns E
// consecutive inner positions of one row.  ix.strides[k] for inputs k < N,
// ix.strides[N] for the output.  modes: 2 bits per operand, output at bit 2*N.
// STRAIGHT: every operand is contiguous along the inner dim and read once (`modes` says so for all of them): the
// loads one after the other, no tests of an operand's mode in between.  A kernel of its own, for the functors
// that have it (straight_rows_enabled): as a branch of the general kernel it made that kernel's other calls slower
// (a matrix plus a row 80 -> 75 % of the HBM rate).
template <bool STRAIGHT, class Fn, class Out, class... Ins, size_t... I>
DPX_D void ew_rows_body(const Fn &fn, const NdIndex<sizeof...(Ins) + 1> &ix, Out *out,
                        const InPtrs<sizeof...(Ins)> &in, uint32_t modes, int tx_log2,
                        int64_t nrows, int64_t col_blocks, std::index_sequence<I...>)
{
    constexpr int N = sizeof...(Ins);
    constexpr int E = ew_traits<Out, Ins...>::E;
    const int tx = threadIdx.x & ((1 << tx_log2) - 1);
    const int ty = threadIdx.x >> tx_log2;
    // blockIdx.x < 2^31 and col_blocks <= gridDim.x: 32-bit division
    const uint32_t rb = blockIdx.x / (uint32_t)col_blocks;
    const uint32_t cb = blockIdx.x - rb * (uint32_t)col_blocks;
    const int64_t row = (int64_t)rb * ((int)blockDim.x >> tx_log2) + ty;
    const int inner = ix.nd - 1;
    const int64_t ncols = ix.shape[inner];
    const int64_t col0 = (((int64_t)cb << tx_log2) + tx) * E;
    // (STRAIGHT: the packs are moved back by up to E - 1 columns, below, and the host counts a thread more per row)
    if (row >= nrows || col0 >= ncols + (STRAIGHT ? E - 1 : 0)) return;

    int64_t off[N + 1];
#pragma unroll
    for (int k = 0; k <= N; ++k) off[k] = col0 * ix.strides[k][inner];
    if (nrows <= 0x7fffffff) { // the usual case: 32-bit div/mod chain
        uint32_t r = (uint32_t)row;
        for (int d = inner - 1; d >= 0; --d) {
            const uint32_t q = (d == 0) ? 0u : r / (uint32_t)ix.shape[d];
            const int64_t i = r - q * (uint32_t)ix.shape[d];
#pragma unroll
            for (int k = 0; k <= N; ++k) off[k] += i * ix.strides[k][d];
            r = q;
        }
    }
    else {
        int64_t r = row;
        for (int d = inner - 1; d >= 0; --d) {
            const int64_t q = (d == 0) ? 0 : r / ix.shape[d];
            const int64_t i = r - q * ix.shape[d];
#pragma unroll
            for (int k = 0; k <= N; ++k) off[k] += i * ix.strides[k][d];
            r = q;
        }
    }
    const int cnt = (ncols - col0 < E) ? (int)(ncols - col0) : E;
    // the 64 lanes of this wave lie in one row and every one of them has a full pack that is
    // not the last of the row
    const bool wave_full = tx_log2 >= 6 && col0 - (int64_t)(threadIdx.x & 63) * E + 64 * E < ncols;
    if constexpr (STRAIGHT) {
        // (fp32 A[:, :h] + A[:, h:] and A[::2] + B[::2] over 16384 x 16384: 73 -> 77-79 % of the HBM rate)
        // The packs of a row are laid so that the stores are aligned: a row of the output that starts m elements
        // past a pack boundary (rows of A[1:-1, 1:-1], rows of odd length) has its packs moved back by m columns;
        // the first thread of the row then holds E - m elements, the last what is left.
        const int m = (int)(((uintptr_t)(out + off[N] - col0) / sizeof(Out)) & (uintptr_t)(E - 1));
        const int64_t c = col0 - m;
        const int64_t first = c < 0 ? 0 : c, last = (c + E < ncols) ? c + E : ncols;
        if (last <= first) return;
        const int64_t shift = first - col0;
        if (last - first == E) {
            std::tuple<pack<Ins, E>...> x;
            ((std::get<I>(x) = load_pack<Ins, E>((const Ins *)in.p[I] + off[I] + shift)), ...);
            (keep_whole(std::get<I>(x)), ...);
            pack<Out, E> r;
#pragma unroll
            for (int e = 0; e < E; ++e) r.v[e] = to_storage<Out>(fn(to_value(std::get<I>(x).v[e])...));
            store_pack<Out, E>(out + off[N] + shift, r);
        }
        else {
            for (int64_t e = shift; e < last - col0; ++e)
                out[off[N] + e] = to_storage<Out>(fn(to_value(load_one((const Ins *)in.p[I] + off[I] + e))...));
        }
        return;
    }
    std::tuple<pack<Ins, E>...> v;
    auto load_operand = [&](auto *p, int64_t o, int64_t st, uint32_t mode, bool keep) {
        using T = std::remove_cv_t<std::remove_pointer_t<decltype(p)>>;
        pack<T, E> r;
        if (mode == MODE_VEC && cnt == E) {
            // an operand that is re-read along a broadcast dim stays in cache
            r = keep ? load_pack<T, E, false>(p + o) : load_pack<T, E>(p + o);
        }
        else if (mode == MODE_BCAST) {
            r = splat<T, E>(load_one(p + o));
        }
        else if (mode == MODE_VEC2 && cnt == E && col0 + E < ncols) {
            // stride 2 (x[:, ::2], real/imag parts): two contiguous 16-byte loads, keep every
            // other element.  The loads reach one element past the last one used, which lies
            // inside the view for every pack but the last of a row (that one goes scalar).
            if constexpr (E >= 2) {
                bool done = false;
                if constexpr (sizeof(T) * E == 16) {
                    if (wave_full) {
                        r = load_stride2_wave<T, E>(p + o);
                        done = true;
                    }
                }
                if (!done) {
                    const pack<T, E> lo = load_pack<T, E>(p + o), hi = load_pack<T, E>(p + o + E);
#pragma unroll
                    for (int e = 0; e < E; ++e) r.v[e] = (2 * e < E) ? lo.v[(2 * e) % E] : hi.v[(2 * e) % E];
                }
            }
        }
        else {
#pragma unroll
            for (int e = 0; e < E; ++e) r.v[e] = load_one(p + o + ((e < cnt) ? e : 0) * st);
        }
        return r;
    };
    ((std::get<I>(v) = load_operand((const Ins *)in.p[I], off[I], ix.strides[I][inner],
                                    (modes >> (2 * I)) & 3u, (modes >> (MODE_KEEP_SHIFT + I)) & 1u)),
     ...);
    (keep_whole(std::get<I>(v)), ...);
    pack<Out, E> r;
#pragma unroll
    for (int e = 0; e < E; ++e) r.v[e] = to_storage<Out>(fn(to_value(std::get<I>(v).v[e])...));
    if (((modes >> (2 * N)) & 3u) == MODE_VEC && cnt == E) {
        store_pack<Out, E>(out + off[N], r);
    }
    else {
        const int64_t st = ix.strides[N][inner];
#pragma unroll
        for (int e = 0; e < E; ++e)
            if (e < cnt) out[off[N] + e * st] = r.v[e];
    }
}

template <class Fn, class Out, class... Ins>
__global__ __launch_bounds__(EW_BLOCK) void ew_rows_kernel(Fn fn,
                                                          NdIndex<sizeof...(Ins) + 1> ix,
                                                          Out *out, InPtrs<sizeof...(Ins)> in,
                                                          uint32_t modes, int tx_log2,
                                                          int64_t nrows, int64_t col_blocks)
{
    ew_rows_body<false, Fn, Out, Ins...>(fn, ix, out, in, modes, tx_log2, nrows, col_blocks,
                                         std::index_sequence_for<Ins...>{});
}
template <class Fn, class Out, class... Ins>
__global__ __launch_bounds__(EW_BLOCK) void ew_rows_straight_kernel(Fn fn, NdIndex<sizeof...(Ins) + 1> ix, Out *out,
                                                                   InPtrs<sizeof...(Ins)> in, int tx_log2, int64_t nrows,
                                                                   int64_t col_blocks)
{
    ew_rows_body<true, Fn, Out, Ins...>(fn, ix, out, in, 0u, tx_log2, nrows, col_blocks,
                                        std::index_sequence_for<Ins...>{});
}
// functors that have it (one more kernel per functor and element type)
template <class Fn> struct straight_rows_enabled : std::false_type {};

// ---- calls that only write: an outer sum, a row plus a column --------------------------------
// Every input is either a row vector (contiguous along the inner dim, the same for all rows of dim inner - 1) or
// one value per row (it does not move along the inner dim; `per_row` has its bit).  A block owns up to
// EW_OUTER_ROWS consecutive rows of dim inner - 1 under one index of the dims before it and blockDim.x * E columns:
// a thread loads its pack of every row vector once, lane l of each wave the per-row values of row l, and then a
// row is a lane read (v_readlane), the arithmetic and one 16-byte store.  The rows kernel above spends its index
// arithmetic and a load of every operand on each pack of output (fp32 row + column into 16384 x 16384: 63 % of
// the HBM rate where a fill of the same matrix writes at 84 %).  Few rows per block: a thread that stores one
// row after the other writes slower the longer it goes on (a stand-alone kernel of 256 threads storing 4 KiB runs
// of 2 / 4 / 8 / 16 / 64 rows of 64 KiB: 84 / 82 / 82 / 78 / 55 % of the HBM rate; where the rows are no longer than
// the runs, so that a block's rows lie end to end, 2 / 8 rows: 75 / 67 %; rows dealt to the blocks in turn instead
// of in runs: 60 %).  Two rows per block for such short rows help where the row vector is one for the whole call
// (67 -> 74 %) and cost more than that where every block has to fetch its own (68 -> 49 %), so 8 it is.
constexpr int EW_OUTER_ROWS = 8;
template <class T> DPX_D T lane_value(T v, int lane) // v of lane `lane` (uniform), for every lane
{
    constexpr int W = (sizeof(T) + 3) / 4;
    union {
        T t;
        uint32_t w[W];
    } a, b;
#pragma unroll
    for (int i = 0; i < W; ++i) a.w[i] = 0;
    a.t = v;
#pragma unroll
    for (int i = 0; i < W; ++i) b.w[i] = (uint32_t)__builtin_amdgcn_readlane((int)a.w[i], lane);
    return b.t;
}
template <class Fn, class Out, class... Ins, size_t... I>
DPX_D void ew_outer_body(const Fn &fn, const NdIndex<sizeof...(Ins) + 1> &ix, Out *out,
                         const InPtrs<sizeof...(Ins)> &in, uint32_t per_row, uint32_t mid_blocks, uint32_t col_blocks,
                         std::index_sequence<I...>)
{
    constexpr int N = sizeof...(Ins);
    constexpr int E = ew_traits<Out, Ins...>::E;
    const int inner = ix.nd - 1, mid = inner - 1;
    const int64_t ncols = ix.shape[inner];
    uint32_t b = blockIdx.x;
    const uint32_t cb = b % col_blocks;
    b /= col_blocks;
    const uint32_t mb = b % mid_blocks;
    uint32_t o = b / mid_blocks; // index over the dims before `mid`
    const int64_t row0 = (int64_t)mb * EW_OUTER_ROWS;
    const int nr = (ix.shape[mid] - row0 < EW_OUTER_ROWS) ? (int)(ix.shape[mid] - row0) : EW_OUTER_ROWS;
    int64_t base[N + 1];
#pragma unroll
    for (int k = 0; k <= N; ++k) base[k] = 0;
    for (int d = mid - 1; d >= 0; --d) {
        const uint32_t q = (d == 0) ? 0u : o / (uint32_t)ix.shape[d];
        const int64_t i = o - q * (uint32_t)ix.shape[d];
#pragma unroll
        for (int k = 0; k <= N; ++k) base[k] += i * ix.strides[k][d];
        o = q;
    }
    const int lane = threadIdx.x & 63;
    const int64_t col0 = ((int64_t)cb * blockDim.x + threadIdx.x) * E;
    const bool active = col0 < ncols;
    const int cnt = (ncols - col0 < E) ? (int)(ncols - col0) : E;
    // the per-row values of row `lane` (every lane of the wave takes part, also those past the row's end) ...
    std::tuple<Ins...> mine;
    auto load_row_value = [&](auto *p, int64_t bk, int64_t sm, bool is_per_row) {
        using T = std::remove_cv_t<std::remove_pointer_t<decltype(p)>>;
        T v{};
        if (is_per_row && lane < nr) v = load_one(p + bk + (row0 + lane) * sm);
        return v;
    };
    ((std::get<I>(mine) = load_row_value((const Ins *)in.p[I], base[I], ix.strides[I][mid], (per_row >> I) & 1u)), ...);
    // ... and this thread's pack of the row vectors: one for all rows, or one per row where the vector moves along
    // dim inner - 1 (it is then the same for every index of an earlier dim: X[:, None, :] - Y[None, :, :])
    constexpr int R = EW_OUTER_ROWS;
    std::tuple<std::array<pack<Ins, E>, R>...> vec;
    auto load_vectors = [&](auto &dstv, auto *p, int64_t bk, int64_t sm, bool is_per_row) {
        using T = std::remove_cv_t<std::remove_pointer_t<decltype(p)>>;
#pragma unroll
        for (int j = 0; j < R; ++j) {
            dstv[j] = pack<T, E>{};
            if (is_per_row || !active || j >= nr || (j > 0 && sm == 0)) continue;
            const T *src = p + bk + (row0 + j) * sm + col0;
            if (cnt == E) dstv[j] = load_pack<T, E, false>(src);
            else {
#pragma unroll
                for (int e = 0; e < E; ++e) dstv[j].v[e] = load_one(src + (e < cnt ? e : 0));
            }
        }
    };
    (load_vectors(std::get<I>(vec), (const Ins *)in.p[I], base[I], ix.strides[I][mid], (per_row >> I) & 1u), ...);
    Out *q = out + base[N] + row0 * ix.strides[N][mid] + col0;
    const int64_t ostep = ix.strides[N][mid];
#pragma unroll
    for (int j = 0; j < R; ++j) {
        if (j >= nr) break;
        std::tuple<pack<Ins, E>...> x;
        ((std::get<I>(x) = ((per_row >> I) & 1u) ? splat<Ins, E>(lane_value(std::get<I>(mine), j))
                                                 : std::get<I>(vec)[ix.strides[I][mid] == 0 ? 0 : j]),
         ...);
        pack<Out, E> r;
#pragma unroll
        for (int e = 0; e < E; ++e) r.v[e] = to_storage<Out>(fn(to_value(std::get<I>(x).v[e])...));
        if (active) {
            if (cnt == E) store_pack<Out, E>(q + j * ostep, r);
            else {
                // (places by constant index: indexed by a running one the pack is kept in LDS, full packs included)
#pragma unroll
                for (int e = 0; e < E; ++e)
                    if (e < cnt) q[j * ostep + e] = r.v[e];
            }
        }
    }
}
template <class Fn, class Out, class... Ins>
__global__ __launch_bounds__(EW_BLOCK) void ew_outer_kernel(Fn fn, NdIndex<sizeof...(Ins) + 1> ix, Out *out,
                                                           InPtrs<sizeof...(Ins)> in, uint32_t per_row,
                                                           uint32_t mid_blocks, uint32_t col_blocks)
{
    ew_outer_body<Fn, Out, Ins...>(fn, ix, out, in, per_row, mid_blocks, col_blocks, std::index_sequence_for<Ins...>{});
}
// functors whose calls may take it (two-operand functions: one more kernel per functor and element type)
template <class Fn> struct outer_enabled : std::false_type {};

// ---- two rows per thread, the way each input is read fixed at compile time --------------------
// The kernel for calls with a stride-2 input (x[:, ::2], the real or imaginary parts of a complex
// array) whose rows are whole waves of packs: A[:, ::2] * row, exp(A[:, ::2]), where(mask, A[:, ::2], row),
// I[:, ::2] & J[:, ::2].  Such a call moves twice the bytes through the vector memory pipeline that
// it uses (every 64-byte line of the base array is fetched for half of its elements), and at one
// row per thread the loads of a row operand cost as much of that pipeline as the output does: on
// MI355X the pipeline, not HBM, then bounds the kernel (fp32 A[:, ::2] * row, 8192 x 4096 outputs:
// 73.6 us at one row per thread, 61.3 us at two with the row operand loaded once; HBM time of the
// 403 MB it moves: 50 us).  The rows kernel above decides how to read each operand at run time,
// and the branches that takes between its loads keep the compiler from issuing them together, so
// here the reading is part of the kernel's type:
//   PAT, 2 bits per input: RC_ROWS  contiguous along the inner dim, moves with the rows: one
//                                   16-byte (or narrower) pack per row;
//                          RC_S2    stride 2 along the inner dim: wave-interleaved loads, see
//                                   stride2_wave_issue;
//                          RC_ONCE  does not move along dim inner - 1 (a row vector, or a scalar
//                                   when it does not move along the inner dim either: bit k of
//                                   `scalar`): loaded once for both rows.
// A thread owns E consecutive outputs of two neighbouring rows (dim inner - 1, extent even); every
// wave lies inside one row and has 64 full packs (the host checks ncols % (64 E) == 0); the output
// is contiguous along the inner dim.  Wave-interleaved loads read one element past the last one a
// wave uses: the wave that ends the last row of the iteration space reads element by element instead.
enum : int { RC_ROWS = 0, RC_S2 = 1, RC_ONCE = 2 };
template <class T> using raw_pair_t = std::pair<u32x4, u32x4>; // the two loads of a stride-2 input
constexpr int rc_of(int pat, int k) { return (pat >> (2 * k)) & 3; }

template <int PAT, class Fn, class Out, class... Ins, size_t... I>
DPX_D void ew_rows2_body(const Fn &fn, const NdIndex<sizeof...(Ins) + 1> &ix, Out *out,
                         const InPtrs<sizeof...(Ins)> &in, uint32_t scalar, uint32_t waves_per_row,
                         int64_t npairs, std::index_sequence<I...>)
{
    constexpr int N = sizeof...(Ins);
    constexpr int E = ew_traits<Out, Ins...>::E;
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * ((int)blockDim.x >> 6) + (threadIdx.x >> 6);
    const int64_t pair = wave / waves_per_row; // (uniform over the wave)
    if (pair >= npairs) return;
    const uint32_t cw = (uint32_t)(wave - pair * waves_per_row);
    const int inner = ix.nd - 1;
    const int64_t col0 = ((int64_t)cw * 64 + lane) * E;
    int64_t off[N + 1];
#pragma unroll
    for (int k = 0; k <= N; ++k) off[k] = col0 * ix.strides[k][inner];
    {
        int64_t r = pair * 2;
        for (int d = inner - 1; d >= 0; --d) {
            const int64_t q = (d == 0) ? 0 : r / ix.shape[d];
            const int64_t i = r - q * ix.shape[d];
#pragma unroll
            for (int k = 0; k <= N; ++k) off[k] += i * ix.strides[k][d];
            r = q;
        }
    }
    int64_t rstep[N + 1];
#pragma unroll
    for (int k = 0; k <= N; ++k) rstep[k] = ix.strides[k][inner - 1];

    if (pair == npairs - 1 && cw == waves_per_row - 1) {
        // the wave that ends the last row: no read past its last element
        for (int j = 0; j < 2; ++j)
            for (int e = 0; e < E; ++e)
                out[off[N] + j * rstep[N] + e] = to_storage<Out>(fn(to_value(
                    load_one((const Ins *)in.p[I] + off[I] + j * rstep[I] + e * ix.strides[I][inner]))...));
        return;
    }
    // every load of the thread, then the results
    std::tuple<pack<Ins, E>...> v0, v1;    // RC_ROWS, and RC_ONCE in v0
    std::tuple<raw_pair_t<Ins>...> w0, w1; // RC_S2 (the tuple has an entry per input; unused ones vanish)
    auto issue_rows = [&](auto &v, auto &w, auto *p, int64_t o, int rc) {
        using T = std::remove_cv_t<std::remove_pointer_t<decltype(p)>>;
        if (rc == RC_ROWS) v = load_pack<T, E>(p + o);
        else if (rc == RC_S2) {
            if constexpr (E >= 2 && sizeof(T) * E == 16) stride2_wave_issue<T, E>(p + o, w.first, w.second);
        }
    };
    (issue_rows(std::get<I>(v0), std::get<I>(w0), (const Ins *)in.p[I], off[I], rc_of(PAT, (int)I)), ...);
    (issue_rows(std::get<I>(v1), std::get<I>(w1), (const Ins *)in.p[I], off[I] + rstep[I], rc_of(PAT, (int)I)), ...);
    auto issue_once = [&](auto &v, auto *p, int64_t o, int rc, bool is_scalar) {
        using T = std::remove_cv_t<std::remove_pointer_t<decltype(p)>>;
        if (rc == RC_ONCE) v = is_scalar ? splat<T, E>(load_one(p + o)) : load_pack<T, E, false>(p + o);
    };
    (issue_once(std::get<I>(v0), (const Ins *)in.p[I], off[I], rc_of(PAT, (int)I), (scalar >> I) & 1u), ...);
    auto value = [&](auto &v_first, auto &v_this, auto &w, auto *p, int rc) {
        using T = std::remove_cv_t<std::remove_pointer_t<decltype(p)>>;
        if constexpr (E >= 2 && sizeof(T) * E == 16) {
            if (rc == RC_S2) return stride2_wave_regroup<T, E>(w.first, w.second);
        }
        return rc == RC_ONCE ? v_first : v_this;
    };
    auto produce = [&](std::tuple<pack<Ins, E>...> &v, std::tuple<raw_pair_t<Ins>...> &w, int64_t o) {
        std::tuple<pack<Ins, E>...> x;
        ((std::get<I>(x) = value(std::get<I>(v0), std::get<I>(v), std::get<I>(w), (const Ins *)in.p[I],
                                 rc_of(PAT, (int)I))),
         ...);
        (keep_whole(std::get<I>(x)), ...);
        pack<Out, E> r;
#pragma unroll
        for (int e = 0; e < E; ++e) r.v[e] = to_storage<Out>(fn(to_value(std::get<I>(x).v[e])...));
        store_pack<Out, E>(out + o, r);
    };
    produce(v0, w0, off[N]);
    produce(v1, w1, off[N] + rstep[N]);
}

template <int PAT, class Fn, class Out, class... Ins>
__global__ __launch_bounds__(EW_BLOCK) void ew_rows2_kernel(Fn fn, NdIndex<sizeof...(Ins) + 1> ix, Out *out,
                                                           InPtrs<sizeof...(Ins)> in, uint32_t scalar,
                                                           uint32_t waves_per_row, int64_t npairs)
{
    ew_rows2_body<PAT, Fn, Out, Ins...>(fn, ix, out, in, scalar, waves_per_row, npairs,
                                        std::index_sequence_for<Ins...>{});
}

// Functors whose calls may take ew_rows2_kernel (each pattern is one more kernel per functor and
// element type, so the list is short): specialised next to the functors' definitions.
template <class Fn> struct rows2_enabled : std::false_type {};
// the patterns instantiated for N inputs
template <int N> struct rows2_patterns {
    using seq = std::integer_sequence<int>;
};
template <> struct rows2_patterns<1> {
    using seq = std::integer_sequence<int, RC_S2>;
};
template <> struct rows2_patterns<2> {
    using seq = std::integer_sequence<int, RC_S2 | RC_S2 << 2, RC_S2 | RC_ONCE << 2, RC_ONCE | RC_S2 << 2>;
};
template <> struct rows2_patterns<3> { // where(mask, x[:, ::2], row); where(x[:, ::2] > scalar, x[:, ::2], row) fused
    using seq = std::integer_sequence<int, RC_ROWS | RC_S2 << 2 | RC_ONCE << 4, RC_S2 | RC_ONCE << 2 | RC_ONCE << 4>;
};
template <class F, int... P> inline void for_each_pattern(F &&f, std::integer_sequence<int, P...>)
{
    (f(std::integral_constant<int, P>{}), ...);
}

// ---- transposing through an LDS tile ------------------------------------------------------
// For calls where the output is contiguous along the inner dim but some inputs are
// contiguous along another dim `dT` (op(A.T, out=C), op(A.T, B), ...).  A block owns a
// TI x TJ tile of the (dT, inner) plane, TI = 64 and TJ * widest itemsize = 512 bytes.
// Phase 1: inputs flagged in `tmask` are read with 16-byte accesses running along dT (256 to
// 1024 contiguous bytes per tile row) and copied to LDS as [inner][dT] with an odd row pitch.
// Phase 2: every thread produces 16-byte packs of the output with threads side by side
// along the inner dim (512 contiguous bytes per tile row), gathering the transposed inputs
// from LDS element by element and reading the other inputs in place.  Remaining dims are
// batch dims decoded from the block index.  Measured on MI355X for exp(A.T) -> C-contiguous,
// 8192 x 8192 floats: 5.8 TB/s; 64 x 64 tiles with 4-byte accesses 4.2 TB/s.
// modes: as for the rows kernel; for a flagged input MODE_VEC allows the 16-byte phase-1 reads.
constexpr int EW_TILE_BLOCK = 512;
constexpr size_t EW_TILE_LDS_MAX = 160 * 1024;
// positions along dT per tile: 128 (512-byte runs of 4-byte elements; measured best for 2-, 4- and 8-byte
// elements), 64 for 16-byte elements (1 KiB runs already)
constexpr int ew_tile_ti(int widest_itemsize) { return widest_itemsize <= 8 ? 128 : 64; }
template <class Out, class... Ins> struct tile_traits {
    static constexpr int TI = ew_tile_ti(max_sizeof<Out, Ins...>());
    static constexpr int TJ = 512 / max_sizeof<Out, Ins...>();
    template <class T> static constexpr int pitch() { return TI + (sizeof(T) >= 4 ? 1 : 4 / (int)sizeof(T)); }
    template <class T> static constexpr size_t bytes() { return ((size_t)TJ * pitch<T>() * sizeof(T) + 15) & ~(size_t)15; }
    // LDS of a launch: one tile per staged input
    static size_t lds_bytes(uint32_t tmask)
    {
        const size_t each[sizeof...(Ins) + 1] = {bytes<Ins>()..., 0};
        size_t acc = 0;
        for (size_t k = 0; k < sizeof...(Ins); ++k)
            if ((tmask >> k) & 1u) acc += each[k];
        return acc;
    }
};

template <class Fn, class Out, class... Ins, size_t... I>
DPX_D void ew_tile_body(const Fn &fn, const NdIndex<sizeof...(Ins) + 1> &ix, Out *out,
                        const InPtrs<sizeof...(Ins)> &in, uint32_t tmask, uint32_t modes, int dT, int64_t tiles_t,
                        int64_t tiles_i, unsigned char *smem, std::index_sequence<I...>)
{
    using TT = tile_traits<Out, Ins...>;
    constexpr int N = sizeof...(Ins);
    constexpr int E = ew_traits<Out, Ins...>::E;
    constexpr int TI = TT::TI, TJ = TT::TJ;
    const int inner = ix.nd - 1;
    // the grid has fewer than 2^32 blocks, so every quotient below fits 32 bits (64-bit
    // division is a long routine on this hardware)
    uint32_t b = blockIdx.x;
    const uint32_t nti = (uint32_t)tiles_i, ntt = (uint32_t)tiles_t;
    const uint32_t ti = b % nti;
    b /= nti;
    // diagonal order: consecutive blocks step along both tile axes, so neither the reads
    // (strided along `inner`) nor the writes (strided along dT) of the blocks in flight pile
    // up on the memory channels one power-of-two stride selects
    uint32_t tt = b % ntt + ti % ntt;
    tt = tt >= ntt ? tt - ntt : tt;
    b /= ntt;
    int64_t off[N + 1];
#pragma unroll
    for (int k = 0; k <= N; ++k) off[k] = 0;
    for (int d = inner - 1; d >= 0 && b != 0; --d) {
        if (d == dT) continue;
        const uint32_t extent = ix.shape[d] > 0xffffffffll ? 0xffffffffu : (uint32_t)ix.shape[d];
        const uint32_t q = b / extent;
        const uint32_t i = b - q * extent;
#pragma unroll
        for (int k = 0; k <= N; ++k) off[k] += (int64_t)i * ix.strides[k][d];
        b = q;
    }
    const int64_t i0 = (int64_t)tt * TI, j0 = (int64_t)ti * TJ;
    const int64_t ni = ix.shape[dT], nj = ix.shape[inner];
    // rows / columns of this tile that exist
    const int ci = (ni - i0 < TI) ? (int)(ni - i0) : TI;
    const int cj = (nj - j0 < TJ) ? (int)(nj - j0) : TJ;
    size_t lds_off[N + 1];
    {
        size_t acc = 0;
        ((lds_off[I] = acc, acc += ((tmask >> I) & 1u) ? TT::template bytes<Ins>() : 0), ...);
        lds_off[N] = acc;
    }
    const bool full = ci == TI && cj == TJ;
    // phase 1: transposed inputs -> LDS, threads adjacent along dT
    auto stage = [&](auto *p, int k, size_t l_off) {
        using T = std::remove_cv_t<std::remove_pointer_t<decltype(p)>>;
        if (!((tmask >> k) & 1u)) return;
        constexpr int S = TT::template pitch<T>();
        constexpr int VE = 16 / (int)sizeof(T);      // elements per 16-byte access
        constexpr int VPR = TI / VE;                 // accesses per tile row
        constexpr int RPP = EW_TILE_BLOCK / VPR;          // tile rows per pass
        constexpr int PASSES = (TJ + RPP - 1) / RPP;
        T *tile = reinterpret_cast<T *>(smem + l_off);
        const int64_t sj = ix.strides[k][inner];
        const T *base = p + off[k] + i0 + j0 * sj;
        if (((modes >> (2 * k)) & 3u) == MODE_VEC) {
            const int lv = threadIdx.x % VPR, lr = threadIdx.x / VPR;
            const bool col_ok = lv * VE < ci;
            const bool whole = lv * VE + VE <= ci; // else: the pack that holds the end of dim dT
            pack<T, VE> m[PASSES];
            if (TJ % RPP == 0 && full) {
                // a whole tile, covered by whole passes: nothing to check, all loads in flight before
                // the first LDS write
#pragma unroll
                for (int q = 0; q < PASSES; ++q) m[q] = load_pack<T, VE>(base + (q * RPP + lr) * sj + lv * VE);
#pragma unroll
                for (int q = 0; q < PASSES; ++q)
#pragma unroll
                    for (int e = 0; e < VE; ++e) tile[(q * RPP + lr) * S + lv * VE + e] = m[q].v[e];
                return;
            }
#pragma unroll
            for (int q = 0; q < PASSES; ++q) {
                const int r = q * RPP + lr;
                if (col_ok && r < cj) {
                    const T *src = base + r * sj + lv * VE;
                    if (whole) m[q] = load_pack<T, VE>(src);
                    else {
#pragma unroll
                        for (int e = 0; e < VE; ++e) m[q].v[e] = load_one(src + ((lv * VE + e < ci) ? e : 0));
                    }
                }
            }
#pragma unroll
            for (int q = 0; q < PASSES; ++q) {
                const int r = q * RPP + lr;
                if (col_ok && r < cj) {
#pragma unroll
                    for (int e = 0; e < VE; ++e) tile[r * S + lv * VE + e] = m[q].v[e];
                }
            }
        }
        else {
            const int lo = threadIdx.x % TI, hi = threadIdx.x / TI;
            if (lo < ci)
                for (int r = hi; r < cj; r += EW_TILE_BLOCK / TI) tile[r * S + lo] = load_one(base + r * sj + lo);
        }
    };
    (stage((const Ins *)in.p[I], (int)I, lds_off[I]), ...);
    __syncthreads();
    // phase 2: compute, threads adjacent along the inner dim
    constexpr int CPR = TJ / E;         // packs per tile row (32)
    constexpr int RPP2 = EW_TILE_BLOCK / CPR; // tile rows per pass (16)
    const int lc = threadIdx.x % CPR, lr = threadIdx.x / CPR;
    const int jj = lc * E;
    if (jj >= cj) return;
    const int cnt = (cj - jj < E) ? (cj - jj) : E;
    int64_t col[N + 1];
#pragma unroll
    for (int k = 0; k <= N; ++k) col[k] = off[k] + (j0 + jj) * ix.strides[k][inner] + i0 * ix.strides[k][dT];
    auto fetch = [&](auto *p, int k, size_t l_off, int i) {
        using T = std::remove_cv_t<std::remove_pointer_t<decltype(p)>>;
        pack<T, E> r;
        if ((tmask >> k) & 1u) {
            constexpr int S = TT::template pitch<T>();
            const T *tile = reinterpret_cast<const T *>(smem + l_off);
#pragma unroll
            for (int e = 0; e < E; ++e) r.v[e] = tile[(jj + e) * S + i];
            return r;
        }
        const uint32_t mode = (modes >> (2 * k)) & 3u;
        const T *q = p + col[k] + i * ix.strides[k][dT];
        if (mode == MODE_VEC && cnt == E)
            return ((modes >> (MODE_KEEP_SHIFT + k)) & 1u) ? load_pack<T, E, false>(q) : load_pack<T, E>(q);
        if (mode == MODE_BCAST) return splat<T, E>(load_one(q));
        const int64_t st = ix.strides[k][inner];
#pragma unroll
        for (int e = 0; e < E; ++e) r.v[e] = load_one(q + ((e < cnt) ? e : 0) * st);
        return r;
    };
    const bool out_vec = ((modes >> (2 * N)) & 3u) == MODE_VEC && cnt == E;
    if (full && out_vec && tmask == (1u << N) - 1u) {
        // a whole tile with every input in LDS (exp(A.T), A.T + B.T): no case to tell apart per
        // row, so the rows are unrolled and the LDS reads of one row overlap the arithmetic of
        // the row before
        static_assert(TI % RPP2 == 0, "passes cover the tile exactly");
        Out *q = out + col[N] + lr * ix.strides[N][dT];
        const int64_t qstep = RPP2 * ix.strides[N][dT];
#pragma unroll 2
        for (int it = 0; it < TI / RPP2; ++it) {
            const int i = it * RPP2 + lr;
            std::tuple<pack<Ins, E>...> v;
            auto gather = [&](auto &dstp, size_t l_off) {
                using T = std::remove_cv_t<std::remove_reference_t<decltype(dstp.v[0])>>;
                constexpr int S = TT::template pitch<T>();
                const T *tile = reinterpret_cast<const T *>(smem + l_off);
#pragma unroll
                for (int e = 0; e < E; ++e) dstp.v[e] = tile[(jj + e) * S + i];
            };
            (gather(std::get<I>(v), lds_off[I]), ...);
            pack<Out, E> r;
#pragma unroll
            for (int e = 0; e < E; ++e) r.v[e] = to_storage<Out>(fn(to_value(std::get<I>(v).v[e])...));
            store_pack<Out, E>(q, r);
            q += qstep;
        }
        return;
    }
#pragma unroll 2
    for (int i = lr; i < ci; i += RPP2) {
        std::tuple<pack<Ins, E>...> v;
        ((std::get<I>(v) = fetch((const Ins *)in.p[I], (int)I, lds_off[I], i)), ...);
        pack<Out, E> r;
#pragma unroll
        for (int e = 0; e < E; ++e) r.v[e] = to_storage<Out>(fn(to_value(std::get<I>(v).v[e])...));
        Out *q = out + col[N] + i * ix.strides[N][dT];
        if (out_vec) store_pack<Out, E>(q, r);
        else {
#pragma unroll
            for (int e = 0; e < E; ++e)
                if (e < cnt) q[e] = r.v[e];
        }
    }
}

template <class Fn, class Out, class... Ins>
__global__ __launch_bounds__(EW_TILE_BLOCK) void ew_tile_kernel(Fn fn, NdIndex<sizeof...(Ins) + 1> ix, Out *out,
                                                          InPtrs<sizeof...(Ins)> in, uint32_t tmask, uint32_t modes,
                                                          int dT, int64_t tiles_t, int64_t tiles_i)
{
    extern __shared__ __align__(16) unsigned char ew_tile_smem[];
    ew_tile_body<Fn, Out, Ins...>(fn, ix, out, in, tmask, modes, dT, tiles_t, tiles_i, ew_tile_smem,
                                  std::index_sequence_for<Ins...>{});
}

// ---- host-side plan (element-type independent) ----------------------------------
struct EwPlan {
    int path; // dpx_path
    int nops; // inputs + 1
    int nd;
    int64_t shape[DPX_MAX_ND];
    int64_t strides[5][DPX_MAX_ND]; // inputs..., output (index nops-1)
    int64_t offsets[5];             // element displacement per operand
    int64_t n;                      // total elements
    // launch parameters, filled by ew_finish_plan for a given E / item sizes
    bool vec;
    bool flat2d;     // contiguous path over a row-major matrix with short rows (nd == 2 kept in shape/strides)
    uint32_t bcast;  // contiguous path: 2 bits per input (BC_*)
    uint32_t period; // ... row length for BC_PERIODIC / BC_REPEAT inputs
    uint32_t modes;
    int tx_log2;
    int block; // threads per block
    int64_t nrows, col_blocks, grid;
    // ew_rows2_kernel (pattern >= 0): the way each input is read, inputs that are scalars along the
    // inner dim, waves per row, row pairs
    int rows2_pat;
    uint32_t rows2_scalar, rows2_waves;
    int rows2_wpb; // waves per block
    int64_t rows2_pairs;
    // ew_outer_kernel (outer != 0): inputs that are one value per row, blocks along dim inner - 1
    // (outer_fit: the call fits it, with the launch shape below; outer: the functor has it and it is taken)
    int outer, outer_fit, outer_block;
    uint32_t outer_per_row, outer_mid_blocks;
    int64_t outer_col_blocks, outer_grid;
    // tile path
    uint32_t tmask; // inputs staged through LDS
    int dT;         // the dim those inputs are contiguous along
    int64_t tiles_t, tiles_i;
};

// fills path/nd/shape/strides/offsets from (already validated) views
void ew_make_plan(EwPlan &pl, int nops, const dpx_array_view *const *views);
// fills the launch parameters for E elements per thread and the operands' item sizes
// and (displaced) base pointers
// (U: packs per thread of the contiguous kernel)
void ew_finish_plan(EwPlan &pl, int E, int U, const int *itemsize, const void *const *ptrs);

// dry != 0: only fill the launch parameters of pl
template <class Fn, class Out, class... Ins>
inline hipError_t ew_launch(const Fn &fn, EwPlan &pl, const dpx_array_view *const *views,
                            hipStream_t stream, bool dry = false)
{
    constexpr int N = sizeof...(Ins);
    constexpr int E = ew_traits<Out, Ins...>::E;
    const int sizes[N + 1] = {(int)sizeof(Ins)..., (int)sizeof(Out)};
    const void *ptrs[N + 1];
    for (int k = 0; k <= N; ++k)
        ptrs[k] = (const char *)views[k]->data + pl.offsets[k] * sizes[k];
    if constexpr (N >= 1) {
        if (pl.path == DPX_PATH_EW_TILE) {
            // a block's tiles must fit the CU's LDS: inputs beyond that are read in place
            for (int k = N - 1; k >= 0 && tile_traits<Out, Ins...>::lds_bytes(pl.tmask) > EW_TILE_LDS_MAX; --k)
                pl.tmask &= ~(1u << k);
            if (pl.tmask == 0) pl.path = DPX_PATH_EW_ROWS;
        }
    }
    ew_finish_plan(pl, E, ew_packs_per_thread<Fn, Out, Ins...>(), sizes, ptrs);
    if constexpr (rows2_enabled<Fn>::value && E >= 2 && E <= 4 && N >= 1 && N <= 3) {
        // a call that fits the two-rows kernel in a pattern this functor is instantiated for
        if (pl.path == DPX_PATH_EW_ROWS && pl.rows2_pat >= 0)
            for_each_pattern(
                [&](auto pat_c) {
                    if (pl.rows2_pat == decltype(pat_c)::value) pl.path = DPX_PATH_EW_ROWS2;
                },
                typename rows2_patterns<N>::seq{});
    }
    pl.outer = 0;
    if constexpr (outer_enabled<Fn>::value) {
        if (pl.path == DPX_PATH_EW_ROWS && pl.outer_fit) {
            pl.outer = 1;
            pl.block = pl.outer_block;
            pl.col_blocks = pl.outer_col_blocks;
            pl.grid = pl.outer_grid;
        }
    }
    if (pl.path == DPX_PATH_NOOP || dry) return hipSuccess;
    InPtrs<N> in;
    for (int k = 0; k < N; ++k) in.p[k] = ptrs[k];
    Out *out = (Out *)ptrs[N];
    if (pl.path == DPX_PATH_EW_CONTIG) {
        hipLaunchKernelGGL((ew_contig_kernel<Fn, Out, Ins...>), dim3((unsigned)pl.grid), dim3(pl.block), 0,
                           stream, fn, pl.n, pl.bcast, pl.period, out, in);
    }
    else {
        NdIndex<N + 1> ix;
        ix.nd = pl.nd;
        ix.pad = 0;
        for (int d = 0; d < DPX_MAX_ND; ++d) {
            ix.shape[d] = d < pl.nd ? pl.shape[d] : 1;
            for (int k = 0; k <= N; ++k) ix.strides[k][d] = d < pl.nd ? pl.strides[k][d] : 0;
        }
        if (pl.path == DPX_PATH_EW_TILE) {
            if constexpr (N >= 1) {
                using TT = tile_traits<Out, Ins...>;
                const size_t lds = TT::lds_bytes(pl.tmask);
                if (lds > 65536) {
                    // more dynamic LDS than a launch may ask for by default: raise the kernel's limit,
                    // once per device
                    static std::atomic<uint64_t> raised{0};
                    int dev = 0;
                    hipError_t e = hipGetDevice(&dev);
                    if (e != hipSuccess) return e;
                    const uint64_t bit = 1ull << (dev & 63);
                    if (!(raised.load(std::memory_order_acquire) & bit)) {
                        e = hipFuncSetAttribute((const void *)ew_tile_kernel<Fn, Out, Ins...>,
                                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)EW_TILE_LDS_MAX);
                        if (e != hipSuccess) return e;
                        raised.fetch_or(bit, std::memory_order_release);
                    }
                }
                hipLaunchKernelGGL((ew_tile_kernel<Fn, Out, Ins...>), dim3((unsigned)pl.grid), dim3(EW_TILE_BLOCK), lds,
                                   stream, fn, ix, out, in, pl.tmask, pl.modes, pl.dT, pl.tiles_t, pl.tiles_i);
            }
            return hipGetLastError();
        }
        if constexpr (rows2_enabled<Fn>::value && E >= 2 && E <= 4 && N >= 1 && N <= 3) {
            if (pl.path == DPX_PATH_EW_ROWS2) {
                // one wave per block, like the contiguous kernel: waves are independent here
                const int wpb = pl.rows2_wpb;
                const unsigned grid = (unsigned)((pl.rows2_pairs * pl.rows2_waves + wpb - 1) / wpb);
                for_each_pattern(
                    [&](auto pat_c) {
                        constexpr int PAT = decltype(pat_c)::value;
                        if (pl.rows2_pat == PAT)
                            hipLaunchKernelGGL((ew_rows2_kernel<PAT, Fn, Out, Ins...>), dim3(grid), dim3(64 * wpb), 0,
                                               stream, fn, ix, out, in, pl.rows2_scalar, pl.rows2_waves, pl.rows2_pairs);
                    },
                    typename rows2_patterns<N>::seq{});
                return hipGetLastError();
            }
        }
        if constexpr (outer_enabled<Fn>::value) {
            if (pl.outer) {
                hipLaunchKernelGGL((ew_outer_kernel<Fn, Out, Ins...>), dim3((unsigned)pl.grid), dim3(pl.block), 0, stream,
                                   fn, ix, out, in, pl.outer_per_row, pl.outer_mid_blocks, (uint32_t)pl.col_blocks);
                return hipGetLastError();
            }
        }
        if constexpr (straight_rows_enabled<Fn>::value) {
            constexpr uint32_t ALL_VEC = ((1u << (2 * (N + 1))) - 1u) / 3u; // MODE_VEC for each operand, no keep bit
            if (pl.modes == ALL_VEC) {
                hipLaunchKernelGGL((ew_rows_straight_kernel<Fn, Out, Ins...>), dim3((unsigned)pl.grid), dim3(pl.block), 0,
                                   stream, fn, ix, out, in, pl.tx_log2, pl.nrows, pl.col_blocks);
                return hipGetLastError();
            }
        }
        hipLaunchKernelGGL((ew_rows_kernel<Fn, Out, Ins...>), dim3((unsigned)pl.grid),
                           dim3(pl.block), 0, stream, fn, ix, out, in, pl.modes, pl.tx_log2,
                           pl.nrows, pl.col_blocks);
    }
    return hipGetLastError();
}

} // namespace dpx
