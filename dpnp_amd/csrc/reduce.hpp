// Reduction kernels: sum / prod / max / min (+ squared-deviation sum) and
// argmax / argmin over the trailing axes of a strided array.
//
// They replace the SequentialReduction / ReductionOverGroup* / SearchReduction
// functors and their multi-level launchers
// (libtensor/include/kernels/reductions.hpp:98-620,758-1856,1868-3308).
//
// MI355X layout:
//   * "rows": the reduced run is contiguous.  G = 1..64 lanes of a wave, a
//     256-thread or a 1024-thread block cooperate on one output; each lane reads
//     16-byte packs strided by G packs (coalesced), keeps U independent
//     accumulators, then a wave-64 shuffle tree and an LDS stage combine them.
//   * "cols": outputs are contiguous and the reduced run is strided (axis=0 of
//     a C-contiguous matrix).  Threads sit side by side along the output
//     dimension, so every load is a coalesced 16-byte pack of adjacent columns;
//     TY thread rows walk down the reduced axis and meet in LDS.
//   * when there are too few outputs to fill 256 CUs the reduced run is split
//     over several blocks; partials go to scratch and a second launch of the
//     same kernels folds them.  Partition and fold order are fixed functions of
//     the shapes: results are bit-reproducible run to run, no atomics anywhere.
#pragma once
#include "ops.hpp"
#include "types.hpp"

namespace dpx {

constexpr int RED_U = 4; // independent 16-byte loads in flight per thread

struct RedIndex {
    int32_t nd_i, nd_r;
    int64_t shape_i[DPX_MAX_ND];
    int64_t src_istr[DPX_MAX_ND];
    int64_t dst_str[DPX_MAX_ND];
    int64_t aux_str[DPX_MAX_ND];
    int64_t shape_r[DPX_MAX_ND];
    int64_t src_rstr[DPX_MAX_ND];
};

// launch parameters shared by the kernels
struct RedLaunch {
    int64_t m, n;     // outputs, reduced elements per output
    int64_t chunk;    // reduced elements per split
    int32_t splits;   // blocks cooperating on one output
    int32_t g_log2;   // rows: log2(lanes per output); cols: log2(threads along columns)
    int32_t vec;      // 16-byte packs allowed
    int32_t pad;
    int64_t rstride;  // cols: stride of the reduced axis
    int64_t inner;    // cols: length of the inner (contiguous) iteration dim
    int64_t col_blocks;
};

template <class T> DPX_D T shfl_down_any(T v, int off)
{
    constexpr int W = (sizeof(T) + 3) / 4;
    union {
        T t;
        int w[W];
    } u;
    u.w[W - 1] = 0;
    u.t = v;
#pragma unroll
    for (int i = 0; i < W; ++i) u.w[i] = __shfl_down(u.w[i], off, 64);
    return u.t;
}

// iteration index -> element offsets of src / dst / aux
DPX_D void iter_offsets(const RedIndex &ix, int64_t o, int64_t &so, int64_t &dof, int64_t &ao)
{
    so = dof = ao = 0;
    for (int d = ix.nd_i - 1; d >= 0; --d) {
        const int64_t q = (d == 0) ? 0 : o / ix.shape_i[d];
        const int64_t i = o - q * ix.shape_i[d];
        so += i * ix.src_istr[d];
        dof += i * ix.dst_str[d];
        ao += i * ix.aux_str[d];
        o = q;
    }
}
DPX_D int64_t red_offset(const RedIndex &ix, int64_t pos)
{
    int64_t off = 0;
    for (int d = ix.nd_r - 1; d >= 0; --d) {
        const int64_t q = (d == 0) ? 0 : pos / ix.shape_r[d];
        off += (pos - q * ix.shape_r[d]) * ix.src_rstr[d];
        pos = q;
    }
    return off;
}

// ================================ policies =================================================
// In: stored input element, Out: stored result element, Acc: running value (also the
// element type of partials in scratch), Aux: per-output side input.

template <class Out> struct acc_of {
    using type = Out;
};
template <> struct acc_of<half_t> {
    using type = float; // half sums and products run in float, rounded once at the end
};
template <> struct acc_of<bool_t> {
    using type = int32_t;
};
template <class Out> using acc_of_t = typename acc_of<Out>::type;

template <class Acc, class Out> DPX_D Out acc_to_out(Acc a)
{
    if constexpr (is_bool_v<Out>) return bool_t{(uint8_t)(a != 0)};
    else if constexpr (std::is_same_v<Acc, Out>) return a;
    else return (Out)a;
}
// input element -> accumulator, converting to the result type first
// (reductions.hpp:482-491: val = convert_impl<outT>(in))
template <class In, class Out> DPX_D acc_of_t<Out> in_to_acc(In x)
{
    using Acc = acc_of_t<Out>;
    if constexpr (is_bool_v<Out>) return (int32_t)convert<bool_t, In>(x).v;
    else if constexpr (std::is_same_v<Out, half_t>) return (float)convert<half_t, In>(x);
    else return (Acc)convert<Out, In>(x);
}

enum { K_SUM = 0, K_PROD = 1, K_MAX = 2, K_MIN = 3, K_SUMSQDEV = 4 };

template <int KIND, class T> DPX_D T red_identity()
{
    if constexpr (KIND == K_SUM || KIND == K_SUMSQDEV) {
        if constexpr (is_cplx_v<T>) return T{0, 0};
        else return T(0);
    }
    else if constexpr (KIND == K_PROD) {
        if constexpr (is_cplx_v<T>) return T{1, 0};
        else return T(1);
    }
    else {
        constexpr bool mx = KIND == K_MAX;
        if constexpr (is_cplx_v<T>) {
            using R = real_of_t<T>;
            const R inf = (R)__builtin_inff();
            return mx ? T{-inf, -inf} : T{inf, inf};
        }
        else if constexpr (is_fp_v<T>) return mx ? -(T)__builtin_inff() : (T)__builtin_inff();
        else if constexpr (std::is_signed_v<T>)
            return mx ? (T)((T)1 << (8 * sizeof(T) - 1)) : (T)~((T)1 << (8 * sizeof(T) - 1));
        else return mx ? T(0) : (T)~T(0);
    }
}

// Policy of the first pass (reads In) and, with In == Acc and FINAL, of the fold pass.
template <int KIND, class In_, class Out_, bool FINAL = false> struct RedPolicy {
    using In = In_;
    using Out = Out_;
    using Acc = std::conditional_t<(KIND == K_MAX || KIND == K_MIN),
                                   std::conditional_t<is_bool_v<Out_>, int32_t, Out_>, acc_of_t<Out_>>;
    using Aux = Out_;
    static constexpr bool has_aux = (KIND == K_SUMSQDEV) && !FINAL;
    static constexpr int kind = KIND;
    DPX_D static Acc identity()
    {
        if constexpr (is_bool_v<Out> && (KIND == K_MAX || KIND == K_MIN)) return KIND == K_MAX ? 0 : 1;
        else if constexpr (is_bool_v<Out>) return KIND == K_PROD ? 1 : 0;
        else return red_identity<KIND, Acc>();
    }
    DPX_D static Acc pre(In x, Acc aux)
    {
        if constexpr (FINAL) return x; // In == Acc
        else if constexpr (KIND == K_SUMSQDEV) {
            const Acc d = in_to_acc<In, Out>(x) - aux;
            return d * d;
        }
        else if constexpr (KIND == K_MAX || KIND == K_MIN) {
            if constexpr (is_bool_v<Out>) return (int32_t)(x.v != 0);
            else return x; // In == Out
        }
        else return in_to_acc<In, Out>(x);
    }
    DPX_D static Acc combine(Acc a, Acc b)
    {
        if constexpr (is_bool_v<Out>) {
            if constexpr (KIND == K_PROD || KIND == K_MIN) return a & b;
            else return a | b;
        }
        else if constexpr (KIND == K_SUM || KIND == K_SUMSQDEV) return a + b;
        else if constexpr (KIND == K_PROD) return a * b;
        else if constexpr (KIND == K_MAX) return max_nan(a, b);
        else return min_nan(a, b);
    }
    DPX_D static Out post(Acc a) { return acc_to_out<Acc, Out>(a); }
    DPX_D static Acc load_aux(const Aux *p)
    {
        if constexpr (std::is_same_v<Aux, half_t>) return (float)*p;
        else if constexpr (is_bool_v<Aux>) return (int32_t)p->v;
        else return (Acc)*p;
    }
};

// ================================ rows kernel ================================================
// Linear block id = oblock * splits + split.  G = 1 << g_log2 lanes per output
// (G <= 64, several outputs per block) or the whole block (G == blockDim.x).
template <class P, bool CONTIG>
__global__ __launch_bounds__(1024) void red_rows_kernel(RedIndex ix, RedLaunch L, const typename P::In *src,
                                                       typename P::Out *dst, typename P::Acc *partial,
                                                       const typename P::Aux *aux)
{
    using In = typename P::In;
    using Acc = typename P::Acc;
    constexpr int E = 16 / (int)sizeof(In);
    const int G = 1 << L.g_log2;
    const bool whole_block = G == (int)blockDim.x;
    const int64_t oblock = (int64_t)blockIdx.x / L.splits;
    const int split = (int)((int64_t)blockIdx.x - oblock * L.splits);
    const int lane = threadIdx.x & (G - 1);
    const int64_t o = whole_block ? oblock : oblock * (blockDim.x >> L.g_log2) + (threadIdx.x >> L.g_log2);
    const bool active = o < L.m;

    Acc acc[RED_U];
#pragma unroll
    for (int u = 0; u < RED_U; ++u) acc[u] = P::identity();

    int64_t so = 0, dof = 0, ao = 0;
    if (active) {
        iter_offsets(ix, o, so, dof, ao);
        Acc a = P::identity();
        if constexpr (P::has_aux) a = P::load_aux(aux + ao);
        const int64_t beg = (int64_t)split * L.chunk;
        const int64_t end = (beg + L.chunk < L.n) ? beg + L.chunk : L.n;
        if constexpr (CONTIG) {
            const In *p = src + so;
            if (L.vec) {
                const int64_t vend = beg + ((end - beg) / E) * E;
                const int64_t step = (int64_t)G * E;
                int64_t pos = beg + (int64_t)lane * E;
                for (; pos + (RED_U - 1) * step < vend; pos += RED_U * step) {
                    pack<In, E> v[RED_U];
#pragma unroll
                    for (int u = 0; u < RED_U; ++u) v[u] = load_pack<In, E>(p + pos + u * step);
#pragma unroll
                    for (int u = 0; u < RED_U; ++u)
#pragma unroll
                        for (int e = 0; e < E; ++e) acc[u] = P::combine(acc[u], P::pre(v[u].v[e], a));
                }
                for (; pos < vend; pos += step) {
                    pack<In, E> v = load_pack<In, E>(p + pos);
#pragma unroll
                    for (int e = 0; e < E; ++e) acc[0] = P::combine(acc[0], P::pre(v.v[e], a));
                }
                for (int64_t t = vend + lane; t < end; t += G) acc[1] = P::combine(acc[1], P::pre(load_one(p + t), a));
            }
            else {
                int64_t pos = beg + lane;
                for (; pos + (RED_U - 1) * (int64_t)G < end; pos += RED_U * (int64_t)G) {
                    In v[RED_U];
#pragma unroll
                    for (int u = 0; u < RED_U; ++u) v[u] = load_one(p + pos + u * (int64_t)G);
#pragma unroll
                    for (int u = 0; u < RED_U; ++u) acc[u] = P::combine(acc[u], P::pre(v[u], a));
                }
                for (; pos < end; pos += G) acc[0] = P::combine(acc[0], P::pre(load_one(p + pos), a));
            }
        }
        else {
            const In *p = src + so;
            for (int64_t pos = beg + lane; pos < end; pos += G)
                acc[0] = P::combine(acc[0], P::pre(load_one(p + red_offset(ix, pos)), a));
        }
    }
    Acc r = P::combine(P::combine(acc[0], acc[1]), P::combine(acc[2], acc[3]));
    static_assert(RED_U == 4);

    const int wl = whole_block ? 64 : G; // lanes to fold with shuffles
    for (int off = wl >> 1; off > 0; off >>= 1) r = P::combine(r, shfl_down_any(r, off));
    if (whole_block) {
        __shared__ Acc sm[16];
        const int w = threadIdx.x >> 6;
        if ((threadIdx.x & 63) == 0) sm[w] = r;
        __syncthreads();
        if (threadIdx.x == 0) {
            const int nw = blockDim.x >> 6;
            for (int i = 1; i < nw; ++i) r = P::combine(r, sm[i]);
        }
    }
    if (active && lane == 0 && (!whole_block || threadIdx.x == 0)) {
        if (L.splits == 1) dst[dof] = P::post(r);
        else partial[o * L.splits + split] = r;
    }
}

// ================================ cols kernel ================================================
// Iteration space: outer dims (0 .. nd_i-2) x inner dim (nd_i-1, src stride 1).
// Block = TY x TX threads, TX = 1 << g_log2 along the inner dim, E_ columns per thread
// (E_ = 16 / sizeof(In) when L.vec, else 1).  Linear block id = (outer * splits + split) *
// col_blocks + col_block.  Partials are laid out [split][output] so the fold pass is again
// a coalesced column reduction.
template <class P>
__global__ __launch_bounds__(256) void red_cols_kernel(RedIndex ix, RedLaunch L, const typename P::In *src,
                                                      typename P::Out *dst, typename P::Acc *partial,
                                                      const typename P::Aux *aux)
{
    using In = typename P::In;
    using Acc = typename P::Acc;
    constexpr int E = 16 / (int)sizeof(In);
    const int TX = 1 << L.g_log2, TY = 256 >> L.g_log2;
    const int tx = threadIdx.x & (TX - 1), ty = threadIdx.x >> L.g_log2;
    int64_t b = blockIdx.x;
    const int64_t cb = b % L.col_blocks;
    b /= L.col_blocks;
    const int split = (int)(b % L.splits);
    const int64_t outer = b / L.splits;
    const int ecnt = L.vec ? E : 1;
    const int64_t col0 = (cb * TX + tx) * ecnt;
    const bool active = col0 < L.inner;

    Acc acc[RED_U][E];
#pragma unroll
    for (int u = 0; u < RED_U; ++u)
#pragma unroll
        for (int e = 0; e < E; ++e) acc[u][e] = P::identity();

    // offsets of the outer iteration index
    int64_t so = 0, dof = 0, ao = 0;
    {
        int64_t o = outer;
        for (int d = ix.nd_i - 2; d >= 0; --d) {
            const int64_t q = (d == 0) ? 0 : o / ix.shape_i[d];
            const int64_t i = o - q * ix.shape_i[d];
            so += i * ix.src_istr[d];
            dof += i * ix.dst_str[d];
            ao += i * ix.aux_str[d];
            o = q;
        }
    }
    const int last = ix.nd_i - 1;
    Acc a[E];
#pragma unroll
    for (int e = 0; e < E; ++e) a[e] = P::identity();
    if (active) {
        if constexpr (P::has_aux) {
#pragma unroll
            for (int e = 0; e < E; ++e)
                if (e < ecnt) a[e] = P::load_aux(aux + ao + (col0 + e) * ix.aux_str[last]);
        }
        const In *p = src + so + col0;
        const int64_t beg = (int64_t)split * L.chunk;
        const int64_t end = (beg + L.chunk < L.n) ? beg + L.chunk : L.n;
        int64_t r = beg + ty;
        if (L.vec) {
            for (; r + (RED_U - 1) * TY < end; r += RED_U * TY) {
                pack<In, E> v[RED_U];
#pragma unroll
                for (int u = 0; u < RED_U; ++u) v[u] = load_pack<In, E>(p + (r + u * TY) * L.rstride);
#pragma unroll
                for (int u = 0; u < RED_U; ++u)
#pragma unroll
                    for (int e = 0; e < E; ++e) acc[u][e] = P::combine(acc[u][e], P::pre(v[u].v[e], a[e]));
            }
            for (; r < end; r += TY) {
                pack<In, E> v = load_pack<In, E>(p + r * L.rstride);
#pragma unroll
                for (int e = 0; e < E; ++e) acc[0][e] = P::combine(acc[0][e], P::pre(v.v[e], a[e]));
            }
        }
        else {
            for (; r + (RED_U - 1) * TY < end; r += RED_U * TY) {
                In v[RED_U];
#pragma unroll
                for (int u = 0; u < RED_U; ++u) v[u] = load_one(p + (r + u * TY) * L.rstride);
#pragma unroll
                for (int u = 0; u < RED_U; ++u) acc[u][0] = P::combine(acc[u][0], P::pre(v[u], a[0]));
            }
            for (; r < end; r += TY) acc[0][0] = P::combine(acc[0][0], P::pre(load_one(p + r * L.rstride), a[0]));
        }
    }
    static_assert(RED_U == 4);
    __shared__ Acc sm[256 * E];
#pragma unroll
    for (int e = 0; e < E; ++e)
        sm[threadIdx.x * E + e] = P::combine(P::combine(acc[0][e], acc[1][e]), P::combine(acc[2][e], acc[3][e]));
    __syncthreads();
    if (ty == 0 && active) {
#pragma unroll
        for (int e = 0; e < E; ++e) {
            if (e < ecnt && col0 + e < L.inner) {
                Acc r = sm[tx * E + e];
                for (int y = 1; y < TY; ++y) r = P::combine(r, sm[(y * TX + tx) * E + e]);
                if (L.splits == 1) dst[dof + (col0 + e) * ix.dst_str[last]] = P::post(r);
                else partial[(int64_t)split * L.m + outer * L.inner + col0 + e] = r;
            }
        }
    }
}

// identity fill for an empty reduced run (reductions.hpp:1417-1422)
template <class P>
__global__ __launch_bounds__(256) void red_fill_kernel(RedIndex ix, int64_t m, typename P::Out *dst)
{
    const int64_t o = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (o >= m) return;
    int64_t so, dof, ao;
    iter_offsets(ix, o, so, dof, ao);
    dst[dof] = P::post(P::identity());
}

// ================================ arg kernels =================================================
// Value + position of the extremum: NaN beats every number, equal values keep the
// smaller position (argmax.cpp:137-160; first NaN as NumPy does).
constexpr int64_t ARG_NONE = INT64_MAX;

template <bool IS_MAX, class T> DPX_D bool arg_better(T v, T best)
{
    // true when v must replace best although it comes later
    if constexpr (is_cplx_v<T>) {
        const bool vn = isnan_(v), bn = isnan_(best);
        if (bn) return false;
        if (vn) return true;
        return IS_MAX ? c_greater(v, best) : c_less(v, best);
    }
    else if constexpr (is_fp_v<T>) {
        if constexpr (IS_MAX) return !(v <= best) && (best == best);
        else return !(v >= best) && (best == best);
    }
    else {
        return IS_MAX ? (v > best) : (v < best);
    }
}
template <class T> DPX_D bool arg_same(T a, T b)
{
    if constexpr (is_cplx_v<T>) return (a == b) || (isnan_(a) && isnan_(b));
    else if constexpr (is_fp_v<T>) return (a == b) || (a != a && b != b);
    else return a == b;
}
template <bool IS_MAX, class T> DPX_D void arg_merge(T &v, int64_t &i, T ov, int64_t oi)
{
    if (oi == ARG_NONE) return;
    if (i == ARG_NONE || arg_better<IS_MAX>(ov, v) || (arg_same(ov, v) && oi < i)) {
        v = ov;
        i = oi;
    }
}

// FIRST: reads src, position = index along the reduced run; otherwise reads the partial
// (value, position) pairs of the previous pass, laid out [output][split].
// Linear block id = oblock * splits + split, lanes per output as in red_rows_kernel.
template <class T, bool IS_MAX, bool CONTIG, bool FIRST>
__global__ __launch_bounds__(1024) void arg_rows_kernel(RedIndex ix, RedLaunch L, const T *src,
                                                       const int64_t *src_idx, int64_t *dst, T *pval,
                                                       int64_t *pidx)
{
    using VT = value_of_t<T>;
    constexpr int E = 16 / (int)sizeof(T);
    const int G = 1 << L.g_log2;
    const bool whole_block = G == (int)blockDim.x;
    const int64_t oblock = (int64_t)blockIdx.x / L.splits;
    const int split = (int)((int64_t)blockIdx.x - oblock * L.splits);
    const int lane = threadIdx.x & (G - 1);
    const int64_t o = whole_block ? oblock : oblock * (blockDim.x >> L.g_log2) + (threadIdx.x >> L.g_log2);
    const bool active = o < L.m;

    VT best{};
    int64_t bidx = ARG_NONE;
    int64_t so = 0, dof = 0, ao = 0;
    if (active) {
        iter_offsets(ix, o, so, dof, ao);
        const int64_t beg = (int64_t)split * L.chunk;
        const int64_t end = (beg + L.chunk < L.n) ? beg + L.chunk : L.n;
        const T *p = src + so;
        if constexpr (!FIRST) {
            const int64_t *pi = src_idx + so;
            for (int64_t pos = beg + lane; pos < end; pos += G)
                arg_merge<IS_MAX, VT>(best, bidx, to_value(load_one(p + pos)), pi[pos]);
        }
        else if constexpr (CONTIG) {
            uint32_t bl = 0; // position relative to beg; chunk < 2^32 by construction
            bool have = false;
            if (L.vec) {
                const int64_t vend = beg + ((end - beg) / E) * E;
                const int64_t step = (int64_t)G * E;
                int64_t pos = beg + (int64_t)lane * E;
                if (pos < vend) {
                    best = to_value(load_one(p + pos));
                    bl = (uint32_t)(pos - beg);
                    have = true;
                }
                for (; pos + (RED_U - 1) * step < vend; pos += RED_U * step) {
                    pack<T, E> v[RED_U];
#pragma unroll
                    for (int u = 0; u < RED_U; ++u) v[u] = load_pack<T, E>(p + pos + u * step);
#pragma unroll
                    for (int u = 0; u < RED_U; ++u)
#pragma unroll
                        for (int e = 0; e < E; ++e) {
                            const VT x = to_value(v[u].v[e]);
                            if (arg_better<IS_MAX, VT>(x, best)) {
                                best = x;
                                bl = (uint32_t)(pos + u * step + e - beg);
                            }
                        }
                }
                for (; pos < vend; pos += step) {
                    pack<T, E> v = load_pack<T, E>(p + pos);
#pragma unroll
                    for (int e = 0; e < E; ++e) {
                        const VT x = to_value(v.v[e]);
                        if (arg_better<IS_MAX, VT>(x, best)) {
                            best = x;
                            bl = (uint32_t)(pos + e - beg);
                        }
                    }
                }
                if (have) bidx = beg + bl;
                for (int64_t t = vend + lane; t < end; t += G)
                    arg_merge<IS_MAX, VT>(best, bidx, to_value(load_one(p + t)), t);
            }
            else {
                int64_t pos = beg + lane;
                if (pos < end) {
                    best = to_value(load_one(p + pos));
                    bl = (uint32_t)(pos - beg);
                    have = true;
                }
                for (; pos + (RED_U - 1) * (int64_t)G < end; pos += RED_U * (int64_t)G) {
                    T v[RED_U];
#pragma unroll
                    for (int u = 0; u < RED_U; ++u) v[u] = load_one(p + pos + u * (int64_t)G);
#pragma unroll
                    for (int u = 0; u < RED_U; ++u) {
                        const VT x = to_value(v[u]);
                        if (arg_better<IS_MAX, VT>(x, best)) {
                            best = x;
                            bl = (uint32_t)(pos + u * (int64_t)G - beg);
                        }
                    }
                }
                for (; pos < end; pos += G) {
                    const VT x = to_value(load_one(p + pos));
                    if (arg_better<IS_MAX, VT>(x, best)) {
                        best = x;
                        bl = (uint32_t)(pos - beg);
                    }
                }
                if (have) bidx = beg + bl;
            }
        }
        else {
            for (int64_t pos = beg + lane; pos < end; pos += G) {
                const VT x = to_value(load_one(p + red_offset(ix, pos)));
                if (bidx == ARG_NONE || arg_better<IS_MAX, VT>(x, best)) {
                    best = x;
                    bidx = pos;
                }
            }
        }
    }
    const int wl = whole_block ? 64 : G;
    for (int off = wl >> 1; off > 0; off >>= 1) {
        const VT ov = shfl_down_any(best, off);
        const int64_t oi = shfl_down_any(bidx, off);
        arg_merge<IS_MAX, VT>(best, bidx, ov, oi);
    }
    if (whole_block) {
        __shared__ VT smv[16];
        __shared__ int64_t smi[16];
        const int w = threadIdx.x >> 6;
        if ((threadIdx.x & 63) == 0) {
            smv[w] = best;
            smi[w] = bidx;
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            const int nw = blockDim.x >> 6;
            for (int i = 1; i < nw; ++i) arg_merge<IS_MAX, VT>(best, bidx, smv[i], smi[i]);
        }
    }
    if (active && lane == 0 && (!whole_block || threadIdx.x == 0)) {
        if (L.splits == 1) dst[dof] = bidx;
        else {
            pval[o * L.splits + split] = to_storage<T>(best);
            pidx[o * L.splits + split] = bidx;
        }
    }
}

// Column variant (reduced axis strided by L.rstride, outputs contiguous).  One column per
// thread; partials laid out [split][output].
template <class T, bool IS_MAX, bool FIRST>
__global__ __launch_bounds__(256) void arg_cols_kernel(RedIndex ix, RedLaunch L, const T *src,
                                                      const int64_t *src_idx, int64_t *dst, T *pval,
                                                      int64_t *pidx)
{
    using VT = value_of_t<T>;
    const int TX = 1 << L.g_log2, TY = 256 >> L.g_log2;
    const int tx = threadIdx.x & (TX - 1), ty = threadIdx.x >> L.g_log2;
    int64_t b = blockIdx.x;
    const int64_t cb = b % L.col_blocks;
    b /= L.col_blocks;
    const int split = (int)(b % L.splits);
    const int64_t outer = b / L.splits;
    const int64_t col = cb * TX + tx;
    const bool active = col < L.inner;
    int64_t so = 0, dof = 0;
    {
        int64_t o = outer;
        for (int d = ix.nd_i - 2; d >= 0; --d) {
            const int64_t q = (d == 0) ? 0 : o / ix.shape_i[d];
            const int64_t i = o - q * ix.shape_i[d];
            so += i * ix.src_istr[d];
            dof += i * ix.dst_str[d];
            o = q;
        }
    }
    VT best{};
    int64_t bidx = ARG_NONE;
    if (active) {
        const T *p = src + so + col;
        const int64_t beg = (int64_t)split * L.chunk;
        const int64_t end = (beg + L.chunk < L.n) ? beg + L.chunk : L.n;
        if constexpr (FIRST) {
            int64_t r = beg + ty;
            for (; r + (RED_U - 1) * TY < end; r += RED_U * TY) {
                T v[RED_U];
#pragma unroll
                for (int u = 0; u < RED_U; ++u) v[u] = load_one(p + (r + u * TY) * L.rstride);
#pragma unroll
                for (int u = 0; u < RED_U; ++u) {
                    const VT x = to_value(v[u]);
                    if (bidx == ARG_NONE || arg_better<IS_MAX, VT>(x, best)) {
                        best = x;
                        bidx = r + u * TY;
                    }
                }
            }
            for (; r < end; r += TY) {
                const VT x = to_value(load_one(p + r * L.rstride));
                if (bidx == ARG_NONE || arg_better<IS_MAX, VT>(x, best)) {
                    best = x;
                    bidx = r;
                }
            }
        }
        else {
            const int64_t *pi = src_idx + so + col;
            for (int64_t r = beg + ty; r < end; r += TY)
                arg_merge<IS_MAX, VT>(best, bidx, to_value(load_one(p + r * L.rstride)), pi[r * L.rstride]);
        }
    }
    __shared__ VT smv[256];
    __shared__ int64_t smi[256];
    smv[threadIdx.x] = best;
    smi[threadIdx.x] = bidx;
    __syncthreads();
    if (ty == 0 && active) {
        for (int y = 1; y < TY; ++y) arg_merge<IS_MAX, VT>(best, bidx, smv[y * TX + tx], smi[y * TX + tx]);
        const int last = ix.nd_i - 1;
        if (L.splits == 1) dst[dof + col * ix.dst_str[last]] = bidx;
        else {
            pval[(int64_t)split * L.m + outer * L.inner + col] = to_storage<T>(best);
            pidx[(int64_t)split * L.m + outer * L.inner + col] = bidx;
        }
    }
}

} // namespace dpx
