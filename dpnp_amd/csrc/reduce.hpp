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
//     over several blocks.  Pass one leaves a partial per block in scratch; the
//     block that finishes last for an output (found with a ticket counter) runs
//     pass two in the same launch: it folds that output's partials in index
//     order.  Partition and fold order are fixed functions of the shapes, so
//     results are bit-reproducible run to run; no value is ever accumulated
//     with an atomic.
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
    int32_t tgroup;   // rows: not 0: two levels of tickets, groups of RED_TGROUP blocks (0: one counter per output)
    int64_t rstride;  // cols: stride of the reduced axis
    int64_t inner;    // cols: length of the inner (contiguous) iteration dim
    int64_t col_blocks;
    int32_t mark_fill; // NaN-ignoring searches: report "extreme equals the value NaNs count as" as -1 - index
    double param;      // K_NANVAR: delta degrees of freedom
    // strides of a one-dimensional iteration space (nd_i1 != 0): the rows kernels then never read
    // RedIndex, whose far part of the kernel-argument segment costs them a dependent fetch at start-up
    int32_t nd_i1;
    int64_t istr0, dstr0, astr0;
    // reduced dims that do not collapse into one run (walk != 0): the reduced space as three digits
    // (extents wd, element strides ws; missing leading digits have extent 1), counted in `units` units of the
    // last digit: 16-byte packs along a unit-stride last dim of `inner` elements (vec != 0: the last extent is
    // the packs per run, the last one of a run possibly partial), else single elements.  `chunk` is in units.
    // (The column kernel walks whole rows: its units are the positions of the reduced space.)
    int32_t walk;
    int64_t units;
    int64_t wd[3], ws[3];
    int64_t istep; // walked column reductions: src stride of the inner iteration dim
    int32_t obatch; // column searches: not 0: a block's thread rows are outer indices (see arg_cols_kernel)
};

// Position in a three-digit reduced space that moves by a fixed number of units per step: the element
// offset is kept up to date by additions, so that no access needs a division.  Digit 0 never wraps for
// positions inside the space and is not kept.
struct RedWalker {
    uint32_t k, i1;                // digits 2 and 1 (the host keeps their extents below 2^31)
    int64_t off;                   // element offset
    uint32_t rel;                  // C-order position of the unit's first element minus that of unit `origin`, mod 2^32
    uint32_t sk, s1, d2, d1;       // the step's digits; extents
    uint32_t srel, wrel;           // position change of a step; its correction when digit 2 wraps
    int64_t soff, w2, w1;          // offset change of a step; corrections of a carry out of digit 2, 1
    // positions: a run of the last digit holds `run` of them, a unit `per_unit` (searches; 0, 0 when not needed)
    DPX_D void start(const RedLaunch &L, int64_t q, int64_t step, int64_t run = 0, int per_unit = 0, int64_t origin = 0)
    {
        const int64_t D2 = L.wd[2], D1 = L.wd[1];
        d2 = (uint32_t)D2;
        d1 = (uint32_t)D1;
        w2 = L.ws[1] - D2 * L.ws[2];
        w1 = L.ws[0] - D1 * L.ws[1];
        const int64_t t = step / D2, tq = q / D2;
        sk = (uint32_t)(step % D2);
        s1 = (uint32_t)(t % D1);
        soff = (t / D1) * L.ws[0] + (int64_t)s1 * L.ws[1] + (int64_t)sk * L.ws[2];
        k = (uint32_t)(q % D2);
        i1 = (uint32_t)(tq % D1);
        off = (tq / D1) * L.ws[0] + (int64_t)i1 * L.ws[1] + (int64_t)k * L.ws[2];
        srel = (uint32_t)(t * run + (int64_t)sk * per_unit);
        wrel = (uint32_t)(run - D2 * per_unit);
        rel = (uint32_t)((tq - origin / D2) * run + ((int64_t)k - origin % D2) * per_unit);
    }
    DPX_D void advance()
    {
        k += sk;
        i1 += s1;
        off += soff;
        rel += srel;
        // runs much longer than a step: no lane of the wave carries in most steps, and one branch skips the rest
        // (which is made of selects: as branches per lane they would serialise the loads of a round)
        if (__builtin_amdgcn_ballot_w64((k >= d2) | (i1 >= d1)) != 0) {
            const bool c2 = k >= d2;
            k -= c2 ? d2 : 0;
            i1 += c2 ? 1 : 0;
            off += c2 ? w2 : 0;
            rel += c2 ? wrel : 0;
            const bool c1 = i1 >= d1;
            i1 -= c1 ? d1 : 0;
            off += c1 ? w1 : 0;
        }
    }
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

// v of the lane CTRL selects inside each row of 16 lanes (DPP), word by word; a lane without a
// source (row_shr by s: the first s lanes of a row) gets its own value back
template <int CTRL, class T> DPX_D T dpp_any(T v)
{
    constexpr int W = (sizeof(T) + 3) / 4;
    union {
        T t;
        int w[W];
    } u;
    u.w[W - 1] = 0;
    u.t = v;
#pragma unroll
    for (int i = 0; i < W; ++i) u.w[i] = __builtin_amdgcn_update_dpp(u.w[i], u.w[i], CTRL, 0xf, 0xf, false);
    return u.t;
}
// v of lane `lane` (a constant), in every lane
template <class T> DPX_D T readlane_any(T v, int lane)
{
    constexpr int W = (sizeof(T) + 3) / 4;
    union {
        T t;
        int w[W];
    } u;
    u.w[W - 1] = 0;
    u.t = v;
#pragma unroll
    for (int i = 0; i < W; ++i) u.w[i] = __builtin_amdgcn_readlane(u.w[i], lane);
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
DPX_D void iter_offsets(const RedIndex &ix, const RedLaunch &L, int64_t o, int64_t &so, int64_t &dof, int64_t &ao)
{
    if (L.nd_i1) {
        so = o * L.istr0;
        dof = o * L.dstr0;
        ao = o * L.astr0;
    }
    else iter_offsets(ix, o, so, dof, ao);
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

enum {
    K_SUM = 0, K_PROD = 1, K_MAX = 2, K_MIN = 3, K_SUMSQDEV = 4, K_LOGSUMEXP = 5, K_HYPOT = 6,
    // NaN-ignoring forms: a NaN element contributes the identity (0, 1, nothing, not counted)
    K_NANSUM = 7, K_NANPROD = 8, K_NANMAX = 9, K_NANMIN = 10, K_NANCOUNT = 11, K_NANSUMSQDEV = 12,
    // truth-value reductions of any input type: an element counts as true when it is not zero
    K_ANY = 13, K_ALL = 14, K_COUNT_NONZERO = 15,
    // mean of the elements that are not NaN: sum and count travel together, divided at the end
    K_NANMEAN = 16,
    // variance of the elements that are not NaN around a given mean: squared deviations and count travel
    // together, divided by count - ddof at the end
    K_NANVAR = 17,
    // sum of squared deviations from the mean WITHOUT a given mean, in one pass: (count, mean, sum of squared
    // deviations) triples merged pairwise (Chan, Golub, LeVeque 1979)
    K_SQDEV1 = 18
};
constexpr bool kind_has_count(int k) { return k == K_NANMEAN || k == K_NANVAR; }
// accumulator of K_LOGSUMEXP: log(sum(exp(x))) = m + log(s), m the largest element so far, s = sum(exp(x - m)).
// Merging costs one exp; the pairwise logaddexp it replaces (logsumexp.cpp with math_utils.hpp:129-150) an exp
// and a log1p per element.
template <class A> struct lse_acc {
    A m, s;
};
template <class A> DPX_D A lse_exp(A x) // x <= 0
{
    if constexpr (std::is_same_v<A, float>) return __expf(x);
    else return m_exp(x);
}
template <class A> DPX_D lse_acc<A> lse_merge(lse_acc<A> a, lse_acc<A> b)
{
    const A d = a.m - b.m;
    const bool same = a.m == b.m; // also equal infinities, whose difference is NaN
    const A e = same ? A(1) : lse_exp<A>(d > A(0) ? -d : d);
    const bool ge = d >= A(0) || same; // a NaN operand: false, and e is NaN, which s keeps
    return lse_acc<A>{ge ? a.m : b.m, ge ? a.s + b.s * e : a.s * e + b.s};
}
// accumulator of K_SQDEV1: n elements of mean `mean`, m2 = sum of their squared deviations from it
template <class A> struct sqdev_acc {
    A n, mean, m2;
};
template <class A> DPX_D sqdev_acc<A> sqdev_merge(sqdev_acc<A> a, sqdev_acc<A> b)
{
    const A n = a.n + b.n;
    if (n == A(0)) return a;
    const A d = b.mean - a.mean;
    const A fb = b.n / n;
    return sqdev_acc<A>{n, a.mean + d * fb, a.m2 + b.m2 + d * d * (a.n * fb)};
}
// accumulator of K_NANMEAN
template <class A> struct mean_acc {
    A s;
    int64_t c;
};
constexpr bool kind_is_minmax(int k) { return k == K_MAX || k == K_MIN || k == K_NANMAX || k == K_NANMIN; }

template <int KIND, class T> DPX_D T red_identity()
{
    if constexpr (KIND == K_SUM || KIND == K_SUMSQDEV || KIND == K_HYPOT) {
        if constexpr (is_cplx_v<T>) return T{0, 0};
        else return T(0);
    }
    else if constexpr (KIND == K_LOGSUMEXP) {
        return -(T)__builtin_inff();
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
    // Sums of bools and of 1- and 2-byte integers into a float32 or float64 result (mean of an image stack,
    // sum(mask, dtype=float)) are added up in 64-bit integers, exactly, and converted once: the reference converts
    // every element first (reductions.hpp:482-491) and rounds along the way, so this is never less accurate, and
    // the integer kernels' word arithmetic and narrow column sums apply (uint8 16384 x 65536 averaged down the
    // columns: 41 % of the HBM rate with a conversion and a double addition per element).
    static constexpr bool int_sum = KIND == K_SUM && !FINAL && sizeof(In_) <= 2 &&
                                    (std::is_integral_v<In_> || is_bool_v<In_>) &&
                                    (std::is_same_v<Out_, float> || std::is_same_v<Out_, double>);
    using IntSumAcc = std::conditional_t<std::is_signed_v<In_> && !is_bool_v<In_>, int64_t, uint64_t>;
    using Acc = std::conditional_t<
        int_sum, IntSumAcc,
        std::conditional_t<
        KIND == K_SQDEV1, sqdev_acc<acc_of_t<Out_>>,
        std::conditional_t<KIND == K_LOGSUMEXP, lse_acc<acc_of_t<Out_>>,
        std::conditional_t<
            kind_has_count(KIND), mean_acc<acc_of_t<Out_>>,
            std::conditional_t<kind_is_minmax(KIND), std::conditional_t<is_bool_v<Out_>, int32_t, Out_>, acc_of_t<Out_>>>>>>;
    // sum(|z - mean|^2) of complex input into a real result (variance of complex data,
    // dpnp/dpnp_iface_statistics.py:1849-1851: x * conj(x), real part): the mean is a complex number of the
    // result's precision, the deviation's two parts are squared and added in the real accumulator
    static constexpr bool cplx_dev = KIND == K_SUMSQDEV && is_cplx_v<In_> && !is_cplx_v<Out_> && !FINAL;
    using Aux = std::conditional_t<cplx_dev, cplx<Out_>, Out_>;
    // what a kernel keeps of an output's side input while it reads that output's elements
    using AuxAcc = std::conditional_t<cplx_dev, cplx<acc_of_t<Out_>>, Acc>;
    static constexpr bool has_aux = (KIND == K_SUMSQDEV || KIND == K_NANSUMSQDEV || KIND == K_NANVAR) && !FINAL;
    static constexpr int kind = KIND;
    DPX_D static AuxAcc aux_identity()
    {
        if constexpr (cplx_dev) return AuxAcc{0, 0};
        else return identity();
    }
    DPX_D static Acc identity()
    {
        if constexpr (kind_has_count(KIND)) return Acc{red_identity<K_SUM, acc_of_t<Out>>(), 0};
        else if constexpr (KIND == K_SQDEV1) return Acc{0, 0, 0};
        else if constexpr (KIND == K_LOGSUMEXP) return Acc{-(acc_of_t<Out>)__builtin_inff(), 0};
        else if constexpr (is_bool_v<Out> && (KIND == K_MAX || KIND == K_MIN)) return KIND == K_MAX ? 0 : 1;
        else if constexpr (is_bool_v<Out>) return (KIND == K_PROD || KIND == K_ALL) ? 1 : 0;
        else if constexpr (KIND == K_COUNT_NONZERO) return Acc(0);
        else if constexpr (KIND == K_NANMAX || KIND == K_NANMIN) return (Acc)__builtin_nanf(""); // "nothing yet"
        else if constexpr (KIND == K_NANSUM || KIND == K_NANCOUNT || KIND == K_NANSUMSQDEV)
            return red_identity<K_SUM, Acc>();
        else if constexpr (KIND == K_NANPROD) return red_identity<K_PROD, Acc>();
        else return red_identity<KIND, Acc>();
    }
    DPX_D static Acc pre(In x, AuxAcc aux)
    {
        if constexpr (FINAL) return x; // In == Acc
        else if constexpr (int_sum) {
            if constexpr (is_bool_v<In>) return (Acc)(x.v != 0);
            else return (Acc)x;
        }
        else if constexpr (cplx_dev) {
            const Acc dr = (Acc)x.re - aux.re, di = (Acc)x.im - aux.im;
            return dr * dr + di * di;
        }
        else if constexpr (KIND == K_SQDEV1) return Acc{1, in_to_acc<In, Out>(x) - aux.mean, 0}; // means are kept relative to aux.mean
        else if constexpr (KIND == K_LOGSUMEXP) return Acc{in_to_acc<In, Out>(x), 1};
        else if constexpr (KIND == K_NANMEAN) {
            const bool skip = isnan_(x);
            return Acc{skip ? red_identity<K_SUM, acc_of_t<Out>>() : in_to_acc<In, Out>(x), skip ? 0 : 1};
        }
        else if constexpr (KIND == K_NANVAR) { // aux.s holds the mean
            const acc_of_t<Out> d = in_to_acc<In, Out>(x) - aux.s;
            const bool skip = isnan_(x);
            return Acc{skip ? acc_of_t<Out>(0) : d * d, skip ? 0 : 1};
        }
        else if constexpr (KIND == K_SUMSQDEV) {
            const Acc d = in_to_acc<In, Out>(x) - aux;
            return d * d;
        }
        else if constexpr (KIND == K_NANSUMSQDEV) {
            const Acc d = in_to_acc<In, Out>(x) - aux;
            return isnan_(x) ? Acc(0) : d * d;
        }
        else if constexpr (KIND == K_NANSUM || KIND == K_NANPROD) return isnan_(x) ? identity() : in_to_acc<In, Out>(x);
        else if constexpr (KIND == K_NANCOUNT) return isnan_(x) ? Acc(0) : Acc(1);
        else if constexpr (KIND == K_ANY || KIND == K_ALL || KIND == K_COUNT_NONZERO)
            return (Acc)convert<bool_t, In>(x).v;
        else if constexpr (kind_is_minmax(KIND)) {
            if constexpr (is_bool_v<Out>) return (int32_t)(x.v != 0);
            else return x; // In == Out
        }
        else return in_to_acc<In, Out>(x);
    }
    DPX_D static Acc combine(Acc a, Acc b)
    {
        if constexpr (kind_has_count(KIND)) return Acc{a.s + b.s, a.c + b.c};
        else if constexpr (KIND == K_SQDEV1) return sqdev_merge(a, b);
        else if constexpr (is_bool_v<Out>) {
            if constexpr (KIND == K_PROD || KIND == K_MIN || KIND == K_ALL) return a & b;
            else return a | b;
        }
        else if constexpr (KIND == K_SUM || KIND == K_SUMSQDEV || KIND == K_NANSUM || KIND == K_NANCOUNT ||
                           KIND == K_NANSUMSQDEV || KIND == K_COUNT_NONZERO)
            return a + b;
        else if constexpr (KIND == K_PROD || KIND == K_NANPROD) return a * b;
        else if constexpr (KIND == K_LOGSUMEXP) return lse_merge(a, b);
        else if constexpr (KIND == K_HYPOT) return m_hypot(a, b);
        else if constexpr (KIND == K_MAX) return max_nan(a, b);
        else if constexpr (KIND == K_NANMAX) return isnan_(a) ? b : (isnan_(b) ? a : (a > b ? a : b));
        else if constexpr (KIND == K_NANMIN) return isnan_(a) ? b : (isnan_(b) ? a : (a < b ? a : b));
        else return min_nan(a, b);
    }
    // One-byte inputs of the counting kinds are folded a pack (16 elements, four words) at a time
    // with word arithmetic; element by element the kernel is bound by vector instructions
    // (about 64 per pack against about 20 here).
    static constexpr bool has_pack_fold =
        !FINAL && sizeof(In) == 1 &&
        (KIND == K_ANY || KIND == K_ALL || KIND == K_COUNT_NONZERO ||
         (KIND == K_SUM && (is_int_v<In> || is_bool_v<In>) && (is_int_v<Out> || int_sum)) ||
         ((KIND == K_MAX || KIND == K_MIN) && is_int_v<In> && std::is_same_v<In, Out>));
    DPX_D static Acc fold_pack(Acc acc, const u32x4 &words)
    {
        // (the kernel loads the words as such: a pack of bytes viewed as words makes the compiler
        // split the load)
        struct {
            uint32_t w[4];
        } u = {{words[0], words[1], words[2], words[3]}};
        if constexpr (KIND == K_MAX || KIND == K_MIN) {
            // the bytes of even and of odd places as pairs of 16-bit numbers, eight pairs folded by the packed
            // maximum: 23 instructions for 16 elements where taking them one by one costs about 40
            using S = std::conditional_t<std::is_signed_v<In>, short, unsigned short>;
            typedef S s2 __attribute__((ext_vector_type(2)));
            auto even = [](uint32_t w) {
                if constexpr (std::is_signed_v<In>) return (__builtin_bit_cast(s2, w) << 8) >> 8;
                else return __builtin_bit_cast(s2, w & 0x00ff00ffu);
            };
            auto odd = [](uint32_t w) {
                if constexpr (std::is_signed_v<In>) return __builtin_bit_cast(s2, w) >> 8;
                else return __builtin_bit_cast(s2, (w >> 8) & 0x00ff00ffu);
            };
            auto op = [](s2 a, s2 b) {
                if constexpr (KIND == K_MAX) return __builtin_elementwise_max(a, b);
                else return __builtin_elementwise_min(a, b);
            };
            s2 m = op(even(u.w[0]), odd(u.w[0]));
#pragma unroll
            for (int i = 1; i < 4; ++i) m = op(m, op(even(u.w[i]), odd(u.w[i])));
            const S r = (KIND == K_MAX) ? (m.x > m.y ? m.x : m.y) : (m.x < m.y ? m.x : m.y);
            return combine(acc, (Acc)(In)r);
        }
        else if constexpr (KIND == K_ANY) return acc | (Acc)((u.w[0] | u.w[1] | u.w[2] | u.w[3]) != 0);
        else if constexpr (KIND == K_ALL) {
            uint32_t z = 0; // bit 7 of a byte set: that byte is zero
#pragma unroll
            for (int i = 0; i < 4; ++i) z |= (u.w[i] - 0x01010101u) & ~u.w[i] & 0x80808080u;
            return acc & (Acc)(z == 0);
        }
        else if constexpr (KIND == K_COUNT_NONZERO || is_bool_v<In>) {
            uint32_t c = 0; // bit 7 of a byte set: that byte is not zero
#pragma unroll
            for (int i = 0; i < 4; ++i)
                c += (uint32_t)__builtin_popcount((((u.w[i] & 0x7f7f7f7fu) + 0x7f7f7f7fu) | u.w[i]) & 0x80808080u);
            return acc + (Acc)c;
        }
        else if constexpr (std::is_same_v<In, uint8_t>) {
            uint32_t t = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) t = __builtin_amdgcn_sad_u8(u.w[i], 0u, t);
            return acc + (Acc)t;
        }
        else { // int8: bytes biased by 128 are summed as unsigned
            uint32_t t = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) t = __builtin_amdgcn_sad_u8(u.w[i] ^ 0x80808080u, 0u, t);
            return acc + (Acc)((int32_t)t - 16 * 128);
        }
    }
    DPX_D static Out post(Acc a)
    {
        if constexpr (KIND == K_NANVAR) return post(a, 0.0);
        else if constexpr (KIND == K_SQDEV1) return acc_to_out<acc_of_t<Out>, Out>(a.m2);
        else if constexpr (KIND == K_LOGSUMEXP) return acc_to_out<acc_of_t<Out>, Out>(a.m + m_log(a.s));
        else if constexpr (KIND == K_NANMEAN) {
            // sum / count in the accumulator's type: 0 / 0 = NaN for a run without a number
            using A = acc_of_t<Out>;
            if constexpr (is_cplx_v<A>) {
                using R = real_of_t<A>;
                return acc_to_out<A, Out>(A{a.s.re / (R)a.c, a.s.im / (R)a.c});
            }
            else return acc_to_out<A, Out>(a.s / (A)a.c);
        }
        else return acc_to_out<Acc, Out>(a);
    }
    // result of a run given the launch's scalar parameter
    DPX_D static Out post(Acc a, double param)
    {
        if constexpr (KIND == K_NANVAR) {
            using A = acc_of_t<Out>;
            const A dof = (A)a.c - (A)param;
            return acc_to_out<A, Out>(dof > A(0) ? a.s / dof : (A)__builtin_nanf(""));
        }
        else return post(a);
    }
    DPX_D static AuxAcc load_aux(const Aux *p)
    {
        if constexpr (cplx_dev) return AuxAcc{(Acc)p->re, (Acc)p->im};
        else if constexpr (KIND == K_NANVAR) return Acc{(acc_of_t<Out>)*p, 0};
        else if constexpr (std::is_same_v<Aux, half_t>) return (float)*p;
        else if constexpr (is_bool_v<Aux>) return (int32_t)p->v;
        else return (Acc)*p;
    }
};

// ================================ rows kernel ================================================
// Linear block id = oblock * splits + split.  G = 1 << g_log2 lanes per output
// (G <= 64, several outputs per block) or the whole block (G == blockDim.x).
// Folds r over the G lanes of a group (G <= 64: shuffles only) or over the whole block
// (wave shuffles, then the wave leaders' values through LDS in wave order).  The result is
// valid in lane 0 of the group / thread 0 of the block.
template <class P> DPX_D typename P::Acc group_reduce(typename P::Acc r, bool whole_block, int G)
{
    using Acc = typename P::Acc;
    if (whole_block) {
        // a whole wave (all 64 lanes are here): rows of 16 lanes fold through DPP shifts into their
        // last lane (row_shr:1, 2, 4, 8), the four row results are read from lanes 15, 31, 47, 63 and
        // combined in that order in every lane.  0.3 us shorter than six lane permutes through LDS.
        r = P::combine(r, dpp_any<0x111>(r));
        r = P::combine(r, dpp_any<0x112>(r));
        r = P::combine(r, dpp_any<0x114>(r));
        r = P::combine(r, dpp_any<0x118>(r));
        r = P::combine(P::combine(P::combine(readlane_any(r, 15), readlane_any(r, 31)), readlane_any(r, 47)),
                       readlane_any(r, 63));
    }
    else
        for (int off = G >> 1; off > 0; off >>= 1) r = P::combine(r, shfl_down_any(r, off));
    if (whole_block) {
        __shared__ Acc sm[16];
        __syncthreads(); // sm may still be read by a previous call
        const int w = threadIdx.x >> 6;
        if ((threadIdx.x & 63) == 0) sm[w] = r;
        __syncthreads();
        if (threadIdx.x == 0) {
            const int nw = blockDim.x >> 6;
            for (int i = 1; i < nw; ++i) r = P::combine(r, sm[i]);
        }
    }
    return r;
}

// ---- cross-block hand-off ------------------------------------------------------------------
// A partial travels between blocks through agent-scope atomics only: the producer writes it
// with atomic exchanges (performed at the device's coherence point, so no cache has to be
// written back), takes its ticket with an atomic add whose address depends on the values
// the exchanges returned (the add cannot issue before the exchanges have completed), and
// the one block that draws the last ticket invalidates its caches once and reads the
// partials.  A release fence per block instead (L2 write-back) cost 15-30 % of kernel time.
template <class T> struct Slot {
    static constexpr int W = ((int)sizeof(T) + 3) / 4;
    uint32_t w[W];
};

// Stores v into *p; returns 0, available only once the store has completed device-wide.
template <class T> DPX_D uint32_t slot_publish(Slot<T> *p, const T &v)
{
    union {
        Slot<T> s;
        T t;
    } u;
#pragma unroll
    for (int i = 0; i < Slot<T>::W; ++i) u.s.w[i] = 0;
    u.t = v;
    uint32_t tok = 0;
#pragma unroll
    for (int i = 0; i < Slot<T>::W; ++i)
        tok |= __hip_atomic_exchange(&p->w[i], u.s.w[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    uint32_t zero;
    asm volatile("v_and_b32 %0, 0, %1" : "=v"(zero) : "v"(tok));
    return zero;
}
template <class T> DPX_D T slot_read(const Slot<T> *p)
{
    union {
        Slot<T> s;
        T t;
    } u;
    // atomic loads like the exchanges that wrote the words: served where those were performed
#pragma unroll
    for (int i = 0; i < Slot<T>::W; ++i)
        u.s.w[i] = __hip_atomic_load(&p->w[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return u.t;
}

// Called by every thread of a block, after the threads that hold a partial have published it with
// slot_publish; `zero` is what slot_publish returned in thread 0 (0 if it published nothing).  True,
// for all threads, in the block that took the last of `splits` tickets for this counter: every
// partial of the output is then readable.  The counter is left at zero for the next launch.
// Order: a thread leaves slot_publish only when its exchanges have returned (the asm statement there
// consumes their results), the barrier below is passed when every thread has, and thread 0 draws the
// ticket after the barrier.
DPX_D bool last_block_of(unsigned *counter, int splits, uint32_t zero)
{
    __shared__ int is_last;
    __syncthreads();
    if (threadIdx.x == 0) {
        const unsigned t = __hip_atomic_fetch_add(counter + zero, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        is_last = (t == (unsigned)(splits - 1));
        if (is_last) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    const bool last = is_last != 0;
    if (last) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    return last;
}

// The same with two levels of tickets, for outputs that many blocks share: atomics on one
// address are served one at a time (about 10 ns each on MI355X, 5 us for 512 blocks that
// finish together), so blocks draw their ticket from a counter per group of RED_TGROUP blocks
// and only the last block of a group draws from the output's counter.  `group_counters`
// holds the groups of this output, RED_GROUP_PITCH words apart (separate cache lines).
constexpr int RED_GROUP_PITCH = 32;
constexpr int RED_TGROUP_LOG2 = 5, RED_TGROUP = 1 << RED_TGROUP_LOG2;
DPX_D bool last_block_of_grouped(unsigned *counter, unsigned *group_counters, int split, int splits, uint32_t zero)
{
    __shared__ int is_last2;
    __syncthreads();
    if (threadIdx.x == 0) {
        const int g = split >> RED_TGROUP_LOG2, ng = (splits + RED_TGROUP - 1) >> RED_TGROUP_LOG2;
        const int in_g = (g == ng - 1) ? splits - g * RED_TGROUP : RED_TGROUP;
        unsigned *c1 = group_counters + (size_t)g * RED_GROUP_PITCH;
        const unsigned t = __hip_atomic_fetch_add(c1 + zero, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        int last = 0;
        if (t == (unsigned)(in_g - 1)) {
            __hip_atomic_store(c1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            // the second ticket's address depends on the first ticket: it is drawn after it
            uint32_t z2;
            asm volatile("v_and_b32 %0, 0, %1" : "=v"(z2) : "v"(t));
            const unsigned t2 = __hip_atomic_fetch_add(counter + z2, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (t2 == (unsigned)(ng - 1)) {
                __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                last = 1;
            }
        }
        is_last2 = last;
    }
    __syncthreads();
    const bool last = is_last2 != 0;
    if (last) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    return last;
}
// scratch layout: [RED_MAX_TICKETS output counters | RED_MAX_GROUPS group counters, RED_GROUP_PITCH
// words apart | partials]; the pool hands out zeroed memory and the kernels leave every counter at
// zero again
constexpr int64_t RED_MAX_TICKETS = 16384;
constexpr int64_t RED_MAX_GROUPS = 512;
constexpr size_t RED_COUNTER_BYTES = (RED_MAX_TICKETS + RED_MAX_GROUPS * RED_GROUP_PITCH) * sizeof(unsigned);
// ticket of block `split` of output `o` under the launch's scheme
DPX_D bool last_block_of_output(unsigned *counters, const RedLaunch &L, int64_t o, int split, uint32_t zero)
{
    if (L.tgroup == 0) return last_block_of(counters + o, L.splits, zero);
    const int ng = (L.splits + RED_TGROUP - 1) >> RED_TGROUP_LOG2;
    return last_block_of_grouped(counters + o, counters + RED_MAX_TICKETS + (o * ng) * RED_GROUP_PITCH, split,
                                 L.splits, zero);
}

template <class P, bool CONTIG>
__global__ __launch_bounds__(1024) void red_rows_kernel(RedLaunch L, const typename P::In *src, typename P::Out *dst,
                                                       Slot<typename P::Acc> *partial, const typename P::Aux *aux,
                                                       unsigned *counters, RedIndex ix)
{
    using In = typename P::In;
    using Acc = typename P::Acc;
    constexpr int E = 16 / (int)sizeof(In);
    const int G = 1 << L.g_log2;
    const bool whole_block = G == (int)blockDim.x;
    // (32-bit: the grid has fewer than 2^32 blocks)
    const uint32_t ob32 = (L.splits == 1) ? blockIdx.x : blockIdx.x / (uint32_t)L.splits;
    const int64_t oblock = ob32;
    const int split = (int)(blockIdx.x - ob32 * (uint32_t)L.splits);
    const int lane = threadIdx.x & (G - 1);
    const int64_t o = whole_block ? oblock : oblock * (blockDim.x >> L.g_log2) + (threadIdx.x >> L.g_log2);
    const bool active = o < L.m;

    Acc acc[RED_U];
#pragma unroll
    for (int u = 0; u < RED_U; ++u) acc[u] = P::identity();

    int64_t so = 0, dof = 0, ao = 0;
    if (active) {
        iter_offsets(ix, L, o, so, dof, ao);
        typename P::AuxAcc a = P::aux_identity();
        if constexpr (P::has_aux) a = P::load_aux(aux + ao);
        const int64_t beg = (int64_t)split * L.chunk;
        const int64_t end = (beg + L.chunk < L.n) ? beg + L.chunk : L.n;
        if constexpr (CONTIG) {
            const In *p = src + so;
            if constexpr (P::kind == K_SQDEV1) {
                // Means travel relative to a reference k0 that every lane and block of an output computes alike:
                // merges only use differences of means, and absolute means of data far from zero would round them
                // away.  k0 is the mean of the run's first 64 elements (a whole block per output: its runs are
                // longer) or its first element (short runs).  Being the mean of 64 of the run's N elements it lies
                // within sqrt(N / 64) standard deviations of the run's mean, whatever the data.
                using A = acc_of_t<typename P::Out>;
                A k0;
                if (whole_block) {
                    k0 = in_to_acc<In, typename P::Out>(load_one(p + (threadIdx.x & 63)));
#pragma unroll
                    for (int m = 32; m > 0; m >>= 1) k0 += __shfl_xor(k0, m, 64);
                    k0 *= A(1.0 / 64);
                }
                else k0 = in_to_acc<In, typename P::Out>(load_one(p));
                a = Acc{0, k0, 0};
            }
            if (L.vec) {
                const int64_t vend = beg + ((end - beg) / E) * E;
                const int64_t step = (int64_t)G * E;
                int64_t pos = beg + (int64_t)lane * E;
                if constexpr (P::has_pack_fold) {
                    for (; pos + (RED_U - 1) * step < vend; pos += RED_U * step) {
                        u32x4 v[RED_U];
#pragma unroll
                        for (int u = 0; u < RED_U; ++u) v[u] = load_words16(p + pos + u * step);
#pragma unroll
                        for (int u = 0; u < RED_U; ++u) acc[u] = P::fold_pack(acc[u], v[u]);
                    }
                    for (; pos < vend; pos += step) acc[0] = P::fold_pack(acc[0], load_words16(p + pos));
                }
                else if constexpr (P::kind == K_LOGSUMEXP) {
                    // a round of loads at a time: its largest element first, then one exp per element (and one to
                    // rescale the running sum) instead of a merge, with its compare and select, per element
                    using A = acc_of_t<typename P::Out>;
                    auto take = [&](const A (&x)[RED_U * E], int cnt) {
                        A bm = acc[0].m;
#pragma unroll
                        for (int i = 0; i < RED_U * E; ++i)
                            if (i < cnt) bm = x[i] > bm ? x[i] : bm;
                        A sum = acc[0].m == bm ? acc[0].s : acc[0].s * lse_exp<A>(acc[0].m - bm);
#pragma unroll
                        for (int i = 0; i < RED_U * E; ++i)
                            if (i < cnt) sum += x[i] == bm ? A(1) : lse_exp<A>(x[i] - bm); // (a NaN element: NaN)
                        acc[0] = Acc{bm, sum};
                    };
                    for (; pos + (RED_U - 1) * step < vend; pos += RED_U * step) {
                        pack<In, E> v[RED_U];
#pragma unroll
                        for (int u = 0; u < RED_U; ++u) v[u] = load_pack<In, E>(p + pos + u * step);
                        A x[RED_U * E];
#pragma unroll
                        for (int u = 0; u < RED_U; ++u)
#pragma unroll
                            for (int e = 0; e < E; ++e) x[u * E + e] = in_to_acc<In, typename P::Out>(v[u].v[e]);
                        take(x, RED_U * E);
                    }
                    for (; pos < vend; pos += step) {
                        const pack<In, E> v = load_pack<In, E>(p + pos);
                        A x[RED_U * E];
#pragma unroll
                        for (int e = 0; e < E; ++e) x[e] = in_to_acc<In, typename P::Out>(v.v[e]);
                        take(x, E);
                    }
                }
                else if constexpr (P::kind == K_SQDEV1) {
                    // A lane's elements as sums of d and d^2, d = x - k, k the lane's first element: two
                    // operations per element where a merge of triples takes a division.  count, mean and m2
                    // follow as (n, k + s1 / n, s2 - s1^2 / n).  Because k is one of the elements, s2 is at most
                    // (n + 1) m2, so the rounding of s2 costs m2 a relative error of at most (n + 1) eps, n being
                    // the few thousand elements of one lane; the lanes' triples are merged pairwise.
                    using A = acc_of_t<typename P::Out>;
                    if (pos < vend) {
                        const A k = in_to_acc<In, typename P::Out>(load_one(p + pos));
                        A s1[RED_U], s2[RED_U];
#pragma unroll
                        for (int u = 0; u < RED_U; ++u) s1[u] = s2[u] = A(0);
                        int64_t cnt = 0;
                        for (; pos + (RED_U - 1) * step < vend; pos += RED_U * step) {
                            pack<In, E> v[RED_U];
#pragma unroll
                            for (int u = 0; u < RED_U; ++u) v[u] = load_pack<In, E>(p + pos + u * step);
#pragma unroll
                            for (int u = 0; u < RED_U; ++u)
#pragma unroll
                                for (int e = 0; e < E; ++e) {
                                    const A d = in_to_acc<In, typename P::Out>(v[u].v[e]) - k;
                                    s1[u] += d;
                                    s2[u] += d * d;
                                }
                            cnt += RED_U * E;
                        }
                        for (; pos < vend; pos += step) {
                            const pack<In, E> v = load_pack<In, E>(p + pos);
#pragma unroll
                            for (int e = 0; e < E; ++e) {
                                const A d = in_to_acc<In, typename P::Out>(v.v[e]) - k;
                                s1[0] += d;
                                s2[0] += d * d;
                            }
                            cnt += E;
                        }
                        const A t1 = (s1[0] + s1[1]) + (s1[2] + s1[3]), t2 = (s2[0] + s2[1]) + (s2[2] + s2[3]);
                        const A n = (A)cnt;
                        const A m2 = t2 - t1 * (t1 / n);
                        acc[0] = Acc{n, (k - a.mean) + t1 / n, m2 < A(0) ? A(0) : m2};
                    }
                }
                else {
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
        else if (L.walk) {
            const In *p = src + so;
            const int64_t uend = (beg + L.chunk < L.units) ? beg + L.chunk : L.units;
            const int64_t c = L.inner;
            // (one-pass squared deviations: as in the contiguous form above, with the first element of the
            // output's reduced space as the reference of the means)
            constexpr bool SQ = P::kind == K_SQDEV1;
            using SA = std::conditional_t<SQ, acc_of_t<typename P::Out>, int>;
            if constexpr (SQ) a = Acc{0, in_to_acc<In, typename P::Out>(load_one(p)), 0};
            // MODE 0: units are elements; 1: packs, every run a whole number of them; 2: packs, the last one of
            // a run partial: it is read as the whole pack that ends with the run's last element (a run holds at
            // least one pack) and the elements it shares with the pack before are left out, so that every
            // lane issues the same loads whatever its units are; 3: a run of every other element (L.walk == 2):
            // the lines it touches are read as in mode 2 (`inner` is their length, 2 x elements - 1) and the
            // elements at odd places are left out as well, a quarter of the load instructions of mode 0
            auto walk = [&](auto mode_tag) {
                constexpr int MODE = decltype(mode_tag)::value;
                RedWalker w;
                int64_t q = beg + lane;
                w.start(L, q, G);
                // does element e of a pack read `skip` places early count?
                auto counts = [&](int e, int skip) {
                    if constexpr (MODE == 2) return e >= skip;
                    else if constexpr (MODE == 3) return e >= skip && ((e + skip) & 1) == 0;
                    else return true;
                };
                const uint32_t c32 = (uint32_t)c; // (the host keeps run lengths below 2^31)
                auto skipped = [&](uint32_t k) {
                    const uint32_t rem = c32 - k * E;
                    return rem < (uint32_t)E ? E - (int)rem : 0;
                };
                // element x into accumulator set u, if it counts
                SA sk = 0, s1[RED_U], s2[RED_U];
                int64_t cnt = 0;
#pragma unroll
                for (int u = 0; u < RED_U; ++u) s1[u] = s2[u] = 0;
                if constexpr (SQ) {
                    if (q < uend) sk = in_to_acc<In, typename P::Out>(load_one(p + w.off));
                }
                auto fold = [&](int u, In x, bool ok) {
                    if constexpr (SQ) {
                        const SA d = in_to_acc<In, typename P::Out>(x) - sk;
                        s1[u] += ok ? d : SA(0);
                        s2[u] += ok ? d * d : SA(0);
                        cnt += ok ? 1 : 0;
                    }
                    else {
                        const Acc t = P::combine(acc[u], P::pre(x, a));
                        acc[u] = ok ? t : acc[u];
                    }
                };
                for (; q + (RED_U - 1) * (int64_t)G < uend; q += RED_U * (int64_t)G) {
                    if constexpr (MODE == 0) {
                        In v[RED_U];
#pragma unroll
                        for (int u = 0; u < RED_U; ++u) {
                            v[u] = load_one(p + w.off);
                            w.advance();
                        }
#pragma unroll
                        for (int u = 0; u < RED_U; ++u) fold(u, v[u], true);
                    }
                    else {
                        pack<In, E> v[RED_U];
                        int skip[RED_U];
#pragma unroll
                        for (int u = 0; u < RED_U; ++u) {
                            skip[u] = MODE >= 2 ? skipped(w.k) : 0;
                            v[u] = load_pack<In, E>(p + w.off - skip[u]);
                            w.advance();
                        }
#pragma unroll
                        for (int u = 0; u < RED_U; ++u)
#pragma unroll
                            for (int e = 0; e < E; ++e) fold(u, v[u].v[e], counts(e, skip[u]));
                    }
                }
                for (; q < uend; q += G) {
                    if constexpr (MODE == 0) fold(0, load_one(p + w.off), true);
                    else {
                        const int skip = MODE >= 2 ? skipped(w.k) : 0;
                        const pack<In, E> v = load_pack<In, E>(p + w.off - skip);
#pragma unroll
                        for (int e = 0; e < E; ++e) fold(0, v.v[e], counts(e, skip));
                    }
                    w.advance();
                }
                if constexpr (SQ) {
                    if (cnt > 0) {
                        const SA t1 = (s1[0] + s1[1]) + (s1[2] + s1[3]), t2 = (s2[0] + s2[1]) + (s2[2] + s2[3]);
                        const SA n = (SA)cnt;
                        const SA m2 = t2 - t1 * (t1 / n);
                        acc[0] = Acc{n, (sk - a.mean) + t1 / n, m2 < SA(0) ? SA(0) : m2};
                    }
                }
            };
            if (!L.vec) walk(std::integral_constant<int, 0>{});
            else if (L.walk == 2) {
                if constexpr (E >= 4) walk(std::integral_constant<int, 3>{});
            }
            else if (c % E == 0) walk(std::integral_constant<int, 1>{});
            else walk(std::integral_constant<int, 2>{});
        }
        else {
            const In *p = src + so;
            if constexpr (P::kind == K_SQDEV1) {
                // (as above: the first element of the output's reduced space is the reference of the means)
                using A = acc_of_t<typename P::Out>;
                a = Acc{0, in_to_acc<In, typename P::Out>(load_one(p + red_offset(ix, 0))), 0};
                int64_t pos = beg + lane;
                if (pos < end) {
                    const A k = in_to_acc<In, typename P::Out>(load_one(p + red_offset(ix, pos)));
                    A s1 = 0, s2 = 0;
                    int64_t cnt = 0;
                    for (; pos < end; pos += G) {
                        const A d = in_to_acc<In, typename P::Out>(load_one(p + red_offset(ix, pos))) - k;
                        s1 += d;
                        s2 += d * d;
                        cnt += 1;
                    }
                    const A n = (A)cnt;
                    const A m2 = s2 - s1 * (s1 / n);
                    acc[0] = Acc{n, (k - a.mean) + s1 / n, m2 < A(0) ? A(0) : m2};
                }
            }
            else {
                for (int64_t pos = beg + lane; pos < end; pos += G)
                    acc[0] = P::combine(acc[0], P::pre(load_one(p + red_offset(ix, pos)), a));
            }
        }
    }
    Acc r = P::combine(P::combine(acc[0], acc[1]), P::combine(acc[2], acc[3]));
    static_assert(RED_U == 4);
    r = group_reduce<P>(r, whole_block, G);
    if (L.splits == 1) {
        if (active && lane == 0 && (!whole_block || threadIdx.x == 0)) dst[dof] = P::post(r, L.param);
        return;
    }
    // split mode (always a whole block per output): pass two by the last block to finish
    uint32_t zero = 0;
    if (threadIdx.x == 0) zero = slot_publish(partial + o * L.splits + split, r);
    if (!last_block_of_output(counters, L, o, split, zero)) return;
    Acc v = P::identity();
    for (int i = threadIdx.x; i < L.splits; i += blockDim.x) v = P::combine(v, slot_read(partial + o * L.splits + i));
    v = group_reduce<P>(v, true, G);
    if (threadIdx.x == 0) dst[dof] = P::post(v, L.param);
}

// ================================ cols kernel ================================================
// Iteration space: outer dims (0 .. nd_i-2) x inner dim (nd_i-1, src stride 1).
// Block = TY x TX threads, TX = 1 << g_log2 along the inner dim, TY = blockDim.x / TX rows,
// ecnt columns per thread (ecnt = 16 / sizeof(In) when L.vec, else 1).
// Linear block id = (outer * splits + split) * col_blocks + col_block.
// Partials are laid out [split][output] (coalesced to write and to fold).
// the planner makes blocks of at most 512 threads; the bound leaves the compiler 256 vector registers per
// lane, which the kernels of 1-byte inputs (16 columns per pack) need: under a bound of 1024 they spilled
constexpr int COLS_MAX_BLOCK = 512;

// elements of LDS scratch per thread, packs in flight per thread (LOADS) and accumulator sets they are
// folded into (U): wide inputs keep 4 packs in flight with a set each; 1- and 2-byte inputs, whose packs
// hold 8 or 16 columns, keep 8 in flight (the rows of a block are only 512 bytes wide, so the loads in
// flight are what feeds the memory system: bool 16384^2 summed down its columns ran at 29 % of the HBM
// rate with 2) and fold them into one set, which the registers still hold
template <class In> struct cols_cfg {
    static constexpr int E = 16 / (int)sizeof(In);
    static constexpr int U = E >= 8 ? 1 : 4;
    static constexpr int LOADS = E >= 8 ? 8 : 4;
};

// a cast between integer types that also compiles (and is never executed) where one side is not an integer: the
// narrow accumulation of red_cols_kernel sits in a lambda whose body is checked for every policy
template <class To, class From> DPX_D To int_cast(From x)
{
    if constexpr (std::is_integral_v<To> && std::is_integral_v<From>) return (To)x;
    else return To{};
}

// combines acc over the TY thread rows of the block; result valid for ty == 0
template <class P, int E> DPX_D void cols_block_combine(typename P::Acc (&v)[E], typename P::Acc *sm, int tx, int ty,
                                                        int TX, int TY)
{
    if (TY == 1) return;
    __syncthreads(); // sm may still be read by a previous call
    // place e of all threads side by side: neighbouring lanes then touch neighbouring words (thread by thread, 16
    // 64-bit sums per thread put the lanes of a wave 128 bytes apart, all on the same banks)
    const int NT = TX * TY;
#pragma unroll
    for (int e = 0; e < E; ++e) sm[e * NT + threadIdx.x] = v[e];
    __syncthreads();
    if (ty == 0) {
        for (int y = 1; y < TY; ++y)
#pragma unroll
            for (int e = 0; e < E; ++e) v[e] = P::combine(v[e], sm[e * NT + y * TX + tx]);
    }
}

// WALK: the rows of the reduced space are found by RedWalker (several reduced dims) and the inner iteration dim
// may have any src stride (L.istep; not 1: single elements, L.vec == 0)
template <class P, bool WALK = false>
__global__ __launch_bounds__(COLS_MAX_BLOCK) void red_cols_kernel(RedIndex ix, RedLaunch L,
                                                                 const typename P::In *src, typename P::Out *dst,
                                                                 Slot<typename P::Acc> *partial,
                                                                 const typename P::Aux *aux, unsigned *counters)
{
    using In = typename P::In;
    using Acc = typename P::Acc;
    constexpr int E = cols_cfg<In>::E;
    constexpr int U = cols_cfg<In>::U;
    constexpr int LOADS = cols_cfg<In>::LOADS;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    Acc *sm = reinterpret_cast<Acc *>(smem_raw);
    const int TX = 1 << L.g_log2, TY = (int)blockDim.x >> L.g_log2;
    const int tx = threadIdx.x & (TX - 1), ty = threadIdx.x >> L.g_log2;
    int64_t b = blockIdx.x;
    const int64_t cb = b % L.col_blocks;
    b /= L.col_blocks;
    const int split = (int)(b % L.splits);
    const int64_t outer = b / L.splits;
    const int ecnt = L.vec ? E : 1;
    const int64_t col_first = (cb * TX + tx) * ecnt;
    const bool active = col_first < L.inner;
    // The pack that would cross the end of a row is moved back so that it ends with the row; its first `back`
    // places belong to the thread before.  (Read element by element instead, one row at a time, that one thread
    // was a chain of dependent round trips as long as its column: 16384 x 16383 floats summed down the columns took
    // 369 us, 16384 x 16384 158 us.)  Rows shorter than a pack keep the element-wise form.
    const int back = (L.vec && active && col_first + E > L.inner && L.inner >= E) ? (int)(col_first + E - L.inner) : 0;
    const int64_t col0 = col_first - back;
    // L.walk == 2: every other column of a matrix.  The lines are read whole (L.inner is their length, 2 x
    // columns - 1; L.istep is not used): place e of a thread's pack is column (col0 + e) / 2 of the view when
    // col0 + e is even and nothing otherwise
    const bool half = WALK && L.walk == 2;
    auto has_out = [&](int e) {
        return e < ecnt && e >= back && col0 + e < L.inner && !(half && ((col0 + e) & 1));
    };
    auto out_col = [&](int e) { return half ? (col0 + e) >> 1 : col0 + e; };

    Acc acc[U][E];
#pragma unroll
    for (int u = 0; u < U; ++u)
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
    if (active) {
        typename P::AuxAcc a[E];
#pragma unroll
        for (int e = 0; e < E; ++e) a[e] = P::aux_identity();
        if constexpr (P::has_aux) {
#pragma unroll
            for (int e = 0; e < E; ++e)
                if (has_out(e)) a[e] = P::load_aux(aux + ao + out_col(e) * ix.aux_str[last]);
        }
        const In *p = src + so + col0 * ((WALK && !half) ? L.istep : 1);
        const int64_t beg = (int64_t)split * L.chunk;
        const int64_t end = (beg + L.chunk < L.n) ? beg + L.chunk : L.n;
        int64_t r = beg + ty;
        RedWalker w;
        if constexpr (WALK) w.start(L, r, TY);
        // offset of this thread's next row (each call moves on by TY rows)
        auto next_row = [&](int64_t row) {
            if constexpr (WALK) {
                const int64_t off = w.off;
                w.advance();
                return off;
            }
            else return row * L.rstride;
        };
        if (L.vec) {
            // the pack that holds the end of a row is read element by element: its own copy of the
            // loops, so the loads of the usual case stay free of branches
            auto walk = [&](auto whole_tag) {
                constexpr bool WHOLE = decltype(whole_tag)::value;
                auto load = [&](const In *q) {
                    if constexpr (WHOLE) return load_pack<In, E>(q);
                    else {
                        pack<In, E> t;
#pragma unroll
                        for (int e = 0; e < E; ++e) t.v[e] = load_one(q + ((col0 + e < L.inner) ? e : 0));
                        return t;
                    }
                };
                // the element-wise form keeps one pack in flight: its LOADS x E separate loads and their
                // addresses would set the register count of the whole kernel (and spill for 1-byte inputs)
                constexpr int NL = WHOLE ? LOADS : 1;
                if constexpr (P::kind == K_SQDEV1) {
                    // one-pass squared deviations down the columns, as in red_rows_kernel: per column, sums of d
                    // and d^2 with d = x - k, k the first row this thread meets; means relative to row 0 of the
                    // reduced space (offset 0), which every thread row and block of a column reads alike.  (Places
                    // of a pack that are no column of the view carry numbers nobody reads.)
                    using A = acc_of_t<typename P::Out>;
                    {
                        const pack<In, E> v0 = load(p);
#pragma unroll
                        for (int e = 0; e < E; ++e) a[e] = Acc{0, in_to_acc<In, typename P::Out>(v0.v[e]), 0};
                    }
                    if (r < end) {
                        A k[E], s1[E], s2[E];
                        {
                            int64_t off_k = r * L.rstride;
                            if constexpr (WALK) off_k = w.off; // (the row is met again below: d = 0)
                            const pack<In, E> vk = load(p + off_k);
#pragma unroll
                            for (int e = 0; e < E; ++e) {
                                k[e] = in_to_acc<In, typename P::Out>(vk.v[e]);
                                s1[e] = s2[e] = A(0);
                            }
                        }
                        int64_t cnt = 0;
                        auto take = [&](const pack<In, E> &v) {
#pragma unroll
                            for (int e = 0; e < E; ++e) {
                                const A d = in_to_acc<In, typename P::Out>(v.v[e]) - k[e];
                                s1[e] += d;
                                s2[e] += d * d;
                            }
                        };
                        if constexpr (WHOLE && sizeof(In) <= 2) {
                            // 1- and 2-byte inputs: a round's packs are sent for before the round in hand is taken (the
                            // loop of the sums below, see there: 64 to 128 elements a round at five double-precision
                            // instructions each otherwise pass with nothing in flight).  Unlike the sums, whose arithmetic
                            // is next to nothing, this loop wants whole rounds in flight: float16 16384 x 32768 with 8
                            // packs loaded and then taken 38 % of the HBM rate, 2 + 2 in flight 57 %, 4 + 4: 72 %, 8 + 8: 74 %.
                            static_assert(sizeof(In) * E == 16);
                            constexpr int H = E >= 16 ? 4 : 8;
                            u32x4 va[H], vb[H];
                            auto send_for = [&](u32x4(&d)[H], int64_t row) {
#pragma unroll
                                for (int u = 0; u < H; ++u) d[u] = load_words16(p + next_row(row + u * TY));
                                asm volatile("" ::: "memory");
                            };
                            auto take_words = [&](u32x4(&d)[H]) {
#pragma unroll
                                for (int u = 0; u < H; ++u) {
                                    union {
                                        u32x4 r;
                                        pack<In, E> p;
                                    } c;
                                    c.r = d[u];
                                    asm volatile("" : "+v"(c.r));
                                    take(c.p);
                                }
                                cnt += H;
                            };
                            if (r + (H - 1) * TY < end) {
                                send_for(va, r);
                                while (r + (3 * H - 1) * TY < end) {
                                    send_for(vb, r + H * TY);
                                    take_words(va);
                                    send_for(va, r + 2 * H * TY);
                                    take_words(vb);
                                    r += 2 * H * TY;
                                }
                                take_words(va);
                                r += H * TY;
                            }
                        }
                        else {
                            for (; r + (NL - 1) * TY < end; r += NL * TY) {
                                pack<In, E> v[NL];
#pragma unroll
                                for (int u = 0; u < NL; ++u) v[u] = load(p + next_row(r + u * TY));
#pragma unroll
                                for (int u = 0; u < NL; ++u) take(v[u]);
                                cnt += NL;
                            }
                        }
                        for (; r < end; r += TY) {
                            take(load(p + next_row(r)));
                            cnt += 1;
                        }
                        const A n = (A)cnt;
#pragma unroll
                        for (int e = 0; e < E; ++e) {
                            const A m2 = s2[e] - s1[e] * (s1[e] / n);
                            acc[0][e] = Acc{n, (k[e] - a[e].mean) + s1[e] / n, m2 < A(0) ? A(0) : m2};
                        }
                    }
                    return;
                }
                // 1- and 2-byte inputs, whose packs hold 16 or 8 columns: two packs are sent for before the two in
                // hand are taken apart and added up.  A block of these kernels has a CU to itself, its waves in step,
                // and the 30 to 130 vector instructions a pair of packs costs otherwise pass with nothing in flight;
                // more than two pairs in flight are slower again (int8 summed down the columns of 2^30 bytes, 8 packs
                // loaded and then added up: 65 - 72 % of the HBM rate over the shapes; 8 + 8 in flight 69 - 81;
                // 2 + 2: 73 - 83).
                // Sums and counts of integers into wider integers (NARROW) add up 16384 rows of a thread at a time
                // in 32 bits, an element by one dot-product instruction, before they move on to the wide accumulators.
                constexpr bool PIPE = WHOLE && sizeof(In) <= 2;
                constexpr bool NARROW = PIPE && sizeof(Acc) >= 4 && std::is_integral_v<Acc> && !P::has_aux &&
                                        (P::kind == K_SUM || P::kind == K_COUNT_NONZERO);
                if constexpr (PIPE) {
                    using A32 = std::conditional_t<std::is_signed_v<Acc>, int32_t, uint32_t>;
                    constexpr int H = 2, ROUNDS = 16384 / H;
                    [[maybe_unused]] A32 n32[NARROW ? U : 1][NARROW ? E : 1];
                    if constexpr (NARROW) {
#pragma unroll
                        for (int u = 0; u < U; ++u)
#pragma unroll
                            for (int e = 0; e < E; ++e) n32[u][e] = 0;
                    }
                    // (the packs cross the loop's back edge as the words that were loaded: carried as elements, each
                    // in a register of its own, they are taken apart where they are loaded, which waits for them there)
                    static_assert(sizeof(In) * E == 16);
                    u32x4 va[H], vb[H];
                    int round = 0;
                    auto send_for = [&](u32x4(&d)[H], int64_t row) {
#pragma unroll
                        for (int u = 0; u < H; ++u) d[u] = load_words16(p + next_row(row + u * TY));
                        asm volatile("" ::: "memory"); // (the loads stay in front of the arithmetic that follows)
                    };
                    auto add_up = [&](u32x4(&d)[H]) {
#pragma unroll
                        for (int u = 0; u < H; ++u) {
                            union {
                                u32x4 r;
                                pack<In, E> p;
                            } c;
                            c.r = d[u];
                            asm volatile("" : "+v"(c.r)); // (taken apart here, not where it is loaded)
                            if constexpr (!NARROW) {
#pragma unroll
                                for (int e = 0; e < E; ++e)
                                    acc[u % U][e] = P::combine(acc[u % U][e], P::pre(c.p.v[e], a[e]));
                                continue;
                            }
                            // an element into its sum by one dot-product instruction (the word times a word with a one
                            // in the element's place); counts and bools first turn each element into 0 or 1
                            constexpr bool ZERO_ONE = P::kind == K_COUNT_NONZERO || is_bool_v<In>;
                            constexpr bool SIGNED = std::is_signed_v<In> && !ZERO_ONE;
#pragma unroll
                            for (int i = 0; i < (NARROW ? 4 : 0); ++i) {
                                uint32_t w = c.r[i];
                                if constexpr (sizeof(In) == 1) {
                                    if constexpr (ZERO_ONE) w = ((((w & 0x7f7f7f7fu) + 0x7f7f7f7fu) | w) >> 7) & 0x01010101u;
#pragma unroll
                                    for (int b = 0; b < 4; ++b) {
                                        A32 &t = n32[u % U][4 * i + b];
                                        if constexpr (SIGNED) t = (A32)__builtin_amdgcn_sdot4((int)w, 1 << (8 * b), (int)t, false);
                                        else t = (A32)__builtin_amdgcn_udot4(w, 1u << (8 * b), (uint32_t)t, false);
                                    }
                                }
                                else {
                                    typedef short s16x2 __attribute__((ext_vector_type(2)));
                                    typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
                                    if constexpr (ZERO_ONE) w = ((((w & 0x7fff7fffu) + 0x7fff7fffu) | w) >> 15) & 0x00010001u;
#pragma unroll
                                    for (int b = 0; b < 2; ++b) {
                                        A32 &t = n32[u % U][2 * i + b];
                                        union {
                                            uint32_t w;
                                            s16x2 s;
                                            u16x2 u;
                                        } x, m;
                                        x.w = w;
                                        m.w = 1u << (16 * b);
                                        if constexpr (SIGNED) t = (A32)__builtin_amdgcn_sdot2(x.s, m.s, (int)t, false);
                                        else t = (A32)__builtin_amdgcn_udot2(x.u, m.u, (uint32_t)t, false);
                                    }
                                }
                            }
                        }
                    };
                    auto move_on = [&](bool last) {
                        if constexpr (!NARROW) return;
                        if (++round >= ROUNDS || last) {
#pragma unroll
                            for (int u = 0; u < U; ++u)
#pragma unroll
                                for (int e = 0; e < E; ++e) {
                                    acc[u][e] = P::combine(acc[u][e], int_cast<Acc>(n32[u][e]));
                                    n32[u][e] = 0;
                                }
                            round = 0;
                        }
                    };
                    // Two halves change places, so that no register is moved (a move waits for its load), and the
                    // loop holds no load under a condition and no exit between its halves (either makes the compiler
                    // wait for loads in flight that it cannot tell apart): it runs while three more halves exist.
                    if (r + (H - 1) * TY < end) {
                        send_for(va, r);
                        while (r + (3 * H - 1) * TY < end) {
                            send_for(vb, r + H * TY);
                            add_up(va);
                            move_on(false);
                            send_for(va, r + 2 * H * TY);
                            add_up(vb);
                            move_on(false);
                            r += 2 * H * TY;
                        }
                        add_up(va);
                        move_on(false);
                        r += H * TY;
                    }
                    // what is left, fewer than 2 H rows: the sums send for them together, as zeros where there is no
                    // row (the others leave them to the loop at the end, one round trip each)
                    if constexpr (NARROW) {
                        for (int part = 0; part < 2; ++part) {
#pragma unroll
                            for (int u = 0; u < H; ++u) {
                                va[u] = u32x4{0, 0, 0, 0};
                                if (r + u * TY < end) va[u] = load_words16(p + next_row(r + u * TY));
                            }
                            add_up(va);
                            r += H * TY;
                        }
                        move_on(true);
                    }
                }
                // (not after the loop above, which leaves fewer than a round's rows: this one's element-wise
                // temporaries would set the kernel's register count)
                if constexpr (!PIPE) {
                    for (; r + (NL - 1) * TY < end; r += NL * TY) {
                        pack<In, E> v[NL];
#pragma unroll
                        for (int u = 0; u < NL; ++u) v[u] = load(p + next_row(r + u * TY));
#pragma unroll
                        for (int u = 0; u < NL; ++u)
#pragma unroll
                            for (int e = 0; e < E; ++e) acc[u % U][e] = P::combine(acc[u % U][e], P::pre(v[u].v[e], a[e]));
                    }
                }
                for (; r < end; r += TY) {
                    pack<In, E> v = load(p + next_row(r));
#pragma unroll
                    for (int e = 0; e < E; ++e) acc[0][e] = P::combine(acc[0][e], P::pre(v.v[e], a[e]));
                }
            };
            if (col0 + E <= L.inner) walk(std::true_type{});
            else walk(std::false_type{});
        }
        else if constexpr (P::kind == K_SQDEV1) {
            // the same with one column per thread (columns at a stride, rows shorter than a pack)
            using A = acc_of_t<typename P::Out>;
            a[0] = Acc{0, in_to_acc<In, typename P::Out>(load_one(p)), 0};
            if (r < end) {
                int64_t off_k = r * L.rstride;
                if constexpr (WALK) off_k = w.off;
                const A k = in_to_acc<In, typename P::Out>(load_one(p + off_k));
                A s1[2] = {A(0), A(0)}, s2[2] = {A(0), A(0)};
                int64_t cnt = 0;
                for (; r + (LOADS - 1) * TY < end; r += LOADS * TY) {
                    In v[LOADS];
#pragma unroll
                    for (int u = 0; u < LOADS; ++u) v[u] = load_one(p + next_row(r + u * TY));
#pragma unroll
                    for (int u = 0; u < LOADS; ++u) {
                        const A d = in_to_acc<In, typename P::Out>(v[u]) - k;
                        s1[u & 1] += d;
                        s2[u & 1] += d * d;
                    }
                    cnt += LOADS;
                }
                for (; r < end; r += TY) {
                    const A d = in_to_acc<In, typename P::Out>(load_one(p + next_row(r))) - k;
                    s1[0] += d;
                    s2[0] += d * d;
                    cnt += 1;
                }
                const A t1 = s1[0] + s1[1], t2 = s2[0] + s2[1], n = (A)cnt;
                const A m2 = t2 - t1 * (t1 / n);
                acc[0][0] = Acc{n, (k - a[0].mean) + t1 / n, m2 < A(0) ? A(0) : m2};
            }
        }
        else {
            for (; r + (LOADS - 1) * TY < end; r += LOADS * TY) {
                In v[LOADS];
#pragma unroll
                for (int u = 0; u < LOADS; ++u) v[u] = load_one(p + next_row(r + u * TY));
#pragma unroll
                for (int u = 0; u < LOADS; ++u) acc[u % U][0] = P::combine(acc[u % U][0], P::pre(v[u], a[0]));
            }
            for (; r < end; r += TY) acc[0][0] = P::combine(acc[0][0], P::pre(load_one(p + next_row(r)), a[0]));
        }
    }
    Acc v[E];
#pragma unroll
    for (int e = 0; e < E; ++e) {
        v[e] = acc[0][e];
#pragma unroll
        for (int u = 1; u < U; ++u) v[e] = P::combine(v[e], acc[u][e]);
    }
    cols_block_combine<P, E>(v, sm, tx, ty, TX, TY);
    // results of v: as 16-byte stores when every place of the pack is a column and they lie side by side (few rows
    // and many columns write as much as they read: one store per column and lane, 16 bytes apart, was the slower half)
    auto write_out = [&]() {
        using Out = typename P::Out;
        if (ecnt == E && back == 0 && !half && col0 + E <= L.inner && ix.dst_str[last] == 1) {
            constexpr int PER16 = 16 / (int)sizeof(Out) < 1 ? 1 : 16 / (int)sizeof(Out);
            constexpr int CE = PER16 < E ? PER16 : E;
            Out *q = dst + dof + col0;
#pragma unroll
            for (int e0 = 0; e0 < E; e0 += CE) {
                pack<Out, CE> o;
#pragma unroll
                for (int j = 0; j < CE; ++j) o.v[j] = P::post(v[e0 + j], L.param);
                // (results wider than the inputs: a lane's stores are pieces of a line that only meet in the L2, so
                // they must not bypass it: int8 summed into int64 ran twice as long with streaming stores)
                store_pack<Out, CE, sizeof(Out) <= sizeof(In)>(q + e0, o);
            }
            return;
        }
#pragma unroll
        for (int e = 0; e < E; ++e)
            if (has_out(e)) dst[dof + out_col(e) * ix.dst_str[last]] = P::post(v[e], L.param);
    };
    // flat output index of this thread's column e
    const int64_t out_base = half ? outer * ((L.inner + 1) >> 1) : outer * L.inner;
    auto slot_of = [&](int e) { return out_base + out_col(e); };
    if (L.splits == 1) {
        if (ty == 0 && active) write_out();
        return;
    }
    uint32_t zero = 0;
    if (ty == 0 && active) {
#pragma unroll
        for (int e = 0; e < E; ++e)
            if (has_out(e)) zero |= slot_publish(partial + (int64_t)split * L.m + slot_of(e), v[e]);
    }
    if (!last_block_of(counters + (outer * L.col_blocks + cb), L.splits, zero)) return;
    // pass two.  Threads side by side along the block's outputs, so that a wave reads consecutive partials (the
    // thread that owns a pack would read its E partials 4 or 8 bytes at a time, lanes a pack of partials apart:
    // 128 blocks of 1001 int8 columns summed into int64 spent 70 of their 104 us here).  With fewer outputs than
    // threads, `parts` threads share a column: thread (part, c) folds splits part, part + parts, ... in
    // increasing order, then the parts are folded in order through LDS.
    const int NT = (int)blockDim.x, t = (int)threadIdx.x;
    const int64_t pcol0 = cb * TX * ecnt; // first place of the block along the rows, and how many it has
    const int64_t pcols = (L.inner - pcol0 < (int64_t)TX * ecnt) ? L.inner - pcol0 : (int64_t)TX * ecnt;
    const int64_t ocol0 = half ? pcol0 >> 1 : pcol0; // the same in columns of the output
    const int ncol = (int)(half ? (pcols + 1) >> 1 : pcols);
    const Slot<Acc> *part0 = partial + out_base + ocol0;
    auto fold_from = [&](int c, int first, int step) {
        constexpr int FU = sizeof(Acc) > 8 ? 8 : 16; // partials in flight: a thread's share is a chain of round trips
        Acc r = P::identity();
        int g = first;
        for (; g + (FU - 1) * step < L.splits; g += FU * step) {
            Acc w[FU];
#pragma unroll
            for (int u = 0; u < FU; ++u) w[u] = slot_read(part0 + (int64_t)(g + u * step) * L.m + c);
#pragma unroll
            for (int u = 0; u < FU; ++u) r = P::combine(r, w[u]);
        }
        for (; g < L.splits; g += step) r = P::combine(r, slot_read(part0 + (int64_t)g * L.m + c));
        return r;
    };
    if (ncol >= NT) { // (a single thread row of wide packs: more outputs than threads)
        for (int c = t; c < ncol; c += NT)
            dst[dof + (ocol0 + c) * ix.dst_str[last]] = P::post(fold_from(c, 0, 1), L.param);
        return;
    }
    const int parts = NT / ncol;
    Acc r = P::identity();
    if (t < parts * ncol) r = fold_from(t % ncol, t / ncol, parts);
    __syncthreads(); // sm may still be read by the combine above
    if (t < parts * ncol) sm[t] = r;
    __syncthreads();
    if (t < ncol) {
        for (int q = 1; q < parts; ++q) r = P::combine(r, sm[q * ncol + t]);
        dst[dof + (ocol0 + t) * ix.dst_str[last]] = P::post(r, L.param);
    }
}

// ================================ flat columns kernel =========================================
// A row-major matrix with short rows (a row shorter than 512 bytes), reduced over its rows: the
// column kernel would leave most lanes of a wave without a pack.  Here the matrix is one flat
// stream of 16-byte packs and element i belongs to column i mod inner.  A block has T threads with
// T * E a multiple of inner, thread t takes packs t, t + T, t + 2T, ... of the block's rows, so the
// columns of its E accumulators never change.  Block b owns rows [b * chunk, (b + 1) * chunk).
// LDS holds T * E accumulators, entry k of column k mod inner; a tree over k folds them to one
// entry per column.  With several blocks the last one (ticket) folds the per-block partials,
// laid out [block][column], the same way.  L.m = L.inner = columns, L.n = rows, L.splits = blocks.
template <class P> DPX_D void flat_fold_columns(typename P::Acc *sm, int count, int inner)
{
    const int J = (count + inner - 1) / inner;
    int s = 1;
    while (2 * s < J) s *= 2; // the largest power of two below J (1 when J <= 2)
    if (J < 2) s = 0;
    for (; s >= 1; s >>= 1) {
        __syncthreads();
        const int lim = (count - s * inner < s * inner) ? count - s * inner : s * inner;
        for (int k = threadIdx.x; k < lim; k += (int)blockDim.x) sm[k] = P::combine(sm[k], sm[k + s * inner]);
    }
    __syncthreads();
}

template <class P>
__global__ __launch_bounds__(256) void red_flat_kernel(RedIndex ix, RedLaunch L, const typename P::In *src,
                                                      typename P::Out *dst, Slot<typename P::Acc> *partial,
                                                      const typename P::Aux *aux, unsigned *counters)
{
    using In = typename P::In;
    using Acc = typename P::Acc;
    constexpr int E = cols_cfg<In>::E;
    constexpr int U = E >= 8 ? 2 : (E >= 4 ? 4 : 8); // packs in flight per thread
    extern __shared__ __align__(16) unsigned char smem_raw[];
    Acc *sm = reinterpret_cast<Acc *>(smem_raw);
    const int T = (int)blockDim.x, t = (int)threadIdx.x;
    const int inner = (int)L.inner;
    const int split = (int)blockIdx.x;
    const int64_t row0 = (int64_t)split * L.chunk;
    const int64_t rows = (row0 + L.chunk < L.n) ? L.chunk : L.n - row0;
    const int64_t elems = rows * inner;
    const int64_t packs = elems / E;
    const In *p = src + row0 * inner;

    typename P::AuxAcc a[E];
#pragma unroll
    for (int e = 0; e < E; ++e) a[e] = P::aux_identity();
    if constexpr (P::has_aux) {
        int c = (int)(((int64_t)t * E) % inner);
#pragma unroll
        for (int e = 0; e < E; ++e) {
            a[e] = P::load_aux(aux + (int64_t)c * ix.aux_str[0]);
            c = (c + 1 == inner) ? 0 : c + 1;
        }
    }
    Acc acc[U][E];
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
        for (int e = 0; e < E; ++e) acc[u][e] = P::identity();
    int64_t q = t;
    for (; q + (int64_t)(U - 1) * T < packs; q += (int64_t)U * T) {
        pack<In, E> v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = load_pack<In, E>(p + (q + (int64_t)u * T) * E);
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int e = 0; e < E; ++e) acc[u][e] = P::combine(acc[u][e], P::pre(v[u].v[e], a[e]));
    }
    for (; q < packs; q += T) {
        const pack<In, E> v = load_pack<In, E>(p + q * E);
#pragma unroll
        for (int e = 0; e < E; ++e) acc[0][e] = P::combine(acc[0][e], P::pre(v.v[e], a[e]));
    }
#pragma unroll
    for (int e = 0; e < E; ++e) {
        Acc r = acc[0][e];
#pragma unroll
        for (int u = 1; u < U; ++u) r = P::combine(r, acc[u][e]);
        sm[t * E + e] = r;
    }
    __syncthreads();
    // the elements after the last whole pack of the block (fewer than E): entry k of the table has
    // the column of every flat position congruent to k modulo T * E
    const int tail = (int)(elems - packs * E);
    if (t < tail) {
        const int64_t i = packs * E + t;
        const int k = (int)(i % ((int64_t)T * E));
        typename P::AuxAcc ax = P::aux_identity();
        if constexpr (P::has_aux) ax = P::load_aux(aux + (int64_t)(k % inner) * ix.aux_str[0]);
        sm[k] = P::combine(sm[k], P::pre(load_one(p + i), ax));
    }
    flat_fold_columns<P>(sm, T * E, inner);
    if (L.splits == 1) {
        for (int c = t; c < inner; c += T) dst[(int64_t)c * ix.dst_str[0]] = P::post(sm[c], L.param);
        return;
    }
    uint32_t zero = 0;
    for (int c = t; c < inner; c += T) zero |= slot_publish(partial + (int64_t)split * inner + c, sm[c]);
    if (!last_block_of(counters, L.splits, zero)) return;
    if (inner > T) {
        // more columns than threads (1-byte elements, rows of 257 to 511 bytes): a thread folds whole
        // columns, blocks in index order
        for (int c = t; c < inner; c += T) {
            Acc v = P::identity();
            for (int g = 0; g < L.splits; ++g) v = P::combine(v, slot_read(partial + (int64_t)g * inner + c));
            dst[(int64_t)c * ix.dst_str[0]] = P::post(v, L.param);
        }
        return;
    }
    // the last block: thread t < parts * inner folds blocks part, part + parts, ... of column t mod inner
    const int parts = T / inner;
    Acc v = P::identity();
    if (t < parts * inner) {
        constexpr int FU = 8;
        const int c = t % inner, part = t / inner;
        int g = part;
        for (; g + (FU - 1) * parts < L.splits; g += FU * parts) {
            Acc w[FU];
#pragma unroll
            for (int u = 0; u < FU; ++u) w[u] = slot_read(partial + (int64_t)(g + u * parts) * inner + c);
#pragma unroll
            for (int u = 0; u < FU; ++u) v = P::combine(v, w[u]);
        }
        for (; g < L.splits; g += parts) v = P::combine(v, slot_read(partial + (int64_t)g * inner + c));
    }
    __syncthreads(); // every thread has read its column results of the first fold
    if (t < parts * inner) sm[t] = v;
    flat_fold_columns<P>(sm, parts * inner, inner);
    for (int c = t; c < inner; c += T) dst[(int64_t)c * ix.dst_str[0]] = P::post(sm[c], L.param);
}

// ================================ short rows kernel ===========================================
// A row-major matrix with rows of at most 256 bytes, reduced along its rows (one result per row:
// row norms of points, softmax statistics over a few classes).  With a lane or two per row the
// rows kernel issues 16-byte loads a row pitch apart, which the memory pipeline serves badly, and
// keeps few bytes in flight.  Here a block takes R consecutive rows, i.e. R * n contiguous
// elements, reads them as one flat stream of packs (all loads of a thread issued before the
// first use, up to 8 per thread), spreads the elements into LDS rows of an odd word pitch, and
// thread r then folds rows r, r + 256, ... from LDS (conflict-free across r) in element order.
// L.chunk = R, at most 2048.
constexpr int SROW_LDS_BYTES = 32768;
// elements per LDS row for an element size: the row padded to a whole and odd number of words
// (8- and 16-byte elements: an odd number of elements)
DPX_HD constexpr int srow_pitch_for(int n, int size)
{
    if (size >= 4) return n | 1;
    const int per_word = 4 / size;
    return (((n + per_word - 1) / per_word) | 1) * per_word;
}
template <class In> DPX_HD constexpr int srow_pitch(int n) { return srow_pitch_for(n, (int)sizeof(In)); }

template <class P>
__global__ __launch_bounds__(256) void red_short_rows_kernel(RedIndex ix, RedLaunch L, const typename P::In *src,
                                                            typename P::Out *dst, const typename P::Aux *aux)
{
    using In = typename P::In;
    using Acc = typename P::Acc;
    constexpr int E = 16 / (int)sizeof(In);
    constexpr int MAXP = SROW_LDS_BYTES / 16 / 256; // packs per thread: 8
    extern __shared__ __align__(16) unsigned char smem_raw[];
    In *sm = reinterpret_cast<In *>(smem_raw);
    const int t = (int)threadIdx.x;
    const uint32_t n = (uint32_t)L.n;
    const int pitch = srow_pitch<In>((int)n);
    const int64_t row0 = (int64_t)blockIdx.x * L.chunk;
    const int R = (int)((row0 + L.chunk < L.m) ? L.chunk : L.m - row0);
    const uint32_t elems = (uint32_t)R * n;
    const uint32_t packs = elems / E;
    const In *p = src + row0 * n;
    pack<In, E> v[MAXP];
#pragma unroll
    for (int k = 0; k < MAXP; ++k) {
        const uint32_t q = (uint32_t)t + (uint32_t)k * 256u;
        if (q < packs) v[k] = load_pack<In, E>(p + (int64_t)q * E);
    }
#pragma unroll
    for (int k = 0; k < MAXP; ++k) {
        const uint32_t q = (uint32_t)t + (uint32_t)k * 256u;
        if (q < packs) {
            uint32_t r = (q * E) / n, c = q * E - r * n;
#pragma unroll
            for (int e = 0; e < E; ++e) {
                sm[r * pitch + c] = v[k].v[e];
                if (++c == n) {
                    c = 0;
                    ++r;
                }
            }
        }
    }
    { // the elements after the last whole pack (fewer than E)
        const uint32_t i = packs * E + (uint32_t)t;
        if (i < elems) {
            const uint32_t r = i / n;
            sm[r * pitch + (i - r * n)] = load_one(p + i);
        }
    }
    __syncthreads();
    for (int r = t; r < R; r += 256) { // very short rows: several rows per thread
        const int64_t o = row0 + r;
        typename P::AuxAcc a = P::aux_identity();
        if constexpr (P::has_aux) a = P::load_aux(aux + o * ix.aux_str[0]);
        const In *row = sm + r * pitch;
        Acc acc = P::identity();
        for (uint32_t j = 0; j < n; ++j) acc = P::combine(acc, P::pre(row[j], a));
        dst[o * ix.dst_str[0]] = P::post(acc, L.param);
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

// Folds (value, position) pairs like group_reduce; result valid in lane 0 / thread 0.
template <bool IS_MAX, class VT> DPX_D void arg_group_reduce(VT &best, int64_t &bidx, bool whole_block, int G)
{
    const int wl = whole_block ? 64 : G;
    for (int off = wl >> 1; off > 0; off >>= 1) {
        const VT ov = shfl_down_any(best, off);
        const int64_t oi = shfl_down_any(bidx, off);
        arg_merge<IS_MAX, VT>(best, bidx, ov, oi);
    }
    if (whole_block) {
        __shared__ VT smv[16];
        __shared__ int64_t smi[16];
        __syncthreads();
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
}

// Result of a search as it is stored.  A NaN-ignoring search reads NaN as the infinity that loses, so
// an all-NaN run and a run whose extreme is that infinity look alike; when the caller asks for it
// (L.mark_fill) both are reported as -1 - index, and the caller tells them apart.
template <class T> DPX_D int64_t arg_result(const RedLaunch &L, int64_t idx, value_of_t<T> best)
{
    if constexpr (is_nanskip<T>::value) {
        using V = value_of_t<T>;
        const V inf = (V)__builtin_inff();
        const V fill = is_nanskip<T>::is_max ? -inf : inf;
        if (L.mark_fill && best == fill) return -1 - idx;
    }
    return idx;
}

// Position = index along the reduced run.  Linear block id = oblock * splits + split, lanes
// per output as in red_rows_kernel; partial (value, position) pairs laid out [output][split].
template <class T, bool IS_MAX, bool CONTIG>
__global__ __launch_bounds__(1024) void arg_rows_kernel(RedLaunch L, const T *src, int64_t *dst, Slot<T> *pval,
                                                       Slot<int64_t> *pidx, unsigned *counters, RedIndex ix)
{
    using VT = value_of_t<T>;
    constexpr int E = 16 / (int)sizeof(T);
    const int G = 1 << L.g_log2;
    const bool whole_block = G == (int)blockDim.x;
    // (32-bit: the grid has fewer than 2^32 blocks)
    const uint32_t ob32 = (L.splits == 1) ? blockIdx.x : blockIdx.x / (uint32_t)L.splits;
    const int64_t oblock = ob32;
    const int split = (int)(blockIdx.x - ob32 * (uint32_t)L.splits);
    const int lane = threadIdx.x & (G - 1);
    const int64_t o = whole_block ? oblock : oblock * (blockDim.x >> L.g_log2) + (threadIdx.x >> L.g_log2);
    const bool active = o < L.m;

    VT best{};
    int64_t bidx = ARG_NONE;
    int64_t so = 0, dof = 0, ao = 0;
    if (active) {
        iter_offsets(ix, L, o, so, dof, ao);
        const int64_t beg = (int64_t)split * L.chunk;
        const int64_t end = (beg + L.chunk < L.n) ? beg + L.chunk : L.n;
        const T *p = src + so;
        if constexpr (CONTIG) {
            uint32_t bl = 0; // position relative to beg; chunk < 2^32 by construction
            bool have = false;
            if (L.vec) {
                const int64_t vend = beg + ((end - beg) / E) * E;
                const int64_t step = (int64_t)G * E;
                int64_t pos = beg + (int64_t)lane * E;
                auto take = [&](const pack<T, E> &v, int64_t at) {
#pragma unroll
                    for (int e = 0; e < E; ++e) {
                        const VT x = to_value(v.v[e]);
                        if (arg_better<IS_MAX, VT>(x, best)) {
                            best = x;
                            bl = (uint32_t)(at + e - beg);
                        }
                    }
                };
                if (pos < vend) {
                    // the lane's first element seeds the running extremum; it comes with the first round of loads
                    // (read on its own ahead of them it was one more round trip to memory: short rows)
                    have = true;
                    pack<T, E> v[RED_U];
#pragma unroll
                    for (int u = 0; u < RED_U; ++u)
                        if (pos + u * step < vend) v[u] = load_pack<T, E>(p + pos + u * step);
                    best = to_value(v[0].v[0]);
                    bl = (uint32_t)(pos - beg);
#pragma unroll
                    for (int u = 0; u < RED_U; ++u)
                        if (pos + u * step < vend) take(v[u], pos + u * step);
                    pos += RED_U * step;
                }
                for (; pos + (RED_U - 1) * step < vend; pos += RED_U * step) {
                    pack<T, E> v[RED_U];
#pragma unroll
                    for (int u = 0; u < RED_U; ++u) v[u] = load_pack<T, E>(p + pos + u * step);
#pragma unroll
                    for (int u = 0; u < RED_U; ++u) take(v[u], pos + u * step);
                }
                for (; pos < vend; pos += step) take(load_pack<T, E>(p + pos), pos);
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
        else if (L.walk) {
            // as in red_rows_kernel; a lane meets its positions in increasing order, so a later value only
            // replaces the best one when it is better.  Positions are kept relative to the chunk's first one, in
            // 32 bits (the host keeps a chunk's positions below 2^32), and updated by selects: written as
            // branches, sixteen dependent ones per round of loads, the kernel ran at 65 % of the HBM rate
            const int64_t uend = (beg + L.chunk < L.units) ? beg + L.chunk : L.units;
            const int64_t c = L.inner;
            auto walk = [&](auto mode_tag) {
                constexpr int MODE = decltype(mode_tag)::value; // (mode 3: see red_rows_kernel)
                constexpr int UE = MODE == 0 ? 1 : (MODE == 3 ? E / 2 : E); // positions per unit
                const int64_t run = MODE == 3 ? (c + 1) / 2 : c;           // positions per run
                RedWalker w;
                int64_t q = beg + lane;
                w.start(L, q, G, run, UE, beg);
                const int64_t pbase = (beg / L.wd[2]) * run + (beg % L.wd[2]) * UE;
                const uint32_t c32 = (uint32_t)c; // (the host keeps run lengths below 2^31)
                auto skipped = [&](uint32_t k) {
                    const uint32_t rem = c32 - k * E;
                    return rem < (uint32_t)E ? E - (int)rem : 0;
                };
                // position of the first element of the unit the walker stands on, relative to pbase
                auto unit_rel = [&]() { return w.rel; };
                uint32_t bl = 0;
                const bool have = q < uend;
                if (have) {
                    best = to_value(load_one(p + w.off));
                    bl = unit_rel();
                }
                auto take = [&](VT x, bool counts, uint32_t rel) {
                    const bool better = counts & arg_better<IS_MAX, VT>(x, best);
                    best = better ? x : best;
                    bl = better ? rel : bl;
                };
                // `rel`: position of the element at place 0 of the pack as read (`skip` places early)
                auto take_pack = [&](const pack<T, E> &v, int skip, uint32_t rel) {
#pragma unroll
                    for (int e = 0; e < E; ++e) {
                        if constexpr (MODE == 3)
                            take(to_value(v.v[e]), e >= skip && ((e + skip) & 1) == 0, rel + (uint32_t)((e - skip) >> 1));
                        else take(to_value(v.v[e]), MODE != 2 || e >= skip, rel + e);
                    }
                };
                for (; q + (RED_U - 1) * (int64_t)G < uend; q += RED_U * (int64_t)G) {
                    uint32_t rel[RED_U];
                    if constexpr (MODE == 0) {
                        T v[RED_U];
#pragma unroll
                        for (int u = 0; u < RED_U; ++u) {
                            rel[u] = unit_rel();
                            v[u] = load_one(p + w.off);
                            w.advance();
                        }
#pragma unroll
                        for (int u = 0; u < RED_U; ++u) take(to_value(v[u]), true, rel[u]);
                    }
                    else {
                        pack<T, E> v[RED_U];
                        int skip[RED_U];
#pragma unroll
                        for (int u = 0; u < RED_U; ++u) {
                            skip[u] = MODE >= 2 ? skipped(w.k) : 0;
                            rel[u] = MODE == 3 ? unit_rel() : unit_rel() - skip[u];
                            v[u] = load_pack<T, E>(p + w.off - skip[u]);
                            w.advance();
                        }
#pragma unroll
                        for (int u = 0; u < RED_U; ++u) take_pack(v[u], skip[u], rel[u]);
                    }
                }
                for (; q < uend; q += G) {
                    if constexpr (MODE == 0) take(to_value(load_one(p + w.off)), true, unit_rel());
                    else {
                        const int skip = MODE >= 2 ? skipped(w.k) : 0;
                        take_pack(load_pack<T, E>(p + w.off - skip), skip, MODE == 3 ? unit_rel() : unit_rel() - skip);
                    }
                    w.advance();
                }
                if (have) bidx = pbase + bl;
            };
            if (!L.vec) walk(std::integral_constant<int, 0>{});
            else if (L.walk == 2) {
                if constexpr (E >= 4) walk(std::integral_constant<int, 3>{});
            }
            else if (c % E == 0) walk(std::integral_constant<int, 1>{});
            else walk(std::integral_constant<int, 2>{});
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
    arg_group_reduce<IS_MAX, VT>(best, bidx, whole_block, G);
    if (L.splits == 1) {
        if (active && lane == 0 && (!whole_block || threadIdx.x == 0)) dst[dof] = arg_result<T>(L, bidx, best);
        return;
    }
    uint32_t zero = 0;
    if (threadIdx.x == 0) {
        zero = slot_publish(pval + o * L.splits + split, to_storage<T>(best));
        zero |= slot_publish(pidx + o * L.splits + split, bidx);
    }
    if (!last_block_of_output(counters, L, o, split, zero)) return;
    best = VT{};
    bidx = ARG_NONE;
    for (int i = threadIdx.x; i < L.splits; i += blockDim.x)
        arg_merge<IS_MAX, VT>(best, bidx, to_value(slot_read(pval + o * L.splits + i)),
                              slot_read(pidx + o * L.splits + i));
    arg_group_reduce<IS_MAX, VT>(best, bidx, true, G);
    if (threadIdx.x == 0) dst[dof] = arg_result<T>(L, bidx, best);
}

// Column variant (reduced axis strided by L.rstride, outputs contiguous).  A thread owns the E
// adjacent columns of one 16-byte pack and walks down the reduced axis, TY thread rows apart;
// 256 threads per block; partials laid out [split][output].  Positions inside a chunk are kept
// in 32 bits (the host keeps chunks below 2^32 rows).
template <class T, bool IS_MAX>
__global__ __launch_bounds__(256) void arg_cols_kernel(RedIndex ix, RedLaunch L, const T *src, int64_t *dst,
                                                      Slot<T> *pval, Slot<int64_t> *pidx, unsigned *counters)
{
    using VT = value_of_t<T>;
    constexpr int E = 16 / (int)sizeof(T);
    constexpr int U = E >= 8 ? 8 : 4; // rows in flight per thread (see cols_cfg)
    // (position, value) of every place of every thread: sized by the launch (blockDim.x x E pairs; a block of one
    // wave that held the LDS of 256 threads left a CU room for 13 waves)
    extern __shared__ __align__(16) unsigned char smem_raw[];
    int64_t *smi = reinterpret_cast<int64_t *>(smem_raw);
    VT *smv = reinterpret_cast<VT *>(smem_raw + (size_t)blockDim.x * E * sizeof(int64_t));
    const int TX = 1 << L.g_log2, TYB = (int)blockDim.x >> L.g_log2;
    const int tx = threadIdx.x & (TX - 1), tyb = threadIdx.x >> L.g_log2;
    // obatch != 0 (short columns, many outer indices, one block per column block): the thread rows of a block are
    // consecutive outer indices and a thread walks its whole column, so nothing is combined in LDS.  Four thread rows
    // that shared columns of 32 rows spent more time meeting in LDS than reading (65536 x 32 x 128 floats along the
    // middle axis: 61 % of the HBM rate, 65536 x 64 x 64: 44 %).
    const bool batch = L.obatch != 0;
    const int TY = batch ? 1 : TYB, ty = batch ? 0 : tyb; // thread rows that share a column, and this thread's
    int64_t b = blockIdx.x;
    const int64_t cb = b % L.col_blocks;
    b /= L.col_blocks;
    const int split = (int)(b % L.splits);
    const int64_t outer = batch ? (b / L.splits) * TYB + tyb : b / L.splits;
    const int64_t col_first = (cb * TX + tx) * E;
    const bool active = col_first < L.inner && (!batch || outer < L.m / L.inner);
    // the pack that would cross the end of a row is moved back to end with it; its first `back` places belong
    // to the thread before (see red_cols_kernel)
    const int back = (active && col_first + E > L.inner && L.inner >= E) ? (int)(col_first + E - L.inner) : 0;
    const int64_t col0 = col_first - back;
    const bool whole = col0 + E <= L.inner;
    auto mine = [&](int e) { return e >= back && col0 + e < L.inner; };
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
    VT best[E];
    int64_t bidx[E];
#pragma unroll
    for (int e = 0; e < E; ++e) {
        best[e] = VT{};
        bidx[e] = ARG_NONE;
    }
    if (active) {
        const T *p = src + so + col0;
        const int64_t beg = (int64_t)split * L.chunk;
        const int64_t end = (beg + L.chunk < L.n) ? beg + L.chunk : L.n;
        int64_t r = beg + ty;
        uint32_t bl[E];
        const bool have = r < end;
        // the pack that holds the end of a row is read element by element, in its own copy of the loops
        auto walk = [&](auto whole_tag) {
            constexpr bool WHOLE = decltype(whole_tag)::value;
            auto load = [&](const T *q) {
                if constexpr (WHOLE) return load_pack<T, E>(q);
                else {
                    pack<T, E> t;
#pragma unroll
                    for (int e = 0; e < E; ++e) t.v[e] = load_one(q + ((col0 + e < L.inner) ? e : 0));
                    return t;
                }
            };
            auto take = [&](const pack<T, E> &v, int64_t row) {
#pragma unroll
                for (int e = 0; e < E; ++e) {
                    const VT x = to_value(v.v[e]);
                    if (arg_better<IS_MAX, VT>(x, best[e])) {
                        best[e] = x;
                        bl[e] = (uint32_t)(row - beg);
                    }
                }
            };
            constexpr int NL = WHOLE ? U : 1; // the element-wise form keeps one pack in flight (registers)
            if (have) {
                // The first row seeds the running extremum.  It comes with the first round of loads: read on its
                // own ahead of them it was one more round trip to memory, half as long again a life for a block
                // whose threads meet 8 rows (argmax along the middle axis of 65536 x 32 x 128 floats: 55 % of the
                // HBM rate where max ran at 77 %).
                pack<T, E> v[NL];
#pragma unroll
                for (int u = 0; u < NL; ++u)
                    if (r + u * TY < end) v[u] = load(p + (r + u * TY) * L.rstride);
#pragma unroll
                for (int e = 0; e < E; ++e) {
                    best[e] = to_value(v[0].v[e]);
                    bl[e] = (uint32_t)(r - beg);
                }
#pragma unroll
                for (int u = 1; u < NL; ++u)
                    if (r + u * TY < end) take(v[u], r + u * TY);
                r += NL * TY;
            }
            for (; r + (NL - 1) * TY < end; r += NL * TY) {
                pack<T, E> v[NL];
#pragma unroll
                for (int u = 0; u < NL; ++u) v[u] = load(p + (r + u * TY) * L.rstride);
#pragma unroll
                for (int u = 0; u < NL; ++u) take(v[u], r + u * TY);
            }
            if (r < end) { // fewer than NL rows are left: their loads go out together as well
                pack<T, E> v[NL];
#pragma unroll
                for (int u = 0; u < NL; ++u)
                    if (r + u * TY < end) v[u] = load(p + (r + u * TY) * L.rstride);
#pragma unroll
                for (int u = 0; u < NL; ++u)
                    if (r + u * TY < end) take(v[u], r + u * TY);
            }
        };
        if (whole) walk(std::true_type{});
        else walk(std::false_type{});
        if (have) {
#pragma unroll
            for (int e = 0; e < E; ++e) bidx[e] = beg + bl[e];
        }
    }
    auto combine_rows = [&]() {
        if (TY == 1) return;
        __syncthreads();
#pragma unroll
        for (int e = 0; e < E; ++e) {
            smv[threadIdx.x * E + e] = best[e];
            smi[threadIdx.x * E + e] = bidx[e];
        }
        __syncthreads();
        if (ty == 0)
            for (int y = 1; y < TY; ++y) {
#pragma unroll
                for (int e = 0; e < E; ++e)
                    arg_merge<IS_MAX, VT>(best[e], bidx[e], smv[(y * TX + tx) * E + e], smi[(y * TX + tx) * E + e]);
            }
    };
    auto write_out = [&]() {
        const int last = ix.nd_i - 1;
        int64_t *q = dst + dof + col0 * ix.dst_str[last];
        if constexpr (E >= 2) {
            if (whole && back == 0 && ix.dst_str[last] == 1) {
#pragma unroll
                for (int e = 0; e < E; e += 2) {
                    pack<int64_t, 2> t;
                    t.v[0] = arg_result<T>(L, bidx[e], best[e]);
                    t.v[1] = arg_result<T>(L, bidx[e + 1], best[e + 1]);
                    store_pack<int64_t, 2>(q + e, t);
                }
                return;
            }
        }
#pragma unroll
        for (int e = 0; e < E; ++e)
            if (mine(e)) q[e * ix.dst_str[last]] = arg_result<T>(L, bidx[e], best[e]);
    };
    combine_rows();
    const int64_t out0 = outer * L.inner + col0;
    if (L.splits == 1) {
        if (ty == 0 && active) write_out();
        return;
    }
    uint32_t zero = 0;
    if (ty == 0 && active) {
#pragma unroll
        for (int e = 0; e < E; ++e)
            if (mine(e)) {
                zero |= slot_publish(pval + (int64_t)split * L.m + out0 + e, to_storage<T>(best[e]));
                zero |= slot_publish(pidx + (int64_t)split * L.m + out0 + e, bidx[e]);
            }
    }
    // pass two, as in red_cols_kernel: threads side by side along the block's outputs read consecutive partial
    // pairs; with fewer outputs than threads, `parts` threads share a column and meet in LDS.  (arg_merge takes the
    // better value and, of equal ones, the smaller position: the order of the merges does not matter.)
    // With many blocks per output (tgroup != 0) the pass has two levels: the last block of every group of
    // RED_TGROUP splits folds the group's pairs and leaves the result in the place of the group's first split,
    // and the last of those blocks folds the groups' results.  One block folding 512 pairs per column took
    // 35 us of a 200 us launch (2^21 x 128 floats), a chain of 16 round trips to memory per thread.
    const int NT = (int)blockDim.x, t = (int)threadIdx.x;
    const int last = ix.nd_i - 1;
    const int64_t ocol0 = cb * TX * E;
    const int ncol = (int)((L.inner - ocol0 < (int64_t)TX * E) ? L.inner - ocol0 : (int64_t)TX * E);
    const int64_t slot0 = outer * L.inner + ocol0;
    // pairs first, first + step, ... of the `count` pairs of column c that stand `scale` splits apart from `base`
    auto fold_from = [&](int c, int base, int count, int scale, int first, int step, VT &b, int64_t &bi) {
        constexpr int FU = sizeof(T) > 8 ? 8 : 16; // pairs in flight: a thread's share is a chain of round trips
        b = VT{};
        bi = ARG_NONE;
        auto at = [&](int g) { return (int64_t)(base + g * scale) * L.m + slot0 + c; };
        int g = first;
        for (; g + (FU - 1) * step < count; g += FU * step) {
            T wv[FU];
            int64_t wi[FU];
#pragma unroll
            for (int u = 0; u < FU; ++u) {
                wv[u] = slot_read(pval + at(g + u * step));
                wi[u] = slot_read(pidx + at(g + u * step));
            }
#pragma unroll
            for (int u = 0; u < FU; ++u) arg_merge<IS_MAX, VT>(b, bi, to_value(wv[u]), wi[u]);
        }
        for (; g < count; g += step)
            arg_merge<IS_MAX, VT>(b, bi, to_value(slot_read(pval + at(g))), slot_read(pidx + at(g)));
    };
    // every column of the block folded over those pairs; emit(c, value, position) in one thread per column
    auto fold_block = [&](int base, int count, int scale, auto &&emit) {
        VT fb{};
        int64_t fi = ARG_NONE;
        if (ncol >= NT) {
            for (int c = t; c < ncol; c += NT) {
                fold_from(c, base, count, scale, 0, 1, fb, fi);
                emit(c, fb, fi);
            }
            return;
        }
        const int parts = NT / ncol;
        if (t < parts * ncol) fold_from(t % ncol, base, count, scale, t / ncol, parts, fb, fi);
        __syncthreads(); // the LDS may still be read by an earlier combine
        if (t < parts * ncol) {
            smv[t] = fb;
            smi[t] = fi;
        }
        __syncthreads();
        if (t < ncol) {
            for (int q = 1; q < parts; ++q) arg_merge<IS_MAX, VT>(fb, fi, smv[q * ncol + t], smi[q * ncol + t]);
            emit(t, fb, fi);
        }
    };
    auto to_dst = [&](int c, VT fb, int64_t fi) {
        dst[dof + (ocol0 + c) * ix.dst_str[last]] = arg_result<T>(L, fi, fb);
    };
    unsigned *ticket = counters + (outer * L.col_blocks + cb);
    if (L.tgroup == 0) {
        if (!last_block_of(ticket, L.splits, zero)) return;
        fold_block(0, L.splits, 1, to_dst);
        return;
    }
    const int grp = split >> RED_TGROUP_LOG2, ngrp = (L.splits + RED_TGROUP - 1) >> RED_TGROUP_LOG2;
    const int g_first = grp << RED_TGROUP_LOG2;
    const int g_count = (L.splits - g_first < RED_TGROUP) ? L.splits - g_first : RED_TGROUP;
    unsigned *gticket = counters + RED_MAX_TICKETS + ((outer * L.col_blocks + cb) * ngrp + grp) * RED_GROUP_PITCH;
    if (!last_block_of(gticket, g_count, zero)) return;
    zero = 0;
    // (a thread overwrites the pair of the group's first split only after reading it: it is among those it folds)
    fold_block(g_first, g_count, 1, [&](int c, VT fb, int64_t fi) {
        zero |= slot_publish(pval + (int64_t)g_first * L.m + slot0 + c, to_storage<T>(fb));
        zero |= slot_publish(pidx + (int64_t)g_first * L.m + slot0 + c, fi);
    });
    if (!last_block_of(ticket, ngrp, zero)) return;
    fold_block(0, ngrp, RED_TGROUP, to_dst);
}

// Flat variant (see red_flat_kernel): the row of the extremum of every column of a row-major matrix whose rows
// are shorter than 512 bytes.  Thread t reads packs t, t + NT, ... of the block's rows, so element e of its packs
// stays in one column and moves down NT * E / inner rows per pack: a thread keeps, per column, the best value and
// how many rows below its first pack it stood (32 bits: the host keeps a block's rows below 2^32).  LDS holds
// NT * E (row, value) pairs, entry k of column k mod inner, folded by a tree; blocks leave (row, value) partials
// laid out [block][column] for the last one.
template <bool IS_MAX, class VT> DPX_D void arg_flat_fold(VT *smv, int64_t *smi, int count, int inner)
{
    const int J = (count + inner - 1) / inner;
    int s = 1;
    while (2 * s < J) s *= 2;
    if (J < 2) s = 0;
    for (; s >= 1; s >>= 1) {
        __syncthreads();
        const int lim = (count - s * inner < s * inner) ? count - s * inner : s * inner;
        for (int k = threadIdx.x; k < lim; k += (int)blockDim.x)
            arg_merge<IS_MAX, VT>(smv[k], smi[k], smv[k + s * inner], smi[k + s * inner]);
    }
    __syncthreads();
}

template <class T, bool IS_MAX>
__global__ __launch_bounds__(256) void arg_flat_kernel(RedIndex ix, RedLaunch L, const T *src, int64_t *dst,
                                                      Slot<T> *pval, Slot<int64_t> *pidx, unsigned *counters)
{
    using VT = value_of_t<T>;
    constexpr int E = 16 / (int)sizeof(T);
    constexpr int U = E >= 8 ? 2 : (E >= 4 ? 4 : 8); // packs in flight per thread
    extern __shared__ __align__(16) unsigned char smem_raw[];
    const int NT = (int)blockDim.x, t = (int)threadIdx.x;
    int64_t *smi = reinterpret_cast<int64_t *>(smem_raw);
    VT *smv = reinterpret_cast<VT *>(smem_raw + (size_t)NT * E * sizeof(int64_t));
    const int inner = (int)L.inner;
    const int split = (int)blockIdx.x;
    const int64_t row0 = (int64_t)split * L.chunk;
    const int64_t rows = (row0 + L.chunk < L.n) ? L.chunk : L.n - row0;
    const int64_t elems = rows * inner;
    const int64_t packs = elems / E;
    const T *p = src + row0 * inner;
    const uint32_t rstep = (uint32_t)(NT * E / inner); // rows between a thread's consecutive packs

    VT best[E];
    uint32_t bl[E];
    const bool have = t < packs;
#pragma unroll
    for (int e = 0; e < E; ++e) {
        best[e] = VT{};
        bl[e] = 0;
    }
    if (have) { // the first pack seeds the running extrema (and is then visited once more)
        const pack<T, E> v = load_pack<T, E>(p + (int64_t)t * E);
#pragma unroll
        for (int e = 0; e < E; ++e) best[e] = to_value(v.v[e]);
    }
    auto take = [&](const pack<T, E> &v, uint32_t below) {
#pragma unroll
        for (int e = 0; e < E; ++e) {
            const VT x = to_value(v.v[e]);
            const bool better = arg_better<IS_MAX, VT>(x, best[e]);
            best[e] = better ? x : best[e];
            bl[e] = better ? below : bl[e];
        }
    };
    uint32_t cur = 0; // rows below the thread's first pack
    int64_t q = t;
    for (; q + (int64_t)(U - 1) * NT < packs; q += (int64_t)U * NT) {
        pack<T, E> v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = load_pack<T, E>(p + (q + (int64_t)u * NT) * E);
#pragma unroll
        for (int u = 0; u < U; ++u) take(v[u], cur + (uint32_t)u * rstep);
        cur += (uint32_t)U * rstep;
    }
    for (; q < packs; q += NT) {
        take(load_pack<T, E>(p + q * E), cur);
        cur += rstep;
    }
#pragma unroll
    for (int e = 0; e < E; ++e) {
        smv[t * E + e] = best[e];
        smi[t * E + e] = have ? row0 + (t * E + e) / inner + bl[e] : ARG_NONE;
    }
    __syncthreads();
    // the elements after the last whole pack of the block (fewer than E), as in red_flat_kernel
    const int tail = (int)(elems - packs * E);
    if (t < tail) {
        const int64_t i = packs * E + t;
        const int k = (int)(i % ((int64_t)NT * E));
        arg_merge<IS_MAX, VT>(smv[k], smi[k], to_value(load_one(p + i)), row0 + i / inner);
    }
    arg_flat_fold<IS_MAX, VT>(smv, smi, NT * E, inner);
    if (L.splits == 1) {
        for (int c = t; c < inner; c += NT) dst[(int64_t)c * ix.dst_str[0]] = arg_result<T>(L, smi[c], smv[c]);
        return;
    }
    uint32_t zero = 0;
    for (int c = t; c < inner; c += NT) {
        zero |= slot_publish(pval + (int64_t)split * inner + c, to_storage<T>(smv[c]));
        zero |= slot_publish(pidx + (int64_t)split * inner + c, smi[c]);
    }
    if (!last_block_of(counters, L.splits, zero)) return;
    if (inner > NT) { // more columns than threads (1-byte elements): a thread folds whole columns
        for (int c = t; c < inner; c += NT) {
            VT b{};
            int64_t bi = ARG_NONE;
            for (int g = 0; g < L.splits; ++g)
                arg_merge<IS_MAX, VT>(b, bi, to_value(slot_read(pval + (int64_t)g * inner + c)),
                                      slot_read(pidx + (int64_t)g * inner + c));
            dst[(int64_t)c * ix.dst_str[0]] = arg_result<T>(L, bi, b);
        }
        return;
    }
    // thread t < parts * inner folds blocks part, part + parts, ... of column t mod inner
    const int parts = NT / inner;
    VT b{};
    int64_t bi = ARG_NONE;
    if (t < parts * inner) {
        constexpr int FU = 4;
        const int c = t % inner, part = t / inner;
        int g = part;
        for (; g + (FU - 1) * parts < L.splits; g += FU * parts) {
            T wv[FU];
            int64_t wi[FU];
#pragma unroll
            for (int u = 0; u < FU; ++u) {
                wv[u] = slot_read(pval + (int64_t)(g + u * parts) * inner + c);
                wi[u] = slot_read(pidx + (int64_t)(g + u * parts) * inner + c);
            }
#pragma unroll
            for (int u = 0; u < FU; ++u) arg_merge<IS_MAX, VT>(b, bi, to_value(wv[u]), wi[u]);
        }
        for (; g < L.splits; g += parts)
            arg_merge<IS_MAX, VT>(b, bi, to_value(slot_read(pval + (int64_t)g * inner + c)),
                                  slot_read(pidx + (int64_t)g * inner + c));
    }
    __syncthreads(); // every thread has read its column results of the first fold
    if (t < parts * inner) {
        smv[t] = b;
        smi[t] = bi;
    }
    arg_flat_fold<IS_MAX, VT>(smv, smi, parts * inner, inner);
    for (int c = t; c < inner; c += NT) dst[(int64_t)c * ix.dst_str[0]] = arg_result<T>(L, smi[c], smv[c]);
}

// Short rows variant (see red_short_rows_kernel): position of the extremum of each row of a
// row-major matrix with rows of at most 256 bytes (the predicted class of each sample).
template <class T, bool IS_MAX>
__global__ __launch_bounds__(256) void arg_short_rows_kernel(RedIndex ix, RedLaunch L, const T *src, int64_t *dst)
{
    using VT = value_of_t<T>;
    constexpr int E = 16 / (int)sizeof(T);
    constexpr int MAXP = SROW_LDS_BYTES / 16 / 256;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T *sm = reinterpret_cast<T *>(smem_raw);
    const int t = (int)threadIdx.x;
    const uint32_t n = (uint32_t)L.n;
    const int pitch = srow_pitch<T>((int)n);
    const int64_t row0 = (int64_t)blockIdx.x * L.chunk;
    const int R = (int)((row0 + L.chunk < L.m) ? L.chunk : L.m - row0);
    const uint32_t elems = (uint32_t)R * n;
    const uint32_t packs = elems / E;
    const T *p = src + row0 * n;
    pack<T, E> v[MAXP];
#pragma unroll
    for (int k = 0; k < MAXP; ++k) {
        const uint32_t q = (uint32_t)t + (uint32_t)k * 256u;
        if (q < packs) v[k] = load_pack<T, E>(p + (int64_t)q * E);
    }
#pragma unroll
    for (int k = 0; k < MAXP; ++k) {
        const uint32_t q = (uint32_t)t + (uint32_t)k * 256u;
        if (q < packs) {
            uint32_t r = (q * E) / n, c = q * E - r * n;
#pragma unroll
            for (int e = 0; e < E; ++e) {
                sm[r * pitch + c] = v[k].v[e];
                if (++c == n) {
                    c = 0;
                    ++r;
                }
            }
        }
    }
    {
        const uint32_t i = packs * E + (uint32_t)t;
        if (i < elems) {
            const uint32_t r = i / n;
            sm[r * pitch + (i - r * n)] = load_one(p + i);
        }
    }
    __syncthreads();
    for (int r = t; r < R; r += 256) {
        const T *row = sm + r * pitch;
        VT best = to_value(row[0]);
        uint32_t bj = 0;
        for (uint32_t j = 1; j < n; ++j) {
            const VT x = to_value(row[j]);
            if (arg_better<IS_MAX, VT>(x, best)) {
                best = x;
                bj = j;
            }
        }
        dst[(row0 + r) * ix.dst_str[0]] = arg_result<T>(L, (int64_t)bj, best);
    }
}

} // namespace dpx
