// Glue between the C entry points and the templated elementwise launcher.
#pragma once
#include "ew.hpp"
#include "host.hpp"
#include "ops.hpp"

namespace dpx {

int ew_validate(int nops, const dpx_array_view *const *views, int64_t &n);
void ew_export_plan(const EwPlan &pl, dpx_plan *out);

// views = inputs..., dst (already validated).  plan_out != nullptr: report only.
template <class Fn, class Out, class... Ins>
inline int run_ew(const Fn &fn, const dpx_array_view *const *views, hipStream_t stream,
                  dpx_plan *plan_out)
{
    EwPlan pl;
    ew_make_plan(pl, (int)sizeof...(Ins) + 1, views);
    hipError_t e = ew_launch<Fn, Out, Ins...>(fn, pl, views, stream, plan_out != nullptr);
    if (plan_out) {
        ew_export_plan(pl, plan_out);
        plan_out->vec = pl.vec || (pl.path == DPX_PATH_EW_ROWS) ? ew_traits<Out, Ins...>::E : 1;
        return DPX_OK;
    }
    return e == hipSuccess ? DPX_OK : fail_hip(e, "elementwise kernel launch");
}

// unary functions of doubles that cost enough vector instructions to pay for two packs per thread
template <class Op> struct op_two_packs : std::false_type {};
#define DPX_TWO_PACKS(OP) \
    template <> struct op_two_packs<OP> : std::true_type {};
DPX_TWO_PACKS(Expm1Op) DPX_TWO_PACKS(Log2Op) DPX_TWO_PACKS(SinhOp) DPX_TWO_PACKS(TanhOp)
// (log1p and the inverse hyperbolic functions: 60 to 90 instructions in one dependent chain per element)
DPX_TWO_PACKS(Log1pOp) DPX_TWO_PACKS(AsinhOp) DPX_TWO_PACKS(AcoshOp) DPX_TWO_PACKS(AtanhOp)
// (pow of doubles: a table look-up that waits for the base sits in every element's chain; a second pack per
// thread keeps the memory system busy meanwhile)
DPX_TWO_PACKS(PowOp)
// (sin, cos, tan of doubles: 45 to 60 instructions in one chain; sin 70-78 -> 82 %, cos 75-78 -> 82 %, tan 65 -> 69 % of
// the HBM rate with the second pack; log, log10, exp, erf, acos, atan gain nothing or lose a point)
DPX_TWO_PACKS(SinOp) DPX_TWO_PACKS(CosOp) DPX_TWO_PACKS(TanOp)
// (logaddexp and logaddexp2 of doubles, an exp and a log1p per element: 63-68 -> 70-75 %)
DPX_TWO_PACKS(LogaddexpOp) DPX_TWO_PACKS(Logaddexp2Op)
#undef DPX_TWO_PACKS
// ... and of floats (pow: its table look-up sits in every element's chain like the one of doubles)
template <class Op> struct op_two_packs_float : std::false_type {};
template <> struct op_two_packs_float<PowOp> : std::true_type {};
template <class Op, class T, class = void> struct op_two_phase : std::false_type {};
template <class Op, class T> struct op_two_phase<Op, T, std::enable_if_t<Op::template two_phase<T>>> : std::true_type {};
template <class Op, class T> struct UnaryFn {
    static constexpr bool two_packs = op_two_packs<Op>::value && std::is_same_v<T, double>;
    static constexpr bool two_phase = op_two_phase<Op, T>::value; // (see BinaryFn)
    static constexpr bool has_cheap = false;
    DPX_D auto operator()(V<T> x) const { return Op::template apply<T>(x); }
    DPX_D auto fast(V<T> x) const { return Op::template fast<T>(x); }
    DPX_D auto fixup(V<T> r, V<T> x) const { return Op::template fixup<T>(r, x); }
};
// An op may split its work in two phases for element type T (Op::two_phase<T>): fast(a, b) is
// straight-line code that gives the result or NaN where it does not apply, fixup(r, a, b) branches to the
// complete routine for those.  The contiguous kernel runs the first phase for all elements of a pack
// before the second, so that the chains of the elements interleave (see ew_contig_pack).  Such an op
// also names arguments with a cheap exact form (cheap_applies / cheap), which a wave takes alone when
// all its lanes have them.
template <class Op, class T> struct BinaryFn {
    static constexpr bool two_packs = (op_two_packs<Op>::value && std::is_same_v<T, double>) ||
                                      (op_two_packs_float<Op>::value && std::is_same_v<T, float>);
    static constexpr bool two_phase = op_two_phase<Op, T>::value;
    static constexpr bool has_cheap = true;
    DPX_D auto operator()(V<T> a, V<T> b) const { return Op::template apply<T>(a, b); }
    DPX_D auto fast(V<T> a, V<T> b) const { return Op::template fast<T>(a, b); }
    DPX_D auto fixup(V<T> r, V<T> a, V<T> b) const { return Op::template fixup<T>(r, a, b); }
    // arguments with a cheap exact form, taken when every lane of the wave has them
    DPX_D bool cheap_applies(V<T> a, V<T> b) const { return Op::template cheap_applies<T>(a, b); }
    DPX_D auto cheap(V<T> a, V<T> b) const { return Op::template cheap<T>(a, b); }
};
template <class Op, class T> struct rows2_enabled<UnaryFn<Op, T>> : std::true_type {};
template <class Op, class T> struct rows2_enabled<BinaryFn<Op, T>> : std::true_type {};
template <class Op, class T> struct outer_enabled<BinaryFn<Op, T>> : std::true_type {};
template <class Op, class T> struct straight_rows_enabled<BinaryFn<Op, T>> : std::true_type {};

} // namespace dpx
