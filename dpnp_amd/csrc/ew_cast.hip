// dpx_copy_cast: ti._copy_usm_ndarray_into_usm_ndarray
// (libtensor/source/copy_and_cast_usm_to_usm.cpp:137-216, kernels copy_and_cast.hpp:90-520):
// dst = convert(src) for every dtype pair, any strides.  Equal dtypes move raw
// bytes by size class.
#include "ew_dispatch.hpp"

namespace dpx {

template <class From, class To> struct CastFn {
    DPX_D V<To> operator()(V<From> x) const
    {
        return to_value(convert<To, From>(to_storage<From>(x)));
    }
};
template <class T> struct CopyFn {
    DPX_D T operator()(T x) const { return x; }
};

template <class F> static bool for_size_class(int bytes, F &&f)
{
    switch (bytes) {
    case 1: f(tag<uint8_t>{}); return true;
    case 2: f(tag<uint16_t>{}); return true;
    case 4: f(tag<uint32_t>{}); return true;
    case 8: f(tag<uint64_t>{}); return true;
    case 16: f(tag<c128>{}); return true;
    default: return false;
    }
}

static int copy_cast_call(const dpx_array_view *src, const dpx_array_view *dst, void *stream,
                          dpx_plan *plan_out)
{
    const dpx_array_view *views[2] = {src, dst};
    int64_t n = 0;
    if (int rc = ew_validate(2, views, n)) return rc;
    hipStream_t s = (hipStream_t)stream;
    int rc = DPX_ERR_NOT_IMPLEMENTED;
    if (src->dtype == dst->dtype) {
        for_size_class(itemsize_of(src->dtype), [&](auto t) {
            using T = typename decltype(t)::type;
            rc = run_ew<CopyFn<T>, T, T>({}, views, s, plan_out);
        });
        return rc;
    }
    for_dtype(src->dtype, [&](auto ft) {
        using From = typename decltype(ft)::type;
        for_dtype(dst->dtype, [&](auto tt) {
            using To = typename decltype(tt)::type;
            if constexpr (!std::is_same_v<From, To>)
                rc = run_ew<CastFn<From, To>, To, From>({}, views, s, plan_out);
        });
    });
    return rc;
}

} // namespace dpx

extern "C" int dpx_copy_cast(const dpx_array_view *src, const dpx_array_view *dst, void *stream)
{
    if (!dpx::view_ok(src) || !dpx::view_ok(dst))
        return dpx::fail(DPX_ERR_BAD_ARGUMENT, "malformed array descriptor");
    return dpx::copy_cast_call(src, dst, stream, nullptr);
}
