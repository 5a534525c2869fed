// Element types, conversions and 128-bit memory accessors shared by all kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>
#include "../../include/dpnp_amd.h"

namespace dpx {

#define DPX_HD __host__ __device__ __forceinline__
#define DPX_D __device__ __forceinline__

using half_t = _Float16;

// Storage of a NumPy bool: one byte, any set bit reads as true, written as 0/1
// (convert_impl, libtensor/include/utils/type_utils.hpp:80-93).
struct bool_t {
    uint8_t v;
};

template <class R> struct cplx {
    R re, im;
};
using c64 = cplx<float>;
using c128 = cplx<double>;

template <class T> struct is_cplx : std::false_type {};
template <class R> struct is_cplx<cplx<R>> : std::true_type {};
template <class T> inline constexpr bool is_cplx_v = is_cplx<T>::value;
template <class T> inline constexpr bool is_bool_v = std::is_same_v<T, bool_t>;
template <class T>
inline constexpr bool is_fp_v = std::is_same_v<T, half_t> || std::is_same_v<T, float> ||
                                std::is_same_v<T, double>;
template <class T>
inline constexpr bool is_int_v = std::is_integral_v<T> && !std::is_same_v<T, bool>;
template <class T> inline constexpr bool is_sint_v = is_int_v<T> && std::is_signed_v<T>;
template <class T> inline constexpr bool is_uint_v = is_int_v<T> && std::is_unsigned_v<T>;
template <class T> inline constexpr bool is_real_v = is_int_v<T> || is_fp_v<T>;

template <class T> struct real_of {
    using type = T;
};
template <class R> struct real_of<cplx<R>> {
    using type = R;
};
template <class T> using real_of_t = typename real_of<T>::type;

// dtype id <-> C++ type
template <int ID> struct type_of;
template <> struct type_of<DPX_BOOL> { using type = bool_t; };
template <> struct type_of<DPX_INT8> { using type = int8_t; };
template <> struct type_of<DPX_UINT8> { using type = uint8_t; };
template <> struct type_of<DPX_INT16> { using type = int16_t; };
template <> struct type_of<DPX_UINT16> { using type = uint16_t; };
template <> struct type_of<DPX_INT32> { using type = int32_t; };
template <> struct type_of<DPX_UINT32> { using type = uint32_t; };
template <> struct type_of<DPX_INT64> { using type = int64_t; };
template <> struct type_of<DPX_UINT64> { using type = uint64_t; };
template <> struct type_of<DPX_HALF> { using type = half_t; };
template <> struct type_of<DPX_FLOAT> { using type = float; };
template <> struct type_of<DPX_DOUBLE> { using type = double; };
template <> struct type_of<DPX_CFLOAT> { using type = c64; };
template <> struct type_of<DPX_CDOUBLE> { using type = c128; };

template <class T> struct id_of;
#define DPX_ID_OF(T, ID) \
    template <> struct id_of<T> { static constexpr int value = ID; };
DPX_ID_OF(bool_t, DPX_BOOL)
DPX_ID_OF(int8_t, DPX_INT8)
DPX_ID_OF(uint8_t, DPX_UINT8)
DPX_ID_OF(int16_t, DPX_INT16)
DPX_ID_OF(uint16_t, DPX_UINT16)
DPX_ID_OF(int32_t, DPX_INT32)
DPX_ID_OF(uint32_t, DPX_UINT32)
DPX_ID_OF(int64_t, DPX_INT64)
DPX_ID_OF(uint64_t, DPX_UINT64)
DPX_ID_OF(half_t, DPX_HALF)
DPX_ID_OF(float, DPX_FLOAT)
DPX_ID_OF(double, DPX_DOUBLE)
DPX_ID_OF(c64, DPX_CFLOAT)
DPX_ID_OF(c128, DPX_CDOUBLE)
#undef DPX_ID_OF
template <class T> inline constexpr int id_of_v = id_of<T>::value;

template <class T> struct tag {
    using type = T;
};

// Calls f(tag<T>{}) for the element type with id dt; returns false for a bad id.
template <class F> inline bool for_dtype(int dt, F &&f)
{
    switch (dt) {
    case DPX_BOOL: f(tag<bool_t>{}); return true;
    case DPX_INT8: f(tag<int8_t>{}); return true;
    case DPX_UINT8: f(tag<uint8_t>{}); return true;
    case DPX_INT16: f(tag<int16_t>{}); return true;
    case DPX_UINT16: f(tag<uint16_t>{}); return true;
    case DPX_INT32: f(tag<int32_t>{}); return true;
    case DPX_UINT32: f(tag<uint32_t>{}); return true;
    case DPX_INT64: f(tag<int64_t>{}); return true;
    case DPX_UINT64: f(tag<uint64_t>{}); return true;
    case DPX_HALF: f(tag<half_t>{}); return true;
    case DPX_FLOAT: f(tag<float>{}); return true;
    case DPX_DOUBLE: f(tag<double>{}); return true;
    case DPX_CFLOAT: f(tag<c64>{}); return true;
    case DPX_CDOUBLE: f(tag<c128>{}); return true;
    default: return false;
    }
}

// ---- conversions (convert_impl, type_utils.hpp:64-117) --------------------

template <class To, class From> DPX_HD To convert(const From &v)
{
    if constexpr (std::is_same_v<To, From>) {
        return v;
    }
    else if constexpr (is_bool_v<To>) {
        if constexpr (is_cplx_v<From>)
            return bool_t{(uint8_t)((v.re != 0) || (v.im != 0))};
        else
            return bool_t{(uint8_t)(v != From(0))};
    }
    else if constexpr (is_bool_v<From>) {
        if constexpr (is_cplx_v<To>)
            return To{(real_of_t<To>)(v.v != 0 ? 1 : 0), (real_of_t<To>)0};
        else
            return (To)(v.v != 0 ? 1 : 0);
    }
    else if constexpr (is_cplx_v<From> && is_cplx_v<To>) {
        return To{(real_of_t<To>)v.re, (real_of_t<To>)v.im};
    }
    else if constexpr (is_cplx_v<From>) {
        return convert<To, real_of_t<From>>(v.re);
    }
    else if constexpr (is_cplx_v<To>) {
        return To{(real_of_t<To>)v, (real_of_t<To>)0};
    }
    else if constexpr (is_fp_v<From> && is_uint_v<To>) {
        // negative values wrap like two's complement: go through a signed type
        using mid_t = std::conditional_t<(sizeof(To) < 4), int32_t, int64_t>;
        return (v < From(0)) ? (To)(mid_t)v : (To)v;
    }
    else {
        return (To)v;
    }
}

// Value seen by the functors for a stored element: bool_t -> bool, else itself.
template <class T> struct value_of {
    using type = T;
};
template <> struct value_of<bool_t> {
    using type = bool;
};
// A floating element read as "NaN loses": NaN becomes -inf for a maximum search and +inf for a
// minimum search (nanargmax / nanargmin replace NaN this way before searching,
// dpnp/dpnp_iface_nanfunctions.py:195,279).
template <class T, bool IS_MAX> struct nanskip {
    T v;
};
template <class T> struct is_nanskip : std::false_type {};
template <class T, bool M> struct is_nanskip<nanskip<T, M>> : std::true_type {
    static constexpr bool is_max = M;
};
template <class T, bool M> struct value_of<nanskip<T, M>> {
    using type = T;
};
template <class T> using value_of_t = typename value_of<T>::type;

template <class T> DPX_HD value_of_t<T> to_value(const T &s)
{
    if constexpr (is_bool_v<T>)
        return s.v != 0;
    else if constexpr (is_nanskip<T>::value) {
        using V = value_of_t<T>;
        const V inf = (V)__builtin_inff();
        return (s.v != s.v) ? (is_nanskip<T>::is_max ? -inf : inf) : s.v;
    }
    else
        return s;
}
template <class T> DPX_HD T to_storage(const value_of_t<T> &v)
{
    if constexpr (is_bool_v<T>)
        return bool_t{(uint8_t)(v ? 1 : 0)};
    else if constexpr (is_nanskip<T>::value)
        return T{v};
    else
        return v;
}

// ---- N-byte memory accessors ------------------------------------------------
// Streaming kernels touch every byte once, so loads and stores carry the
// non-temporal hint (keeps L2/MALL from being churned; measured worth 5-8 % of
// HBM bandwidth on MI355X).

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// Register image of a pack.  The types carry alignment 1: global loads and stores of 4, 8 and 16
// bytes need no alignment on this hardware (the compiler emits the same full-width instruction), so
// packs may start at any element: rows of odd length, views that start at x[1:].  Measured on
// MI355X, fp32 add of 2^28 elements: 6.75 TB/s with 16-byte aligned operands, 5.65 TB/s with
// every operand off by one element - the rate of element-wise coalesced accesses, now reached
// from any layout whose inner stride is 1.
template <int BYTES> struct raw_of;
template <> struct raw_of<1> { typedef uint8_t type; };
template <> struct raw_of<2> { typedef uint16_t type __attribute__((aligned(1))); };
template <> struct raw_of<4> { typedef uint32_t type __attribute__((aligned(1))); };
template <> struct raw_of<8> { typedef u32x2 type __attribute__((aligned(1))); };
template <> struct raw_of<16> { typedef u32x4 type __attribute__((aligned(1))); };

template <class T, int N> struct alignas(sizeof(T) * N >= 16 ? 16 : sizeof(T) * N) pack {
    T v[N];
};

template <class T, int N, bool NT = true> DPX_D pack<T, N> load_pack(const T *p)
{
    static_assert(sizeof(T) * N <= 16);
    using raw_t = typename raw_of<sizeof(T) * N>::type;
    union {
        raw_t r;
        pack<T, N> p;
    } u;
    if constexpr (NT)
        u.r = __builtin_nontemporal_load(reinterpret_cast<const raw_t *>(p));
    else
        u.r = *reinterpret_cast<const raw_t *>(p);
    return u.p;
}
template <class T, int N, bool NT = true> DPX_D void store_pack(T *p, const pack<T, N> &v)
{
    static_assert(sizeof(T) * N <= 16);
    using raw_t = typename raw_of<sizeof(T) * N>::type;
    union {
        raw_t r;
        pack<T, N> p;
    } u;
    u.p = v;
    if constexpr (NT)
        __builtin_nontemporal_store(u.r, reinterpret_cast<raw_t *>(p));
    else
        *reinterpret_cast<raw_t *>(p) = u.r;
}

// 16 bytes as four words (for code that works on words whatever the element type)
template <bool NT = true> DPX_D u32x4 load_words16(const void *p)
{
    using raw_t = typename raw_of<16>::type;
    if constexpr (NT) return __builtin_nontemporal_load(reinterpret_cast<const raw_t *>(p));
    else return *reinterpret_cast<const raw_t *>(p);
}

// Called on a loaded pack where its elements are first used, after every load of the thread has
// been issued: the compiler then sees a use of all its bytes.  Without it, where only parts of
// the elements are used (int16 -> int8 needs the low bytes), the 16-byte load is split into one
// narrow load per element.  (Inside load_pack it would make every load wait for the one before.)
template <class T, int N> DPX_D void keep_whole(pack<T, N> &p)
{
    if constexpr (N > 1 && sizeof(T) * N >= 4) {
        using raw_t = typename raw_of<sizeof(T) * N>::type;
        union {
            raw_t r;
            pack<T, N> p;
        } u;
        u.p = p;
        asm("" : "+v"(u.r));
        p = u.p;
    }
}

template <class T> DPX_D T load_one(const T *p)
{
    return load_pack<T, 1, false>(p).v[0];
}

constexpr int cmax(int a, int b) { return a > b ? a : b; }
template <class... Ts> constexpr int max_sizeof()
{
    int m = 1;
    ((m = cmax(m, (int)sizeof(Ts))), ...);
    return m;
}

} // namespace dpx
