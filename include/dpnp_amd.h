/*
 * dpnp_amd.h -- C ABI of libdpnp_amd.so: the elementwise + axis-reduction hot
 * path of dpnp.tensor for AMD MI355X (gfx950).
 *
 * Every entry point replaces one family of pybind11 functions that the
 * reference's Python layer calls in the extension modules _tensor_impl,
 * _tensor_elementwise_impl and _tensor_reductions_impl.  The reference passes
 * usm_ndarray objects, a sycl::queue and a list of events and gets back a pair
 * of events; here the caller passes plain array descriptors and a hipStream_t
 * and gets back a status code.  Work is enqueued on the given (in-order)
 * stream and is asynchronous with respect to the host.
 *
 * Conventions
 *   - all array arguments are borrowed for the duration of the call; the
 *     caller keeps the device memory alive until the stream has passed the work;
 *   - `dst` is always allocated by the caller; the library allocates only
 *     scratch (partial results of multi-block reductions) from a grow-only,
 *     per-stream pool it owns, and four 16 MiB pinned host buffers per device
 *     for the host <-> device copies;
 *   - strides are in ELEMENTS (as usm_ndarray.strides), may be zero
 *     (broadcast) or negative; `data` points at the element with all indices 0;
 *   - a return value != DPX_OK leaves `dst` untouched (all validation happens
 *     before the first launch); dpx_last_error() gives the message of the last
 *     failure on the calling thread;
 *   - zero-size iteration spaces return DPX_OK without launching.
 *
 * citations: paths are relative to the reference tree, libtensor =
 * dpnp/tensor/libtensor.
 */
#ifndef DPNP_AMD_H
#define DPNP_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DPX_MAX_ND 12

/* dtype ids: same order as typenum_t,
 * libtensor/include/utils/type_dispatch_building.hpp:45-61 */
typedef enum dpx_dtype {
    DPX_BOOL = 0,
    DPX_INT8 = 1,
    DPX_UINT8 = 2,
    DPX_INT16 = 3,
    DPX_UINT16 = 4,
    DPX_INT32 = 5,
    DPX_UINT32 = 6,
    DPX_INT64 = 7,
    DPX_UINT64 = 8,
    DPX_HALF = 9,
    DPX_FLOAT = 10,
    DPX_DOUBLE = 11,
    DPX_CFLOAT = 12,
    DPX_CDOUBLE = 13,
    DPX_NUM_DTYPES = 14
} dpx_dtype;

/* flag bits: dpnp/include/usm_ndarray_constants.h:33-38 */
#define DPX_C_CONTIGUOUS 1
#define DPX_F_CONTIGUOUS 2
#define DPX_WRITABLE 4

/* array descriptor: the fields of the usm_ndarray struct the kernels glue
 * reads (dpnp/tensor/_usmarray.pxd:81-97, dpnp/include/dpnp4pybind11.hpp:402-447) */
typedef struct dpx_array_view {
    void *data;                  /* device pointer, element offset applied */
    int32_t nd;                  /* 0 <= nd <= DPX_MAX_ND */
    int32_t dtype;               /* dpx_dtype */
    int32_t flags;               /* DPX_C_CONTIGUOUS | DPX_F_CONTIGUOUS | DPX_WRITABLE */
    int32_t reserved;
    int64_t shape[DPX_MAX_ND];
    int64_t strides[DPX_MAX_ND]; /* in elements */
} dpx_array_view;

/* status codes; the Python shim maps them to the exception classes the
 * reference raises (libtensor/source/elementwise_functions/elementwise_functions.hpp:96-141,
 * libtensor/source/reductions/reduction_over_axis.hpp:188-238,456-458) */
typedef enum dpx_status {
    DPX_OK = 0,
    DPX_ERR_BAD_DTYPE = 1,       /* ValueError: dst dtype is not op's result type */
    DPX_ERR_SHAPE_MISMATCH = 2,  /* ValueError */
    DPX_ERR_RANK_MISMATCH = 3,   /* ValueError */
    DPX_ERR_NOT_WRITABLE = 4,    /* ValueError */
    DPX_ERR_OVERLAP = 5,         /* ValueError */
    DPX_ERR_NOT_AMPLE = 6,       /* ValueError */
    DPX_ERR_NOT_IMPLEMENTED = 7, /* RuntimeError */
    DPX_ERR_HIP = 8,             /* RuntimeError */
    DPX_ERR_BAD_ARGUMENT = 9     /* ValueError */
} dpx_status;

/* unary elementwise ops (one functor header each under
 * libtensor/include/kernels/elementwise_functions/) */
typedef enum dpx_unary_op {
    DPX_U_ABS = 0,
    DPX_U_NEGATIVE,
    DPX_U_POSITIVE,
    DPX_U_SQUARE,
    DPX_U_SQRT,
    DPX_U_EXP,
    DPX_U_LOG,
    DPX_U_ERF, /* dpnp/backend/kernels/elementwise_functions/erf.hpp:52-95 */
    DPX_U_SIN,
    DPX_U_COS,
    DPX_U_TAN,
    DPX_U_TANH,
    DPX_U_EXP2,
    DPX_U_EXPM1,
    DPX_U_LOG2,
    DPX_U_LOG10,
    DPX_U_LOG1P,
    DPX_U_RSQRT,
    DPX_U_CBRT,
    DPX_U_RECIPROCAL,
    DPX_U_FLOOR,
    DPX_U_CEIL,
    DPX_U_TRUNC,
    DPX_U_SIGN,
    DPX_U_ISNAN,
    DPX_U_ISINF,
    DPX_U_ISFINITE,
    DPX_U_LOGICAL_NOT,
    DPX_U_BITWISE_INVERT,
    DPX_U_SIGNBIT,
    DPX_U_ASIN,
    DPX_U_ACOS,
    DPX_U_ATAN,
    DPX_U_SINH,
    DPX_U_COSH,
    DPX_U_ASINH,
    DPX_U_ACOSH,
    DPX_U_ATANH,
    DPX_U_ROUND,
    DPX_U_CONJ,
    DPX_U_REAL,
    DPX_U_IMAG,
    DPX_U_PROJ,
    DPX_U_ANGLE,
    /* the reference's ufunc extension, dpnp/backend/extensions/ufunc/elementwise_functions/:
     * fabs.cpp, degrees.cpp, radians.cpp, sinc.cpp, spacing.cpp, bitwise_count.cpp,
     * erf_funcs.cpp, i0.cpp */
    DPX_U_FABS,
    DPX_U_DEGREES,
    DPX_U_RADIANS,
    DPX_U_SINC,
    DPX_U_SPACING,
    DPX_U_BITWISE_COUNT,
    DPX_U_ERFC,
    DPX_U_ERFCX,
    DPX_U_ERFINV,
    DPX_U_ERFCINV,
    DPX_U_I0,
    DPX_U_NUM_OPS
} dpx_unary_op;

typedef enum dpx_binary_op {
    DPX_B_ADD = 0,
    DPX_B_SUBTRACT,
    DPX_B_MULTIPLY,
    DPX_B_DIVIDE,
    DPX_B_BITWISE_AND,
    DPX_B_BITWISE_OR,
    DPX_B_BITWISE_XOR,
    DPX_B_EQUAL,
    DPX_B_NOT_EQUAL,
    DPX_B_LESS,
    DPX_B_LESS_EQUAL,
    DPX_B_GREATER,
    DPX_B_GREATER_EQUAL,
    DPX_B_MAXIMUM,
    DPX_B_MINIMUM,
    DPX_B_LOGICAL_AND,
    DPX_B_LOGICAL_OR,
    DPX_B_LOGICAL_XOR,
    DPX_B_POW,
    DPX_B_FLOOR_DIVIDE,
    DPX_B_REMAINDER,
    DPX_B_ATAN2,
    DPX_B_HYPOT,
    DPX_B_COPYSIGN,
    DPX_B_LEFT_SHIFT,
    DPX_B_RIGHT_SHIFT,
    DPX_B_LOGADDEXP,
    DPX_B_NEXTAFTER,
    /* the reference's ufunc extension, dpnp/backend/extensions/ufunc/elementwise_functions/:
     * fmax.cpp, fmin.cpp, fmod.cpp, logaddexp2.cpp, heaviside.cpp, gcd.cpp, lcm.cpp */
    DPX_B_FMAX,
    DPX_B_FMIN,
    DPX_B_FMOD,
    DPX_B_LOGADDEXP2,
    DPX_B_HEAVISIDE,
    DPX_B_GCD,
    DPX_B_LCM,
    DPX_B_NUM_OPS
} dpx_binary_op;

typedef enum dpx_reduce_op {
    DPX_R_SUM = 0,
    DPX_R_PROD,
    DPX_R_MAX,
    DPX_R_MIN,
    DPX_R_SUMSQDEV, /* sum(|x - aux|^2): second pass of var (also with a caller's mean, also of complex
                     * input: dpnp/dpnp_iface_statistics.py:1832-1869), see dpx_reduce */
    DPX_R_LOGSUMEXP, /* log(sum(exp(x))), libtensor/source/reductions/logsumexp.cpp */
    DPX_R_HYPOT,     /* sqrt(sum(x^2)) by pairwise hypot, libtensor/source/reductions/reduce_hypot.cpp */
    /* NaN-ignoring forms, floating inputs only.  The reference composes them from a masked copy
     * and the plain reduction (dpnp/dpnp_iface_nanfunctions.py:48-116,509-518,600-636,1318-1390);
     * here NaN elements are replaced as they are read.  NANMAX / NANMIN give NaN for a run that
     * holds nothing but NaN; NANCOUNT counts the elements that are not NaN (int64 result);
     * NANSUMSQDEV is SUMSQDEV with NaN elements contributing zero. */
    DPX_R_NANSUM,
    DPX_R_NANPROD,
    DPX_R_NANMAX,
    DPX_R_NANMIN,
    DPX_R_NANCOUNT,
    DPX_R_NANSUMSQDEV,
    /* truth-value reductions of any input type (an element is true when it is not zero):
     * ANY / ALL give bool (py_boolean_reduction, reduction_over_axis.hpp:1057-1303: tri._any,
     * tri._all), COUNT_NONZERO gives int64 (dpnp/tensor/_reduction.py:472-512) */
    DPX_R_ANY,
    DPX_R_ALL,
    DPX_R_COUNT_NONZERO,
    /* mean of the elements that are not NaN in one pass (sum and count travel together; NaN
     * for a run without a number): dpnp.nanmean, dpnp/dpnp_iface_nanfunctions.py:521-635 */
    DPX_R_NANMEAN,
    /* variance of the elements that are not NaN around the mean given in `aux`, in one pass:
     * sum of squared deviations / (count - ddof), NaN where count <= ddof (dpnp.nanvar,
     * dpnp/dpnp_iface_nanfunctions.py:1188-1391).  ddof is 0 through dpx_reduce; dpx_nan_variance
     * takes it as an argument. */
    DPX_R_NANVAR,
    /* sum((x - mean(x))^2) in ONE pass over the input, without a given mean: float32, float64 or an integer
     * type in, float64 out.  The reference's var reads the input for the mean, then again for the deviations
     * (dpnp/tensor/_statistical_functions.py:140-230: sum, divide, subtract, multiply, sum); this op carries
     * (count, mean, sum of squared deviations) triples and merges them pairwise.  Every layout dpx_reduce
     * takes for DPX_R_SUM is taken, at the rate of that sum: reduced runs that are contiguous in memory,
     * columns (outputs side by side, plain or at a stride), reduced dims that stay apart.  A thread sums
     * d and d^2 with d = x - k, k being the first element it meets; means travel relative to the first
     * element of the output's reduced space. */
    DPX_R_SQDEV_ONEPASS,
    DPX_R_NUM_OPS
} dpx_reduce_op;

typedef enum dpx_search_op {
    DPX_S_ARGMAX = 0,
    DPX_S_ARGMIN = 1,
    /* NaN elements never win (real floating inputs): dpnp.nanargmax / nanargmin,
     * dpnp/dpnp_iface_nanfunctions.py:119-284 */
    DPX_S_NANARGMAX = 2,
    DPX_S_NANARGMIN = 3,
    /* the same searches, for callers that must raise on an all-NaN run as dpnp.nanargmax does
     * (dpnp/dpnp_iface_nanfunctions.py:195-200) without a pass of their own over the input: a run
     * whose extreme equals the infinity that NaNs are read as (-inf for the maximum, +inf for the
     * minimum) is all-NaN or really has that extreme, and its result is stored as -1 - index.
     * No negative result: no all-NaN run, and every index is final. */
    DPX_S_NANARGMAX_MARKED = 4,
    DPX_S_NANARGMIN_MARKED = 5
} dpx_search_op;

/* which kernel family a call resolves to (reported by the dpx_*_plan queries;
 * lets the host-side dispatch be tested without a GPU) */
typedef enum dpx_path {
    DPX_PATH_NOOP = 0,          /* zero-size: nothing launched */
    DPX_PATH_EW_CONTIG = 1,     /* 1-D unit-stride, 128-bit accesses */
    DPX_PATH_EW_ROWS = 2,       /* N-D, threads vectorised along the inner dim (calls of two-operand functions that
                                   read nothing of the output's size, an outer sum, take blocks of 8 rows) */
    DPX_PATH_EW_ROWS2 = 3,      /* a stride-2 input, rows of whole waves: two rows per thread, reads fixed at compile time */
    DPX_PATH_EW_TILE = 4,       /* inputs contiguous along another dim than the output: LDS tile */
    DPX_PATH_RED_ROWS = 10,     /* reduced run contiguous: block or wave per output */
    DPX_PATH_RED_ROWS_SPLIT = 11, /* ... several blocks per output, folded by the last one */
    DPX_PATH_RED_COLS = 12,     /* outputs contiguous, reduced run strided */
    DPX_PATH_RED_COLS_SPLIT = 13, /* ... reduced run split over blocks, folded by the last one */
    DPX_PATH_RED_GENERIC = 14,  /* fully strided */
    DPX_PATH_RED_SMALL = 15,    /* tiny reduced run: one thread per output */
    DPX_PATH_RED_FLAT = 16,     /* row-major matrix with short rows reduced over its rows: a flat
                                   stream of 16-byte packs, column = position modulo row length */
    DPX_PATH_RED_SHORT_ROWS = 17 /* ... reduced along its rows: a block stages whole rows in LDS */
} dpx_path;

typedef struct dpx_plan {
    int32_t path;   /* dpx_path */
    int32_t nd;     /* dims left after stride collapsing (iteration space) */
    int32_t red_nd; /* collapsed reduction dims (reductions only) */
    int32_t vec;    /* elements per thread */
    int64_t shape[DPX_MAX_ND];
    int64_t strides[4][DPX_MAX_ND]; /* per operand, dst last */
    int64_t offsets[4];             /* element displacement per operand */
    int64_t grid[3];
    int32_t block;
    int32_t splits;        /* blocks cooperating on one output (reductions) */
    int64_t scratch_bytes; /* pool bytes the call would use */
} dpx_plan;

/* ---- library ---------------------------------------------------------- */

/* version of this ABI (bumped on incompatible change) */
int dpx_abi_version(void);
/* message of the last failing call on this thread ("" if none) */
const char *dpx_last_error(void);
/* number of bytes of element type dt, or -1 */
int dpx_dtype_itemsize(int dt);
/* release the scratch pool (device must be idle) */
int dpx_release_scratch(void);

/* ---- dtype queries ---------------------------------------------------- */

/* result dtype of op for the exact input dtype(s), or -1 when no kernel exists:
 * the _X_result_type functions, elementwise_functions.hpp:256-285,567-603 */
int dpx_unary_result_type(int op, int dt);
int dpx_binary_result_type(int op, int dt1, int dt2);
/* 1 if `lhs op= rhs` has a kernel (py_binary_inplace_ufunc's table,
 * elementwise_functions.hpp:612-650) */
int dpx_binary_inplace_supported(int op, int lhs_dt, int rhs_dt);
/* Result dtype of `op` for operands of two different dtypes when the conversion is folded into
 * the kernel (add, subtract, multiply, divide with one operand already of the result type:
 * float64 with float32/int32/int64/bool, float32 with bool/int8/uint8/int16; or with both
 * converted: float32 with int32/int64 gives float64), else -1.
 * No counterpart in the reference, whose kernels take same-dtype pairs and whose Python layer
 * casts the other operand into a temporary first (_find_buf_dtype2,
 * dpnp/tensor/_type_utils.py:389-485): a caller that has settled on "cast operand k (or both) to
 * T, then op" may call dpx_binary / dpx_binary_inplace with the original operands instead when this
 * returns T.  dpx_binary_result_type does not report these pairs. */
int dpx_binary_fused_cast_result_type(int op, int dtype1, int dtype2);
/* _sum_over_axis_dtype_supported & co., libtensor/source/reductions/sum.cpp:445-456 */
int dpx_reduce_dtype_supported(int op, int src_dt, int dst_dt);
/* argmax/argmin: any dtype -> int64, libtensor/source/reductions/argmax.cpp:77-127 */
int dpx_search_dtype_supported(int op, int src_dt, int dst_dt);

/* ---- host predicates --------------------------------------------------- */

/* ti._array_overlap, libtensor/include/utils/memory_overlap.hpp:56-113 */
int dpx_array_overlap(const dpx_array_view *a, const dpx_array_view *b);
/* ti._same_logical_tensors, memory_overlap.hpp:115-155 */
int dpx_same_logical(const dpx_array_view *a, const dpx_array_view *b);

/* ---- elementwise ------------------------------------------------------- */

/* py_unary_ufunc, elementwise_functions.hpp:77-251  (ti._exp, ti._sqrt, ...) */
int dpx_unary(int op, const dpx_array_view *src, const dpx_array_view *dst,
              void *stream);
/* py_binary_ufunc, elementwise_functions.hpp:305-563  (ti._add, ti._multiply, ...).
 * Inputs are already broadcast to dst's shape (zero strides). */
int dpx_binary(int op, const dpx_array_view *src1, const dpx_array_view *src2,
               const dpx_array_view *dst, void *stream);
/* py_binary_inplace_ufunc, elementwise_functions.hpp:612-804 (ti._add_inplace, ...) */
int dpx_binary_inplace(int op, const dpx_array_view *lhs,
                       const dpx_array_view *rhs, void *stream);
/* py_where, libtensor/source/where.cpp:74-247  (ti._where) */
int dpx_where(const dpx_array_view *cond, const dpx_array_view *x1,
              const dpx_array_view *x2, const dpx_array_view *dst,
              void *stream);
/* tei._divide_by_scalar, libtensor/source/elementwise_functions/true_divide.cpp:249-430;
 * the scalar is converted to dst's real type before the division */
int dpx_divide_by_scalar(const dpx_array_view *src, double scalar,
                         const dpx_array_view *dst, void *stream);

/* dst = x with NaN replaced by `nan`, +inf by `posinf`, -inf by `neginf` (complex: part by part);
 * float16/32/64 and complex, src and dst of one dtype.  Replaces the contiguous and strided
 * nan_to_num calls of dpnp/backend/extensions/ufunc/elementwise_functions/nan_to_num.cpp
 * (kernels: dpnp/backend/kernels/elementwise_functions/nan_to_num.hpp:44-104). */
int dpx_nan_to_num(const dpx_array_view *src, double nan, double posinf,
                   double neginf, const dpx_array_view *dst, void *stream);
/* dst (bool) = |a - b| <= atol + rtol * |b| for finite pairs, equal_nan for two NaNs, a == b
 * otherwise; a and b of one floating or complex dtype.  Replaces
 * dpnp/backend/extensions/ufunc/elementwise_functions/isclose.cpp
 * (kernels: dpnp/backend/kernels/elementwise_functions/isclose.hpp:47-92). */
int dpx_isclose(const dpx_array_view *a, const dpx_array_view *b, double rtol,
                double atol, int equal_nan, const dpx_array_view *dst,
                void *stream);
/* dst = min(max(x, lo), hi) elementwise: four arrays of one dtype (any of the 14) and one shape
 * (broadcast operands carry zero strides); a NaN element stays NaN, a NaN bound gives NaN; bool:
 * (x || lo) && hi.  Replaces ti._clip, libtensor/source/clip.cpp:69-263 (kernels:
 * libtensor/include/kernels/clip.hpp:66-86 the functor, 89-225 contiguous, 232-330 strided). */
int dpx_clip(const dpx_array_view *x, const dpx_array_view *lo, const dpx_array_view *hi,
             const dpx_array_view *dst, void *stream);
/* dst = x1 * 2^x2: x1 float16/32/64, x2 int8/16/32/64, dst of x1's dtype; an exponent outside the
 * int range gives +inf (positive) or 0.  Replaces the ldexp calls of
 * dpnp/backend/extensions/ufunc/elementwise_functions/ldexp.cpp:62-180 (kernel:
 * dpnp/backend/kernels/elementwise_functions/ldexp.hpp:39-58).  dpx_ldexp_result_type: the dtype of
 * the result for an operand pair, -1 if the pair is not supported (ufi._ldexp_result_type). */
int dpx_ldexp_result_type(int dtype1, int dtype2);
int dpx_ldexp(const dpx_array_view *x1, const dpx_array_view *x2, const dpx_array_view *dst,
              void *stream);
/* x = mantissa * 2^exponent, |mantissa| in [0.5, 1): x and mantissa of one dtype (float16/32/64),
 * exponent int32; the outputs must not overlap each other, the mantissa may be written over x.
 * Replaces dpnp/backend/extensions/ufunc/elementwise_functions/frexp.cpp:70-200 (kernel:
 * dpnp/backend/kernels/elementwise_functions/frexp.hpp:36-56; the reference runs one kernel with
 * two outputs, here the exponent and the mantissa are written by one launch each). */
int dpx_frexp(const dpx_array_view *x, const dpx_array_view *mantissa,
              const dpx_array_view *exponent, void *stream);
/* ti._copy_usm_ndarray_into_usm_ndarray,
 * libtensor/source/copy_and_cast_usm_to_usm.cpp:137-216: dst = cast(src), any
 * dtype pair, equal shapes */
int dpx_copy_cast(const dpx_array_view *src, const dpx_array_view *dst,
                  void *stream);

/* Contiguous byte copies between pageable host memory and device memory, staged through a
 * pool of pinned buffers filled and drained by several host threads.  Replaces the
 * sycl::queue::memcpy calls behind dpnp.asarray / dpnp.asnumpy
 * (libtensor/source/copy_numpy_ndarray_into_usm_ndarray.cpp:60-190 for the contiguous
 * same-dtype case, dpnp/tensor/_copy_utils.py:54-135).
 * dpx_copy_from_host returns once src_host has been read (the device side completes in
 * stream order); dpx_copy_to_host is enqueued on `stream` and returns when dst_host holds
 * the data. */
int dpx_copy_from_host(void *dst_device, const void *src_host, size_t nbytes,
                       void *stream);
int dpx_copy_to_host(void *dst_host, const void *src_device, size_t nbytes,
                     void *stream);
/* ---- device, streams and device memory -----------------------------------------------------
 * For hosts that bring no allocator or stream of their own.  The reference gets both from
 * dpctl: usm_ndarray allocates a dpctl.memory.MemoryUSMDevice for buffer="device"
 * (dpnp/tensor/_usmarray.pyx:270-305) and every call runs on a dpctl.SyclQueue
 * (dpnp/tensor/_device.py:160-175); an array frees its memory when its last reference goes,
 * also while kernels that use it are still queued.
 * dpx_mem_alloc hands out device memory of the current device for use on `stream`;
 * dpx_mem_free takes the stream the block was LAST USED on and makes the block available
 * again in stream order: at once to later work on that stream, after a device-side wait to
 * work on another stream.  Neither call waits for the device, with one exception: when the driver is
 * out of memory dpx_mem_alloc waits for the device (hipDeviceSynchronize), returns every cached block to
 * the driver and tries once more.  Freed blocks stay cached in the
 * process until dpx_mem_release_cached() (which waits for the device).  A stream passed to
 * dpx_mem_free must stay valid while the block is cached: destroy library streams with
 * dpx_stream_destroy, and call dpx_stream_synchronize(stream) before destroying a foreign
 * stream that blocks were freed on.  Thread-safe. */
int dpx_device_count(int *count);                       /* 0 when no device or no driver */
int dpx_device_name(int device, char *buf, size_t len);
int dpx_stream_create(void **stream);                   /* default priority, non-blocking */
int dpx_stream_synchronize(void *stream);
int dpx_stream_destroy(void *stream);                   /* waits for the stream first */
int dpx_mem_alloc(void **ptr, size_t nbytes, void *stream);
int dpx_mem_free(void *ptr, void *stream);
int dpx_mem_release_cached(void);
int dpx_mem_stats(size_t *in_use_bytes, size_t *cached_bytes);

/* dst = value (converted to dst's dtype): ti._full_usm_ndarray,
 * libtensor/source/full_ctor.cpp. value_im is used for complex dst only. */
int dpx_fill(const dpx_array_view *dst, double value_re, double value_im,
             int64_t value_int, int use_int, void *stream);

/* plans: the dispatch decision of the calls above without launching */
int dpx_unary_plan(int op, const dpx_array_view *src,
                   const dpx_array_view *dst, dpx_plan *plan);
int dpx_binary_plan(int op, const dpx_array_view *src1,
                    const dpx_array_view *src2, const dpx_array_view *dst,
                    dpx_plan *plan);
int dpx_where_plan(const dpx_array_view *cond, const dpx_array_view *x1,
                   const dpx_array_view *x2, const dpx_array_view *dst,
                   dpx_plan *plan);

/* ---- fused chains (no counterpart in the reference, which runs them as
 * sequences of the kernels above; results follow the unfused op order) ---- */

/* dst = (lhs CMP rhs) ? x1 : x2 in one pass; cmp_op is one of the six
 * comparison ids of dpx_binary_op.  Equivalent to ti._greater (etc.) into a
 * bool temporary followed by ti._where. */
int dpx_where_compare(int cmp_op, const dpx_array_view *lhs,
                      const dpx_array_view *rhs, const dpx_array_view *x1,
                      const dpx_array_view *x2, const dpx_array_view *dst,
                      void *stream);
/* Black-Scholes call/put prices (formula of examples/example_bs.py:50-78),
 * float64 or float32, all five arrays 1-D contiguous of n elements */
int dpx_black_scholes(const void *price, const void *strike, const void *t,
                      double rate, double vol, void *call, void *put,
                      int64_t n, int dtype, void *stream);

/* ---- reductions --------------------------------------------------------- */

/* py_reduction_over_axis / py_tree_reduction_over_axis,
 * reduction_over_axis.hpp:174-501,508-777 (tri._sum_over_axis, _prod_over_axis,
 * _max_over_axis, _min_over_axis).  The last `trailing_dims_to_reduce` axes of
 * src are reduced; dst has the leading src.nd - trailing axes.
 * op == DPX_R_SUMSQDEV (and DPX_R_NANSUMSQDEV) additionally takes `aux` (same shape and dtype as dst,
 * any strides): dst[i] = sum_j (src[i,j] - aux[i])^2; aux is NULL otherwise.  DPX_R_SUMSQDEV of complex
 * src gives the real dst[i] = sum_j |src[i,j] - aux[i]|^2 (float32 or float64 from complex64, float64 from
 * complex128), with aux complex of dst's precision (complex64 for a float32 dst, else complex128). */
int dpx_reduce(int op, const dpx_array_view *src, int trailing_dims_to_reduce,
               const dpx_array_view *dst, const dpx_array_view *aux,
               void *stream);
/* DPX_R_NANVAR with a delta degrees of freedom: dst[i] = sum_j (src[i,j] - mean[i])^2 /
 * (count_i - ddof) over the elements that are not NaN, NaN where count_i <= ddof.  The second pass
 * of dpnp.nanvar / nanstd (dpnp/dpnp_iface_nanfunctions.py:1318-1390: count, mean, subtract,
 * square, sum and divide as separate calls there). */
int dpx_nan_variance(const dpx_array_view *src, int trailing_dims_to_reduce,
                     const dpx_array_view *mean, double ddof,
                     const dpx_array_view *dst, void *stream);
/* py_search_over_axis, reduction_over_axis.hpp:781-1047 (tri._argmax_over_axis,
 * tri._argmin_over_axis): int64 C-order flat index over the reduced axes,
 * smallest index among equal extrema, NaN counts as the extremum (first NaN) */
int dpx_argreduce(int op, const dpx_array_view *src,
                  int trailing_dims_to_reduce, const dpx_array_view *dst,
                  void *stream);
/* dpx_reduce for callers that cannot allocate device memory (code under HIP graph capture,
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same
 * arguments, validation and results as dpx_reduce (bit for bit: same kernels, same partition).
 * A reduction that is split over several blocks per output keeps its partial results in a static
 * device array of DPX_NOALLOC_SCRATCH_BYTES that every GPU the library runs on holds until the
 * process ends, instead of the per-stream pool; the call clears the array's ticket counters with
 * a fill kernel, launches the reduction, and calls no hipMalloc / hipFree.  A reduction whose
 * partials do not fit fails with DPX_ERR_BAD_ARGUMENT before anything is launched
 * (dpx_reduce_plan(...).scratch_bytes tells in advance: row and full reductions need at most
 * 136 KiB, column reductions at most 1.2 MiB; only reductions over the rows of a row-major matrix
 * of 1- and 2-byte elements with rows of 300 to 511 bytes exceed the limit).  All calls on one GPU share the array: two calls of this entry point that
 * overlap in time on one GPU (different streams, or two host threads) race on it; calls on one
 * stream, or calls ordered by events, are safe. */
#define DPX_NOALLOC_SCRATCH_BYTES (2u << 20)
int dpx_reduce_noalloc(int op, const dpx_array_view *src, int trailing_dims_to_reduce,
                       const dpx_array_view *dst, const dpx_array_view *aux,
                       void *stream);
int dpx_reduce_plan(int op, const dpx_array_view *src,
                    int trailing_dims_to_reduce, const dpx_array_view *dst,
                    dpx_plan *plan);
int dpx_argreduce_plan(int op, const dpx_array_view *src,
                       int trailing_dims_to_reduce, const dpx_array_view *dst,
                       dpx_plan *plan);

/* ---- stride collapsing (exposed for testing) ---------------------------- */

/* Joint collapse of `nops` stride vectors over one shape
 * (simplify_iteration_space*, libtensor/source/simplify_iteration_space.cpp:51-417;
 * libtensor/include/utils/strided_iters.hpp:364-899).  strides is
 * [nops][DPX_MAX_ND]; shape and strides are rewritten in place, offsets[nops]
 * receives the element displacement of each operand.  keep_order != 0 only
 * merges adjacent dims (compact_iteration, strided_iters.hpp:946-983).
 * Returns the new number of dims. */
int dpx_collapse(int nd, int nops, int64_t *shape, int64_t *strides,
                 int64_t *offsets, int keep_order);

#ifdef __cplusplus
}
#endif
#endif /* DPNP_AMD_H */
