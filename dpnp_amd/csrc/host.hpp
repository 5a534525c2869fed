// Host-side glue shared by the entry points: error reporting, view checks, stride
// collapsing, the scratch pool.  No device code here.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string>
#include "../../include/dpnp_amd.h"

namespace dpx {

int fail(int status, const std::string &msg);          // records msg, returns status
int fail_hip(hipError_t e, const char *where);         // DPX_ERR_HIP
inline int itemsize_of(int dt)
{
    static const int sz[DPX_NUM_DTYPES] = {1, 1, 1, 2, 2, 4, 4, 8, 8, 2, 4, 8, 8, 16};
    return (dt >= 0 && dt < DPX_NUM_DTYPES) ? sz[dt] : -1;
}
const char *dtype_name(int dt);

bool view_ok(const dpx_array_view *v);                  // nd / dtype / shape sanity
int64_t view_size(const dpx_array_view *v);             // number of elements
// smallest and largest element offset addressed by the view (0,0 if empty)
void view_minmax(const dpx_array_view *v, int64_t &lo, int64_t &hi);
bool views_overlap(const dpx_array_view *a, const dpx_array_view *b);
bool views_same_logical(const dpx_array_view *a, const dpx_array_view *b);
bool same_shape(const dpx_array_view *a, const dpx_array_view *b);

// Joint collapse of nops stride vectors (rows of `strides`, row length DPX_MAX_ND).
int collapse(int nd, int nops, int64_t *shape, int64_t (*strides)[DPX_MAX_ND],
             int64_t *offsets, bool keep_order);

// Scratch for partial results, owned by the library: one grow-only block per stream.
// Work on one stream is ordered, so reuse by the next call on that stream is safe.
// A newly allocated block is zero-filled (on the stream).
void *scratch_get(hipStream_t stream, size_t bytes);
int scratch_release_all();

// number of compute units of the current device (cached)
int device_cus();

} // namespace dpx
