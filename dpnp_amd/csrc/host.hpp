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

// Scratch for partial results, owned by the library: one block per (device, stream), allocated
// at the stream's first split reduction with SCRATCH_BLOCK_BYTES, which covers every plan the
// reduction planner makes for arrays that fit a device (see red_make_plan).  Work on one stream
// is ordered, so reuse by the next call on that stream is safe.  A block is zero-filled when it
// is allocated (on the stream) and the kernels leave its ticket counters at zero.
// A request beyond the block's size allocates a larger block and RETIRES the old one: a block
// that was ever handed out is not freed before scratch_release_all(), so a launch that another
// host thread is still preparing keeps valid memory, and nothing waits for the stream.
// scratch_mark_dirty(): a launch that used the block reported an error; its ticket counters are
// cleared again (first `counter_bytes` of the block) before the block is handed out next.
constexpr size_t SCRATCH_BLOCK_BYTES = (size_t)8 << 20;
void *scratch_get(hipStream_t stream, size_t bytes, size_t counter_bytes);
void scratch_mark_dirty(hipStream_t stream);
int scratch_release_all();
// fills n16 16-byte words at p with zeros on `stream` (a kernel, not a memset node: memset nodes
// recorded into a stream capture have replayed wrongly on these machines)
hipError_t zero_fill_async(void *p, size_t n16, hipStream_t stream);

// Launch-geometry overrides for sweeps.  The product build compiles them out (every call returns
// its default); a build with -DDPX_TUNING reads the environment variable `name` once per process.
#ifdef DPX_TUNING
int tune_int(const char *name, int dflt);
#else
inline int tune_int(const char *, int dflt) { return dflt; }
#endif

// number of compute units of the current device (cached)
int device_cus();

} // namespace dpx
