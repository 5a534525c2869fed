#include "host.hpp"
#include <algorithm>
#include <cstdlib>
#include <map>
#include <mutex>
#include <numeric>
#include <vector>

namespace dpx {

static thread_local std::string g_last_error;

int fail(int status, const std::string &msg)
{
    g_last_error = msg;
    return status;
}
int fail_hip(hipError_t e, const char *where)
{
    g_last_error = std::string("HIP error in ") + where + ": " + hipGetErrorString(e);
    return DPX_ERR_HIP;
}
const char *dtype_name(int dt)
{
    static const char *names[DPX_NUM_DTYPES] = {"bool",    "int8",    "uint8",     "int16",     "uint16",
                                                "int32",   "uint32",  "int64",     "uint64",    "float16",
                                                "float32", "float64", "complex64", "complex128"};
    return (dt >= 0 && dt < DPX_NUM_DTYPES) ? names[dt] : "?";
}

bool view_ok(const dpx_array_view *v)
{
    if (!v || v->nd < 0 || v->nd > DPX_MAX_ND) return false;
    if (v->dtype < 0 || v->dtype >= DPX_NUM_DTYPES) return false;
    for (int d = 0; d < v->nd; ++d)
        if (v->shape[d] < 0) return false;
    return true;
}
int64_t view_size(const dpx_array_view *v)
{
    int64_t n = 1;
    for (int d = 0; d < v->nd; ++d) n *= v->shape[d];
    return n;
}
void view_minmax(const dpx_array_view *v, int64_t &lo, int64_t &hi)
{
    lo = hi = 0;
    if (view_size(v) == 0) return;
    for (int d = 0; d < v->nd; ++d) {
        const int64_t ext = (v->shape[d] - 1) * v->strides[d];
        if (ext < 0) lo += ext;
        else hi += ext;
    }
}
// byte intervals [x0, x1) and [y0, y1) intersect (memory_overlap.hpp:56-113)
bool views_overlap(const dpx_array_view *a, const dpx_array_view *b)
{
    if (view_size(a) == 0 || view_size(b) == 0) return false;
    int64_t alo, ahi, blo, bhi;
    view_minmax(a, alo, ahi);
    view_minmax(b, blo, bhi);
    const int64_t as = itemsize_of(a->dtype), bs = itemsize_of(b->dtype);
    const char *x0 = (const char *)a->data + alo * as, *x1 = (const char *)a->data + (ahi + 1) * as;
    const char *y0 = (const char *)b->data + blo * bs, *y1 = (const char *)b->data + (bhi + 1) * bs;
    return (x1 > y0) && (y1 > x0);
}
// same pointer, dtype, shape and strides (memory_overlap.hpp:115-155)
bool views_same_logical(const dpx_array_view *a, const dpx_array_view *b)
{
    if (a->nd != b->nd || a->dtype != b->dtype || a->data != b->data) return false;
    for (int d = 0; d < a->nd; ++d)
        if (a->shape[d] != b->shape[d] || a->strides[d] != b->strides[d]) return false;
    return true;
}
bool same_shape(const dpx_array_view *a, const dpx_array_view *b)
{
    if (a->nd != b->nd) return false;
    for (int d = 0; d < a->nd; ++d)
        if (a->shape[d] != b->shape[d]) return false;
    return true;
}

// ---- stride collapsing ---------------------------------------------------------------
// Rewrites (shape, strides[k], offsets[k]) so that the set of address tuples visited is
// unchanged while the number of dims is minimal:
//   1. extent-1 dims vanish;
//   2. (reordering allowed) dims are ordered by decreasing |stride| of the LAST operand
//      (the output), ties broken by the operands before it, then by extent; dims in
//      which no operand moves forward and one moves backward are walked in reverse
//      (the displacement goes into offsets);
//   3. neighbours merge when, for every operand, stride[i] == shape[i+1] * stride[i+1].
// Same contract as simplify_iteration_*_strides / compact_iteration
// (libtensor/include/utils/strided_iters.hpp:340-361,364-899,946-983).
int collapse(int nd, int nops, int64_t *shape, int64_t (*strides)[DPX_MAX_ND],
             int64_t *offsets, bool keep_order)
{
    for (int k = 0; k < nops; ++k) offsets[k] = 0;
    std::vector<int> dims;
    for (int d = 0; d < nd; ++d)
        if (shape[d] != 1) dims.push_back(d);
    auto mag = [](int64_t s) { return s < 0 ? -s : s; };
    if (!keep_order) {
        std::stable_sort(dims.begin(), dims.end(), [&](int a, int b) {
            for (int k = nops - 1; k >= 0; --k) {
                const int64_t sa = mag(strides[k][a]), sb = mag(strides[k][b]);
                if (sa != sb) return sa > sb;
            }
            return shape[a] > shape[b];
        });
    }
    std::vector<int64_t> sh;
    std::vector<std::vector<int64_t>> st(nops);
    for (int d : dims) {
        bool any_neg = false, any_pos = false;
        for (int k = 0; k < nops; ++k) {
            any_neg |= strides[k][d] < 0;
            any_pos |= strides[k][d] > 0;
        }
        const bool flip = !keep_order && any_neg && !any_pos;
        sh.push_back(shape[d]);
        for (int k = 0; k < nops; ++k) {
            int64_t s = strides[k][d];
            if (flip) {
                offsets[k] += s * (shape[d] - 1);
                s = -s;
            }
            st[k].push_back(s);
        }
    }
    int n = (int)sh.size();
    for (int i = 0; i + 1 < n;) {
        bool merge = true;
        for (int k = 0; k < nops && merge; ++k) merge = st[k][i] == sh[i + 1] * st[k][i + 1];
        if (merge) {
            sh[i] *= sh[i + 1];
            sh.erase(sh.begin() + i + 1);
            for (int k = 0; k < nops; ++k) st[k].erase(st[k].begin() + i);
            --n;
            if (i > 0) --i; // the merged dim may now fuse with its left neighbour
        }
        else ++i;
    }
    for (int i = 0; i < n; ++i) {
        shape[i] = sh[i];
        for (int k = 0; k < nops; ++k) strides[k][i] = st[k][i];
    }
    return n;
}

// ---- scratch pool ------------------------------------------------------------------------
namespace {
struct Block {
    void *p = nullptr;
    size_t bytes = 0;
    bool dirty = false;
};
std::mutex g_pool_mu;
std::map<std::pair<int, hipStream_t>, Block> g_pool;
std::vector<void *> g_retired; // outgrown blocks: possibly still in use, freed by scratch_release_all()

__global__ void scratch_zero_kernel(uint4 *p, size_t n16)
{
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x)
        p[i] = uint4{0u, 0u, 0u, 0u};
}
} // namespace

hipError_t zero_fill_async(void *p, size_t n16, hipStream_t stream)
{
    if (n16 == 0) return hipSuccess;
    const unsigned blocks = (unsigned)std::min<size_t>((n16 + 255) / 256, 1024);
    scratch_zero_kernel<<<blocks, 256, 0, stream>>>(static_cast<uint4 *>(p), n16);
    return hipGetLastError();
}

void *scratch_get(hipStream_t stream, size_t bytes, size_t counter_bytes)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return nullptr;
    std::lock_guard<std::mutex> lk(g_pool_mu);
    Block &b = g_pool[{dev, stream}];
    if (b.p && b.bytes >= bytes) {
        if (b.dirty) {
            if (zero_fill_async(b.p, std::min(counter_bytes, b.bytes) / 16, stream) != hipSuccess) return nullptr;
            b.dirty = false;
        }
        return b.p;
    }
    size_t want = std::max<size_t>(bytes, SCRATCH_BLOCK_BYTES);
    want = (want + 4095) & ~(size_t)4095;
    void *fresh = nullptr;
    if (hipMalloc(&fresh, want) != hipSuccess) return nullptr;
    // callers rely on fresh blocks being zero (ticket counters) and keep them zero
    if (zero_fill_async(fresh, want / 16, stream) != hipSuccess) { // want is a multiple of 4096
        (void)hipFree(fresh);
        return nullptr;
    }
    if (b.p) g_retired.push_back(b.p);
    b.p = fresh;
    b.bytes = want;
    b.dirty = false;
    return b.p;
}
void scratch_mark_dirty(hipStream_t stream)
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return;
    std::lock_guard<std::mutex> lk(g_pool_mu);
    auto it = g_pool.find({dev, stream});
    if (it != g_pool.end()) it->second.dirty = true;
}
int scratch_release_all()
{
    std::lock_guard<std::mutex> lk(g_pool_mu);
    for (auto &kv : g_pool)
        if (kv.second.p) (void)hipFree(kv.second.p);
    for (void *p : g_retired) (void)hipFree(p);
    g_pool.clear();
    g_retired.clear();
    return DPX_OK;
}

#ifdef DPX_TUNING
int tune_int(const char *name, int dflt)
{
    static std::mutex mu;
    static std::map<std::string, int> seen;
    std::lock_guard<std::mutex> lk(mu);
    auto it = seen.find(name);
    if (it != seen.end()) return it->second;
    const char *s = std::getenv(name);
    const int v = (s && *s) ? std::atoi(s) : dflt;
    seen[name] = v;
    return v;
}
#endif

int device_cus()
{
    static int cus = 0;
    if (cus == 0) {
        int dev = 0, v = 0;
        if (hipGetDevice(&dev) == hipSuccess &&
            hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0)
            cus = v;
        else
            return 256; // MI355X; planning without a device (CPU-side tests) assumes it
    }
    return cus;
}

} // namespace dpx

extern "C" {
int dpx_abi_version(void) { return 1; }
const char *dpx_last_error(void) { return dpx::g_last_error.c_str(); }
int dpx_dtype_itemsize(int dt) { return dpx::itemsize_of(dt); }
int dpx_release_scratch(void) { return dpx::scratch_release_all(); }
int dpx_array_overlap(const dpx_array_view *a, const dpx_array_view *b)
{
    if (!dpx::view_ok(a) || !dpx::view_ok(b)) return 0;
    return dpx::views_overlap(a, b) ? 1 : 0;
}
int dpx_same_logical(const dpx_array_view *a, const dpx_array_view *b)
{
    if (!dpx::view_ok(a) || !dpx::view_ok(b)) return 0;
    return dpx::views_same_logical(a, b) ? 1 : 0;
}
int dpx_collapse(int nd, int nops, int64_t *shape, int64_t *strides, int64_t *offsets, int keep_order)
{
    if (nd < 0 || nd > DPX_MAX_ND || nops < 1 || nops > 8) return -1;
    return dpx::collapse(nd, nops, shape, reinterpret_cast<int64_t(*)[DPX_MAX_ND]>(strides), offsets,
                         keep_order != 0);
}
}
