// Device memory and streams owned by the library, for hosts that bring no allocator of their own.
//
// The reference allocates USM memory through dpctl (dpnp/tensor/_usmarray.pyx, dpctl.memory) and
// runs every kernel on a sycl::queue; its arrays free their memory when the last reference goes,
// while kernels that use it may still be queued, and the SYCL runtime keeps the allocation alive
// until they have run.  Here the same promise comes from stream order: dpx_mem_free() takes the
// stream the block was last used on and only records the block as free FOR THAT STREAM.  Work
// submitted later to the same stream runs after everything that used the block, so the block can
// be handed out again at once without waiting.  A request from another stream first makes that
// stream wait (hipStreamWaitEvent) for an event recorded on the block's old stream.
//
// Blocks are cached, never returned to the driver before dpx_mem_release_cached(): hipMalloc and
// hipFree cost tens of microseconds and hipFree waits for the device.  Sizes are rounded up to
// 512 bytes below 1 MiB and to 2 MiB above (large blocks then start on 2 MiB boundaries, which
// is what the driver maps with its largest pages); a cached block serves a request when it is
// large enough and wastes at most a quarter of the request.
#include <hip/hip_runtime.h>
#include <map>
#include <mutex>
#include <unordered_map>
#include <unordered_set>
#include <cstring>
#include "host.hpp"

namespace dpx {
namespace {

struct Block {
    void *ptr;
    size_t size;
    hipStream_t stream; // the stream of its last use; meaningful while cached
    bool idle;          // its last use is known to have completed (the stream was synchronized or destroyed)
    uint64_t stamp;     // value of the free counter when it was cached: orders frees against stream waits
};

constexpr int MAX_DEVICES = 64;
std::mutex g_mu;
std::unordered_map<void *, Block> g_live;                // handed out
std::multimap<size_t, Block> g_cache[MAX_DEVICES];       // free, by size
std::unordered_map<void *, int> g_device_of;             // every block the pool owns -> device
std::unordered_set<hipStream_t> g_streams;               // streams made by dpx_stream_create
size_t g_in_use = 0, g_cached = 0;
uint64_t g_free_seq = 0;                                 // counts dpx_mem_free calls

size_t round_size(size_t n)
{
    if (n == 0) n = 1;
    if (n < ((size_t)1 << 20)) return (n + 511) & ~(size_t)511;
    return (n + (((size_t)2 << 20) - 1)) & ~(((size_t)2 << 20) - 1);
}

// frees every cached block of `dev`; the caller holds g_mu and has made the device idle
void drop_cache(int dev)
{
    for (auto &kv : g_cache[dev]) {
        (void)hipFree(kv.second.ptr);
        g_device_of.erase(kv.second.ptr);
        g_cached -= kv.second.size;
    }
    g_cache[dev].clear();
}

} // namespace
} // namespace dpx

using namespace dpx;

extern "C" {

int dpx_device_count(int *count)
{
    if (!count) return fail(DPX_ERR_BAD_ARGUMENT, "device_count: null pointer");
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess) {
        // no driver or no device: not an error of the call, there is just nothing to run on
        (void)hipGetLastError();
        n = 0;
    }
    *count = n;
    return DPX_OK;
}

int dpx_device_name(int device, char *buf, size_t len)
{
    if (!buf || len == 0) return fail(DPX_ERR_BAD_ARGUMENT, "device_name: no buffer");
    hipDeviceProp_t prop;
    hipError_t e = hipGetDeviceProperties(&prop, device);
    if (e != hipSuccess) return fail_hip(e, "hipGetDeviceProperties");
    std::strncpy(buf, prop.name, len - 1);
    buf[len - 1] = 0;
    return DPX_OK;
}

int dpx_stream_create(void **stream)
{
    if (!stream) return fail(DPX_ERR_BAD_ARGUMENT, "stream_create: null pointer");
    hipStream_t s = nullptr;
    // default priority; non-blocking: no implicit ordering against the null stream
    hipError_t e = hipStreamCreateWithFlags(&s, hipStreamNonBlocking);
    if (e != hipSuccess) return fail_hip(e, "hipStreamCreateWithFlags");
    {
        std::lock_guard<std::mutex> lk(g_mu);
        g_streams.insert(s);
    }
    *stream = s;
    return DPX_OK;
}

int dpx_stream_synchronize(void *stream)
{
    // Blocks freed on this stream BEFORE the wait starts have completed when it returns.  Another thread may
    // free a block on the stream while this one waits or before it takes the lock again: that block's work
    // may still be queued, so it must not be marked.
    uint64_t seen;
    {
        std::lock_guard<std::mutex> lk(g_mu);
        seen = g_free_seq;
    }
    hipError_t e = hipStreamSynchronize((hipStream_t)stream);
    if (e != hipSuccess) return fail_hip(e, "hipStreamSynchronize");
    std::lock_guard<std::mutex> lk(g_mu);
    for (auto &cache : g_cache)
        for (auto &kv : cache)
            if (kv.second.stream == (hipStream_t)stream && kv.second.stamp <= seen) kv.second.idle = true;
    return DPX_OK;
}

int dpx_stream_destroy(void *stream)
{
    {
        std::lock_guard<std::mutex> lk(g_mu);
        if (!g_streams.count((hipStream_t)stream))
            return fail(DPX_ERR_BAD_ARGUMENT, "stream_destroy: not a stream of dpx_stream_create");
    }
    // cached blocks last used on it must not refer to a dead stream: wait for it, mark them idle
    int rc = dpx_stream_synchronize(stream);
    if (rc != DPX_OK) return rc;
    {
        std::lock_guard<std::mutex> lk(g_mu);
        g_streams.erase((hipStream_t)stream);
    }
    hipError_t e = hipStreamDestroy((hipStream_t)stream);
    return e == hipSuccess ? DPX_OK : fail_hip(e, "hipStreamDestroy");
}

int dpx_mem_alloc(void **ptr, size_t nbytes, void *stream)
{
    if (!ptr) return fail(DPX_ERR_BAD_ARGUMENT, "mem_alloc: null pointer");
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail_hip(e, "hipGetDevice");
    if (dev < 0 || dev >= MAX_DEVICES) return fail(DPX_ERR_BAD_ARGUMENT, "mem_alloc: device index out of range");
    if (nbytes > ((size_t)1 << 46)) return fail(DPX_ERR_BAD_ARGUMENT, "mem_alloc: more than 64 TiB asked for");
    const size_t size = round_size(nbytes);
    const hipStream_t s = (hipStream_t)stream;
    Block blk{nullptr, 0, nullptr, true, 0};
    {
        std::lock_guard<std::mutex> lk(g_mu);
        auto &cache = g_cache[dev];
        // the smallest cached block that is large enough and not too large; among those one that
        // needs no wait (same stream, or idle) is taken first
        auto pick = cache.end();
        for (auto it = cache.lower_bound(size); it != cache.end() && it->first <= size + size / 4; ++it) {
            if (it->second.stream == s || it->second.idle) {
                pick = it;
                break;
            }
            if (pick == cache.end()) pick = it;
        }
        if (pick != cache.end()) {
            if (pick->second.stream != s && !pick->second.idle) {
                // order this stream after everything queued on the block's old stream so far; under the
                // lock, so that dpx_stream_destroy of the old stream cannot come in between
                hipEvent_t ev;
                e = hipEventCreateWithFlags(&ev, hipEventDisableTiming);
                if (e == hipSuccess) {
                    e = hipEventRecord(ev, pick->second.stream);
                    if (e == hipSuccess) e = hipStreamWaitEvent(s, ev, 0);
                    const hipError_t e2 = hipEventDestroy(ev); // deferred until the event has completed
                    if (e == hipSuccess) e = e2;
                }
                if (e != hipSuccess) return fail_hip(e, "mem_alloc: ordering after the block's previous stream");
            }
            blk = pick->second;
            cache.erase(pick);
            g_cached -= blk.size;
        }
    }
    if (!blk.ptr) {
        void *p = nullptr;
        e = hipMalloc(&p, size);
        if (e != hipSuccess) {
            // out of memory: give the cached blocks back to the driver and try once more
            (void)hipGetLastError();
            e = hipDeviceSynchronize();
            if (e != hipSuccess) return fail_hip(e, "hipDeviceSynchronize");
            {
                std::lock_guard<std::mutex> lk(g_mu);
                drop_cache(dev);
            }
            e = hipMalloc(&p, size);
            if (e != hipSuccess) {
                (void)hipGetLastError();
                return fail(DPX_ERR_HIP, "mem_alloc: hipMalloc of " + std::to_string(size) + " bytes: " + hipGetErrorString(e));
            }
        }
        blk = Block{p, size, s, false, 0};
    }
    blk.stream = s;
    blk.idle = false;
    {
        std::lock_guard<std::mutex> lk(g_mu);
        g_live.emplace(blk.ptr, blk);
        g_device_of[blk.ptr] = dev;
        g_in_use += blk.size;
    }
    *ptr = blk.ptr;
    return DPX_OK;
}

int dpx_mem_free(void *ptr, void *stream)
{
    if (!ptr) return DPX_OK;
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = g_live.find(ptr);
    if (it == g_live.end()) return fail(DPX_ERR_BAD_ARGUMENT, "mem_free: not a live block of dpx_mem_alloc");
    Block blk = it->second;
    g_live.erase(it);
    blk.stream = (hipStream_t)stream;
    blk.idle = false;
    blk.stamp = ++g_free_seq;
    g_in_use -= blk.size;
    g_cached += blk.size;
    g_cache[g_device_of[ptr]].emplace(blk.size, blk);
    return DPX_OK;
}

int dpx_mem_release_cached(void)
{
    int cur = 0;
    hipError_t e = hipGetDevice(&cur);
    if (e != hipSuccess) return fail_hip(e, "hipGetDevice");
    for (int dev = 0; dev < MAX_DEVICES; ++dev) {
        {
            std::lock_guard<std::mutex> lk(g_mu);
            if (g_cache[dev].empty()) continue;
        }
        e = hipSetDevice(dev);
        if (e == hipSuccess) e = hipDeviceSynchronize();
        if (e != hipSuccess) {
            (void)hipSetDevice(cur);
            return fail_hip(e, "mem_release_cached: waiting for the device");
        }
        std::lock_guard<std::mutex> lk(g_mu);
        drop_cache(dev);
    }
    e = hipSetDevice(cur);
    return e == hipSuccess ? DPX_OK : fail_hip(e, "hipSetDevice");
}

int dpx_mem_stats(size_t *in_use_bytes, size_t *cached_bytes)
{
    std::lock_guard<std::mutex> lk(g_mu);
    if (in_use_bytes) *in_use_bytes = g_in_use;
    if (cached_bytes) *cached_bytes = g_cached;
    return DPX_OK;
}

} // extern "C"
