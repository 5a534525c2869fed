// see ew_half_table.hpp
#include "ew_half_table.hpp"
#include "host.hpp"
#include "types.hpp"
#include <map>
#include <mutex>

namespace dpx {

namespace {
constexpr int APPLY_BLOCK = 1024;

// One block per CU (the table takes most of its LDS), which walks its share of the array a pack of 8 elements per
// thread and round.  The next round's load goes out before this round is translated and stored: with 16 waves
// on the CU and nothing else to overlap, a wave that waited for its loads, then stored, then loaded again left
// the memory system alternately reading and writing (2^27 elements: 65 % of the HBM rate against 76 %).
__global__ __launch_bounds__(APPLY_BLOCK) void half_table_apply_kernel(const uint16_t *table, const uint16_t *in,
                                                                        uint16_t *out, int64_t n)
{
    extern __shared__ __align__(16) unsigned char lds_raw[];
    u32x4 *lds16 = reinterpret_cast<u32x4 *>(lds_raw);
    const uint16_t *lut = reinterpret_cast<const uint16_t *>(lds_raw);
    const int64_t npacks = n >> 3;
    const int64_t step = (int64_t)gridDim.x * APPLY_BLOCK;
    int64_t p = (int64_t)blockIdx.x * APPLY_BLOCK + threadIdx.x;
    pack<uint16_t, 8> cur{}, nxt{};
    if (p < npacks) cur = load_pack<uint16_t, 8>(in + p * 8);
    for (int i = threadIdx.x; i < HALF_TABLE_ENTRIES * 2 / 16; i += APPLY_BLOCK)
        lds16[i] = reinterpret_cast<const u32x4 *>(table)[i];
    __syncthreads();
    for (; p < npacks; p += step) {
        if (p + step < npacks) nxt = load_pack<uint16_t, 8>(in + (p + step) * 8);
        pack<uint16_t, 8> r;
#pragma unroll
        for (int e = 0; e < 8; ++e) r.v[e] = lut[cur.v[e]];
        store_pack<uint16_t, 8>(out + p * 8, r);
        cur = nxt;
    }
    // the last n % 8 elements
    if (blockIdx.x == 0 && threadIdx.x < (n & 7)) {
        const int64_t i = (npacks << 3) + threadIdx.x;
        out[i] = lut[in[i]];
    }
}

std::mutex g_mu;
std::map<std::pair<int, int>, uint16_t *> g_tables; // (device, op) -> table, never freed
uint64_t g_lds_raised = 0;                         // devices whose apply kernel may take 128 KiB of LDS
} // namespace

const uint16_t *half_table_for(int op, hipStream_t stream, hipError_t (*build)(uint16_t *, hipStream_t))
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return nullptr;
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = g_tables.find({dev, op});
    if (it != g_tables.end()) return it->second;
    // building allocates and waits for the stream once: not while the stream records a graph
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) {
        (void)hipGetLastError();
        return nullptr;
    }
    uint16_t *t = nullptr;
    if (hipMalloc((void **)&t, HALF_TABLE_ENTRIES * sizeof(uint16_t)) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    // (complete before another stream may read it)
    if (build(t, stream) != hipSuccess || hipStreamSynchronize(stream) != hipSuccess) {
        (void)hipGetLastError();
        (void)hipFree(t);
        return nullptr;
    }
    g_tables[{dev, op}] = t;
    return t;
}

hipError_t half_table_apply(const uint16_t *table, const void *in, void *out, int64_t n, hipStream_t stream)
{
    constexpr int LDS = HALF_TABLE_ENTRIES * (int)sizeof(uint16_t);
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    {
        std::lock_guard<std::mutex> lk(g_mu);
        const uint64_t bit = 1ull << (dev & 63);
        if (!(g_lds_raised & bit)) {
            e = hipFuncSetAttribute((const void *)half_table_apply_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
            if (e != hipSuccess) return e;
            g_lds_raised |= bit;
        }
    }
    const int64_t chunks = ((n >> 3) + APPLY_BLOCK - 1) / APPLY_BLOCK;
    const int64_t grid = std::max<int64_t>(1, std::min<int64_t>(device_cus(), chunks));
    hipLaunchKernelGGL(half_table_apply_kernel, dim3((unsigned)grid), dim3(APPLY_BLOCK), LDS, stream, table,
                       (const uint16_t *)in, (uint16_t *)out, n);
    return hipGetLastError();
}

} // namespace dpx
