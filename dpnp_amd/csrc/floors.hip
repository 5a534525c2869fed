// Measurement kernels ("floors"): what a memory access pattern or an instruction stream costs on its own,
// without the product kernel around it.  bench.py --workload floors times them beside the product's
// kernels; a product kernel that runs as long as its floor is bound by the pattern, not by its code.
// Built into libdpx_floors.so, which only bench.py loads; nothing in the product calls it.
//
//   launch              an empty kernel: the cost of a launch seen by events on the stream
//   bs_streams          the Black-Scholes kernel with its arithmetic taken out: 3 loads + 2 stores of 2^26 doubles
//   bs_arithmetic       the same kernel with its memory streams taken out: the pricing of 2^26 options
//   stream5_f64         3 loads + 2 stores of 2^26 doubles in the plainest shape (256 threads, one pack each)
//   read_f32_2p24       2^24 floats read once and added up per block, partials stored, no cross-block step
//   read_f32_2p24_tickets  the same with the smallest two-level ticket scheme that lets the last block fold
//   stride2_one_input   out[r][c] = A[r][2c] * row[c] over 8192 x 4096: a wave reads its 2 KiB run with two
//                       lane-interleaved 16-byte loads and regroups by lane shuffles, two rows per wave
//   stride2_predicate   out[r][c] = A[r][2c] > 0 as bytes, same access
//   stride2_two_inputs  out[r][c] = A[r][2c] * B[r][2c], same access for both inputs
//   tile_runs_8192      reads 128 x 128 float tiles of an 8192 x 8192 matrix in 512-byte runs and writes the
//                       tile at the transposed place in 512-byte runs WITHOUT transposing it (no LDS): the
//                       global access pattern of the transposing tile kernel
#include <hip/hip_runtime.h>
#include <cstdint>
#include "black_scholes.hpp"

namespace {
using namespace dpx;
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

__device__ inline f32x4 ldn(const float *p) { return __builtin_nontemporal_load((const f32x4 *)p); }
__device__ inline void stn(float *p, f32x4 v) { __builtin_nontemporal_store(v, (f32x4 *)p); }

__global__ void empty_kernel() {}

__global__ void fill_kernel(u32x4 *p, size_t n16, unsigned v)
{
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x)
        p[i] = u32x4{v, v, v, v};
}

// ---- five streams of doubles, plain shape ----------------------------------------------------------------
typedef double f64x2 __attribute__((ext_vector_type(2)));
__global__ __launch_bounds__(256) void stream5_kernel(const double *a, const double *b, const double *c, double *x, double *y)
{
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 2;
    const f64x2 va = __builtin_nontemporal_load((const f64x2 *)(a + i)), vb = __builtin_nontemporal_load((const f64x2 *)(b + i)),
                vc = __builtin_nontemporal_load((const f64x2 *)(c + i));
    __builtin_nontemporal_store(va + vb, (f64x2 *)(x + i));
    __builtin_nontemporal_store(vc * vb, (f64x2 *)(y + i));
}

// ---- 2^24 floats read once ---------------------------------------------------------------------------------
__device__ inline float wave_sum(float r)
{
    for (int o = 32; o > 0; o >>= 1) r += __shfl_down(r, o, 64);
    return r;
}
__device__ inline float block_sum(float r) // 256 threads; valid in thread 0
{
    __shared__ float sm[4];
    r = wave_sum(r);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) sm[threadIdx.x >> 6] = r;
    __syncthreads();
    if (threadIdx.x == 0) r = (sm[0] + sm[1]) + (sm[2] + sm[3]);
    return r;
}
__device__ inline float stream_sum(const float *x, size_t n) // this block's share, four 16-byte loads in flight per lane
{
    const size_t chunk = ((n / gridDim.x) + 1023) / 1024 * 1024;
    const size_t beg = blockIdx.x * chunk, end = beg + chunk < n ? beg + chunk : n;
    float a0 = 0, a1 = 0, a2 = 0, a3 = 0;
    size_t pos = beg + threadIdx.x * 4;
    const size_t step = 1024;
    for (; pos + 3 * step < end; pos += 4 * step) {
        const f32x4 v0 = ldn(x + pos), v1 = ldn(x + pos + step), v2 = ldn(x + pos + 2 * step), v3 = ldn(x + pos + 3 * step);
        a0 += v0[0] + v0[1] + v0[2] + v0[3];
        a1 += v1[0] + v1[1] + v1[2] + v1[3];
        a2 += v2[0] + v2[1] + v2[2] + v2[3];
        a3 += v3[0] + v3[1] + v3[2] + v3[3];
    }
    for (; pos < end; pos += step) {
        const f32x4 v = ldn(x + pos);
        a0 += v[0] + v[1] + v[2] + v[3];
    }
    return (a0 + a1) + (a2 + a3);
}
__global__ __launch_bounds__(256) void read_kernel(const float *x, size_t n, float *part)
{
    const float r = block_sum(stream_sum(x, n));
    if (threadIdx.x == 0) part[blockIdx.x] = r;
}
// Two ticket levels (groups of 32 blocks), partial and tickets by relaxed device-scope atomics, the ticket's address
// made to depend on the value the exchange returned; the block that draws the last ticket folds the partials.
__global__ __launch_bounds__(256) void read_tickets_kernel(const float *x, size_t n, float *part, unsigned *cnt, float *out)
{
    const float r = block_sum(stream_sum(x, n));
    __shared__ int last;
    if (threadIdx.x == 0) {
        const unsigned tok = __hip_atomic_exchange((unsigned *)part + blockIdx.x, __float_as_uint(r), __ATOMIC_RELAXED,
                                                   __HIP_MEMORY_SCOPE_AGENT);
        unsigned z;
        asm volatile("v_and_b32 %0, 0, %1" : "=v"(z) : "v"(tok));
        const int g = blockIdx.x / 32, ng = (gridDim.x + 31) / 32, in_g = (g == ng - 1) ? gridDim.x - g * 32 : 32;
        unsigned *c1 = cnt + 32 + g * 32;
        const unsigned t = __hip_atomic_fetch_add(c1 + z, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        int l = 0;
        if (t == (unsigned)in_g - 1) {
            __hip_atomic_store(c1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            unsigned z2;
            asm volatile("v_and_b32 %0, 0, %1" : "=v"(z2) : "v"(t));
            const unsigned t2 = __hip_atomic_fetch_add(cnt + z2, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (t2 == (unsigned)ng - 1) {
                __hip_atomic_store(cnt, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                l = 1;
            }
        }
        last = l;
    }
    __syncthreads();
    if (!last) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
    float v = 0;
    for (int i = threadIdx.x; i < (int)gridDim.x; i += 256)
        v += __uint_as_float(__hip_atomic_load((unsigned *)part + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
    v = block_sum(v);
    if (threadIdx.x == 0) out[0] = v;
}

// ---- every other column of an 8192 x 8192 matrix -------------------------------------------------------------
struct Raw {
    f32x4 a, b;
};
// the wave's 2 KiB run starting at wave_ptr: two 16-byte loads per lane, lanes 16 bytes apart
__device__ inline Raw ld_raw(const float *wave_ptr, int lane)
{
    const f32x4 *p = (const f32x4 *)wave_ptr;
    return Raw{__builtin_nontemporal_load(p + lane), __builtin_nontemporal_load(p + 64 + lane)};
}
// lane l gets the run's elements 8l, 8l + 2, 8l + 4, 8l + 6 (output columns 4l .. 4l + 3)
__device__ inline f32x4 regroup(const Raw &r, int lane)
{
    const int s = (2 * lane) & 63;
    const float x0 = __shfl(r.a[0], s), x1 = __shfl(r.a[2], s), x2 = __shfl(r.a[0], s + 1), x3 = __shfl(r.a[2], s + 1);
    const float y0 = __shfl(r.b[0], s), y1 = __shfl(r.b[2], s), y2 = __shfl(r.b[0], s + 1), y3 = __shfl(r.b[2], s + 1);
    return lane < 32 ? f32x4{x0, x1, x2, x3} : f32x4{y0, y1, y2, y3};
}
constexpr int S2_ROWS = 2; // rows per wave
enum { S2_ONE = 0, S2_PRED = 1, S2_TWO = 2 };
template <int KIND>
__global__ __launch_bounds__(64) void stride2_kernel(const float *A, const float *B, void *out_, int cin, int cout)
{
    const int cb = blockIdx.x % (cout / 4 / 64), rb = blockIdx.x / (cout / 4 / 64);
    const int lane = threadIdx.x, col = (cb * 64 + lane) * 4, wave_col = cb * 64 * 4;
    f32x4 row = {0, 0, 0, 0};
    if (KIND == S2_ONE) row = *(const f32x4 *)(B + col);
    Raw ra[S2_ROWS], rb2[S2_ROWS];
#pragma unroll
    for (int j = 0; j < S2_ROWS; ++j) {
        const size_t r = (size_t)rb * S2_ROWS + j;
        ra[j] = ld_raw(A + r * cin + 2 * wave_col, lane);
        if (KIND == S2_TWO) rb2[j] = ld_raw(B + r * cin + 2 * wave_col, lane);
    }
#pragma unroll
    for (int j = 0; j < S2_ROWS; ++j) {
        const size_t r = (size_t)rb * S2_ROWS + j;
        const f32x4 v = regroup(ra[j], lane);
        if (KIND == S2_PRED) {
            const unsigned o = (v[0] > 0) | ((v[1] > 0) << 8) | ((v[2] > 0) << 16) | ((v[3] > 0) << 24);
            __builtin_nontemporal_store(o, (unsigned *)((unsigned char *)out_ + r * cout + col));
        }
        else if (KIND == S2_TWO) stn((float *)out_ + r * cout + col, v * regroup(rb2[j], lane));
        else stn((float *)out_ + r * cout + col, v * row);
    }
}

// ---- 512-byte runs on both sides of a transposition, nothing transposed --------------------------------------
__global__ __launch_bounds__(512) void tile_runs_kernel(const float *in, float *out, int N)
{
    constexpr int T = 128;                 // tile edge; 32 threads x 16 bytes = one 512-byte run
    const int tiles = N / T;
    int b = blockIdx.x;
    const int ti = b % tiles;
    b /= tiles;
    const int tt = (b % tiles + ti) % tiles; // diagonal order, as the tile kernel walks its grid
    const int i0 = tt * T, j0 = ti * T;
    const int lv = threadIdx.x % 32, lr = threadIdx.x / 32; // 16 runs per pass, 8 passes
    f32x4 m[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) m[q] = ldn(in + (size_t)(j0 + q * 16 + lr) * N + i0 + lv * 4);
#pragma unroll
    for (int q = 0; q < 8; ++q) stn(out + (size_t)(i0 + q * 16 + lr) * N + j0 + lv * 4, m[q]);
}

struct Floor {
    const char *name, *about;
    double bytes;     // bytes the launch moves (reads + writes of whole lines), 0: none
    size_t workspace; // device bytes it needs
};
constexpr size_t N26 = (size_t)1 << 26, N24 = (size_t)1 << 24, SIDE = 8192, MAT = SIDE * SIDE * 4;
constexpr int READ_BLOCKS = 512;
const Floor FLOORS[] = {
    {"launch", "an empty kernel", 0, 256},
    {"bs_streams", "Black-Scholes kernel, arithmetic removed: 3 loads + 2 stores of 2^26 doubles", 40.0 * N26, 5 * 8 * N26 + (1 << 20)},
    {"bs_arithmetic", "Black-Scholes kernel, memory streams removed: 2^26 options priced", 0, 256},
    {"stream5_f64", "3 loads + 2 stores of 2^26 doubles, 256 threads x one 16-byte pack", 40.0 * N26, 5 * 8 * N26 + (1 << 20)},
    {"read_f32_2p24", "2^24 floats read once, one partial per block stored, no cross-block step", 4.0 * N24, 4 * N24 + (1 << 20)},
    {"read_f32_2p24_tickets", "2^24 floats read once, last block (two ticket levels) folds the partials", 4.0 * N24, 4 * N24 + (1 << 20)},
    {"stride2_one_input", "A[:, ::2] * row -> 8192 x 4096 floats (whole lines of A read)", MAT + MAT / 2.0, MAT + MAT / 2 + (1 << 20)},
    {"stride2_predicate", "A[:, ::2] > 0 -> 8192 x 4096 bytes", MAT + MAT / 8.0, MAT + MAT / 8 + (1 << 20)},
    {"stride2_two_inputs", "A[:, ::2] * B[:, ::2] -> 8192 x 4096 floats", 2.0 * MAT + MAT / 2.0, 2 * MAT + MAT / 2 + (1 << 20)},
    {"tile_runs_8192", "8192 x 8192 floats: 512-byte runs read, 512-byte runs written at the transposed tile", 2.0 * MAT, 2 * MAT},
};
constexpr int NFLOORS = sizeof(FLOORS) / sizeof(FLOORS[0]);
} // namespace

extern "C" {
int dpx_floors_count(void) { return NFLOORS; }
const char *dpx_floors_name(int i) { return (i >= 0 && i < NFLOORS) ? FLOORS[i].name : nullptr; }
const char *dpx_floors_about(int i) { return (i >= 0 && i < NFLOORS) ? FLOORS[i].about : nullptr; }
double dpx_floors_bytes(int i) { return (i >= 0 && i < NFLOORS) ? FLOORS[i].bytes : -1; }
size_t dpx_floors_workspace(int i) { return (i >= 0 && i < NFLOORS) ? FLOORS[i].workspace : 0; }

// fills the workspace with ordinary numbers (1.5f / a double near 0.0078 in every word pair) and clears counters
int dpx_floors_prepare(int i, void *workspace, void *stream)
{
    if (i < 0 || i >= NFLOORS || !workspace) return -1;
    hipLaunchKernelGGL(fill_kernel, dim3(2048), dim3(256), 0, (hipStream_t)stream, (u32x4 *)workspace, FLOORS[i].workspace / 16,
                       0x3fc00000u);
    if (FLOORS[i].name[0] == 'r') // the read kernels: partials and ticket counters live in the last MiB, zeroed
        hipLaunchKernelGGL(fill_kernel, dim3(64), dim3(256), 0, (hipStream_t)stream,
                           (u32x4 *)((char *)workspace + 4 * N24), (size_t)(1 << 20) / 16, 0u);
    return (int)hipGetLastError();
}

int dpx_floors_launch(int i, void *workspace, void *stream_)
{
    if (i < 0 || i >= NFLOORS || !workspace) return -1;
    hipStream_t s = (hipStream_t)stream_;
    char *w = (char *)workspace;
    const BlackScholesFn<double> fn{-0.1, 0.2 * 0.2 * 2, 0.25, 0.5, 1.0};
    constexpr int64_t CHUNK = (int64_t)BS_BLOCK * 2 * BS_PACKS;
    double *d[5];
    for (int k = 0; k < 5; ++k) d[k] = (double *)(w + k * (8 * N26 + 12288)); // staggered like the package's arrays
    float *A = (float *)w, *B = (float *)(w + MAT);
    switch (i) {
    case 0: hipLaunchKernelGGL(empty_kernel, dim3(1), dim3(64), 0, s); break;
    case 1:
        hipLaunchKernelGGL(black_scholes_f64_kernel<BS_STREAMS>, dim3((unsigned)(N26 / CHUNK)), dim3(BS_BLOCK), 0, s, fn, d[0],
                           d[1], d[2], d[3], d[4], (int64_t)N26, (int64_t)(N26 / CHUNK));
        break;
    case 2:
        hipLaunchKernelGGL(black_scholes_f64_kernel<BS_ARITHMETIC>, dim3((unsigned)(N26 / CHUNK)), dim3(BS_BLOCK), 0, s, fn,
                           (const double *)w, (const double *)w, (const double *)w, (double *)w, (double *)w, (int64_t)N26,
                           (int64_t)(N26 / CHUNK));
        break;
    case 3: hipLaunchKernelGGL(stream5_kernel, dim3((unsigned)(N26 / 512)), dim3(256), 0, s, d[0], d[1], d[2], d[3], d[4]); break;
    case 4: hipLaunchKernelGGL(read_kernel, dim3(READ_BLOCKS), dim3(256), 0, s, (const float *)w, N24, (float *)(w + 4 * N24)); break;
    case 5:
        hipLaunchKernelGGL(read_tickets_kernel, dim3(READ_BLOCKS), dim3(256), 0, s, (const float *)w, N24,
                           (float *)(w + 4 * N24 + 65536), (unsigned *)(w + 4 * N24), (float *)(w + 4 * N24 + 131072));
        break;
    case 6:
        hipLaunchKernelGGL(stride2_kernel<S2_ONE>, dim3((unsigned)((SIDE / 2 / 4 / 64) * (SIDE / S2_ROWS))), dim3(64), 0, s, A,
                           A, (void *)(w + MAT), (int)SIDE, (int)(SIDE / 2));
        break;
    case 7:
        hipLaunchKernelGGL(stride2_kernel<S2_PRED>, dim3((unsigned)((SIDE / 2 / 4 / 64) * (SIDE / S2_ROWS))), dim3(64), 0, s, A,
                           A, (void *)(w + MAT), (int)SIDE, (int)(SIDE / 2));
        break;
    case 8:
        hipLaunchKernelGGL(stride2_kernel<S2_TWO>, dim3((unsigned)((SIDE / 2 / 4 / 64) * (SIDE / S2_ROWS))), dim3(64), 0, s, A,
                           B, (void *)(w + 2 * MAT), (int)SIDE, (int)(SIDE / 2));
        break;
    case 9:
        hipLaunchKernelGGL(tile_runs_kernel, dim3((unsigned)((SIDE / 128) * (SIDE / 128))), dim3(512), 0, s, A, (float *)(w + MAT),
                           (int)SIDE);
        break;
    }
    return (int)hipGetLastError();
}
}
