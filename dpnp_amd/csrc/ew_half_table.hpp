// Unary functions of large contiguous float16 arrays through a table of all 65536 results.
//
// A float16 element brings 4 bytes of traffic with it, so a function stays at the HBM rate only up to a
// dozen vector instructions per element; the float routines behind sin, tanh, asinh ... take 20 to 60 and ran
// at 30-65 % of that rate.  The function has 65536 arguments, though.  Its results, computed once per function
// and device by the function's own kernel code, fill 128 KiB, which fit the 160 KiB of LDS of one CU: a
// block stages the table and then translates its share of the array, one 16-bit LDS read per element.
// Results are bit for bit those of the plain kernel.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>

namespace dpx {

constexpr int64_t HALF_TABLE_MIN = (int64_t)1 << 23; // elements from which the staging pays
constexpr int HALF_TABLE_ENTRIES = 65536;

// the table of unary op `op` on the current device: built on first use by `build(table, stream)`, which launches
// the kernel that writes the 65536 entries.  nullptr: not available (out of memory, a stream that is being
// captured into a graph before the table exists): the caller takes the plain kernel.
const uint16_t *half_table_for(int op, hipStream_t stream, hipError_t (*build)(uint16_t *, hipStream_t));
// out[i] = table[in[i]] for n float16 elements
hipError_t half_table_apply(const uint16_t *table, const void *in, void *out, int64_t n, hipStream_t stream);

} // namespace dpx
