// What the kernels of libsmr_gfx950 share beyond the public device header
// (include/smr_device.h: the bounded-spin flag protocol - send / wait / blockwise barrier):
// bf16 packing, the trace buffer's layout and the host-side error plumbing.  gfx950 only.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/smr.h"
#include "../../include/smr_device.h"

namespace smr {

// ---------------------------------------------------------------- host side
void set_last_error(const char* msg);
int fail(int code, const char* msg);            // records msg, returns code
int check_hip(hipError_t e, const char* what);  // 0 or the hip error (recorded)
uint64_t spin_limit_ticks();                    // current timeout in wall_clock64 ticks (0 = none)
uint64_t* trace_buffer(int64_t min_words);      // the registered trace buffer if it is large enough

// Layout of the optional trace buffer (uint64 words of the 100 MHz device clock):
//   [0 .. 63]                       producer: word i = time flag i was raised, word 63 = start
//   [64 + (wg*kTraceSteps + step)*4 + k]   GEMM workgroup wg, its step-th tile:
//        k = 0 tile picked, 1 flag wait over, 2 K loop done, 3 tile stored
constexpr int kTraceProducerWords = 64;
constexpr int kTraceSteps = 16;
constexpr int kTraceGemmWords = 256 * kTraceSteps * 4;

// ---------------------------------------------------------------- bf16
__device__ __forceinline__ float bf16_lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return __uint_as_float(w & 0xFFFF0000u); }

// fp32 -> bf16, round-to-nearest-even, NaN quieted; bit pattern in the low half.
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  uint32_t r = (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
  uint32_t q = (u >> 16) | 0x40u;
  return ((u & 0x7FFFFFFFu) > 0x7F800000u) ? q : r;
}
// Two at once through the hardware conversion (v_cvt_pk_bf16_f32: round-to-nearest-even,
// NaN quieted): one instruction instead of a dozen integer operations per pair.
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

}  // namespace smr
