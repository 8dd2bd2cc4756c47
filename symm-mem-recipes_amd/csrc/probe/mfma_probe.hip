// Measurement aid: what the matrix cores of this part sustain with nothing else going on.
//
// The published bf16 peak (2.5 PFLOP/s) assumes the top clock.  With every compute unit
// issuing v_mfma_f32_16x16x32_bf16 back to back on operands that look like real data the
// part's power management settles at a lower clock, so the figure a GEMM can be compared
// with - before any byte has moved - is lower.  This kernel is that loop: 64 accumulator
// fragments per wave (the GEMM's register tile), one wave per SIMD, operands taken once from
// a caller's buffer, no LDS or memory traffic inside the loop.  It reports the elapsed ticks
// of the GPU's constant 100 MHz clock and the elapsed shader cycles per workgroup.
//
// Built into a library of its own (libsmr_probe.so) that only the benchmark and its test
// load: it is no part of the C ABI of libsmr_gfx950.so.  No reference counterpart (the
// reference's launch metadata publishes flops for a profiler,
// symm_mem_recipes/triton_all_gather_matmul.py:59-69).
//
//   int smr_probe_mfma_only(values_dev, nvalues, workgroups, iters, ticks_dev, sink_dev, stream)
//     values_dev bf16 [nvalues]: operands, read once
//     ticks_dev  uint64 [2 * workgroups]: per workgroup, elapsed ticks of the 100 MHz clock and
//                elapsed shader clock cycles
//     sink_dev   float [256 * workgroups]: keeps the arithmetic alive
//     returns 0, -1 for a bad argument, or the hipError_t of the launch
//   FLOPs issued: workgroups * 4 waves * 64 * iters * 16384.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace smr_probe {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256, 1) void mfma_only_kernel(const uint16_t* __restrict__ values, int nvalues,
                                                           int iters, uint64_t* __restrict__ ticks,
                                                           float* __restrict__ sink) {
  bf16x8 a[8], b[8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      a[i][j] = __builtin_bit_cast(__bf16, values[(threadIdx.x * 8 + i * 2048 + j) % nvalues]);
      b[i][j] = __builtin_bit_cast(__bf16, values[(threadIdx.x * 8 + i * 2048 + j + 16384) % nvalues]);
    }
  f32x4 acc[64];
#pragma unroll
  for (int i = 0; i < 64; ++i) acc[i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  const uint64_t c0 = __builtin_readcyclecounter();
  const uint64_t w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int ni = 0; ni < 8; ++ni)
#pragma unroll
      for (int mi = 0; mi < 8; ++mi)
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[ni * 8 + mi]) : "v"(b[ni]), "v"(a[mi]));
  }
  const uint64_t c1 = __builtin_readcyclecounter();
  const uint64_t w1 = wall_clock64();
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < 64; ++i) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
  sink[blockIdx.x * 256 + threadIdx.x] = s;
  if (threadIdx.x == 0) {
    ticks[2 * blockIdx.x] = w1 - w0;
    ticks[2 * blockIdx.x + 1] = c1 - c0;
  }
}

}  // namespace smr_probe

extern "C" int smr_probe_mfma_only(const void* values_dev, int nvalues, int workgroups, int iters,
                                   uint64_t* ticks_dev, float* sink_dev, void* stream) {
  using namespace smr_probe;
  if (values_dev == nullptr || ticks_dev == nullptr || sink_dev == nullptr) return -1;
  if (nvalues < 1 || workgroups < 1 || workgroups > 1024 || iters < 1) return -1;
  hipLaunchKernelGGL(mfma_only_kernel, dim3(workgroups), dim3(256), 0, reinterpret_cast<hipStream_t>(stream),
                     reinterpret_cast<const uint16_t*>(values_dev), nvalues, iters, ticks_dev, sink_dev);
  return (int)hipGetLastError();
}
