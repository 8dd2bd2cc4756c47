// A kernel library of "somebody else's": compiled against include/ only (smr_device.h, smr.h),
// not against anything under the package's csrc/, and linked with nothing of libsmr_gfx950.so.
// It uses the public device functions the way the reference's kernels import the barrier from
// one another (symm_mem_recipes/triton_one_shot_all_reduce.py:9,70).
#include "smr_device.h"

namespace {

// ws * blocks workgroups; workgroup id -> (block = id / ws, rank = id % ws).  Every round a
// workgroup writes one word with plain stores, runs smr::blockwise_barrier (which publishes and
// acquires), and checks the words its ws partners wrote in that round.  Two copies of the
// words alternate by round parity: a partner can be one round ahead at most.
__global__ __launch_bounds__(64) void client_rounds_kernel(const uint64_t* signal_pad_ptrs, uint32_t* words,
                                                           uint32_t* mismatches, int world_size, int blocks,
                                                           int rounds, uint64_t limit_ticks, uint32_t* status) {
  const int block = blockIdx.x / world_size, rank = blockIdx.x % world_size;
  for (int r = 0; r < rounds; ++r) {
    uint32_t* copy = words + (size_t)(r & 1) * world_size * blocks;
    if (threadIdx.x == 0) copy[(size_t)rank * blocks + block] = (uint32_t)(r * 131 + rank * 7 + block + 1);
    if (!smr::blockwise_barrier(signal_pad_ptrs, (uint32_t)block, rank, world_size, limit_ticks, status)) return;
    if ((int)threadIdx.x < world_size) {
      const uint32_t got = copy[(size_t)threadIdx.x * blocks + block];
      if (got != (uint32_t)(r * 131 + (int)threadIdx.x * 7 + block + 1)) atomicAdd(mismatches, 1u);
    }
  }
}

// One workgroup: writes a payload word, then raises the flag (send_signal publishes).
__global__ void client_send_kernel(uint32_t* flag, uint32_t* payload, uint32_t value, uint64_t limit_ticks,
                                   uint32_t* status) {
  if (threadIdx.x == 0) {
    *payload = value;
    if (!smr::send_signal(flag, limit_ticks)) smr::report(status, SMR_ST_SEND_TIMEOUT, 0u, 0u, 0u);
  }
}

// One workgroup: waits for the flag (left set), every thread then reads the payload; thread 0
// consumes the flag with wait_signal_reset.
__global__ void client_wait_kernel(uint32_t* flag, const uint32_t* payload, uint32_t* out, uint64_t limit_ticks,
                                   uint32_t* status) {
  smr::wait_signal(flag, limit_ticks, status, 0u);
  out[threadIdx.x] = *payload;
  __syncthreads();
  if (threadIdx.x == 0 && !smr::wait_signal_reset(flag, limit_ticks))
    smr::report(status, SMR_ST_WAIT_TIMEOUT, 0u, 0u, 0u);
}

}  // namespace

extern "C" int client_barrier_rounds(const uint64_t* signal_pad_ptrs_dev, uint32_t* words_dev,
                                     uint32_t* mismatches_dev, int world_size, int blocks, int rounds,
                                     uint64_t limit_ticks, uint32_t* status_dev, void* stream) {
  if (world_size < 1 || world_size > SMR_MAX_WORLD_SIZE || blocks < 1 || world_size * blocks > 4096) return -1;
  hipLaunchKernelGGL(client_rounds_kernel, dim3(world_size * blocks), dim3(64), 0, (hipStream_t)stream,
                     signal_pad_ptrs_dev, words_dev, mismatches_dev, world_size, blocks, rounds, limit_ticks,
                     status_dev);
  return (int)hipGetLastError();
}

extern "C" int client_send_then_wait(uint32_t* flag_dev, uint32_t* payload_dev, uint32_t value, uint32_t* out64_dev,
                                     uint64_t limit_ticks, uint32_t* status_dev, void* send_stream,
                                     void* wait_stream) {
  hipLaunchKernelGGL(client_wait_kernel, dim3(1), dim3(64), 0, (hipStream_t)wait_stream, flag_dev, payload_dev,
                     out64_dev, limit_ticks, status_dev);
  hipLaunchKernelGGL(client_send_kernel, dim3(1), dim3(64), 0, (hipStream_t)send_stream, flag_dev, payload_dev,
                     value, limit_ticks, status_dev);
  return (int)hipGetLastError();
}
