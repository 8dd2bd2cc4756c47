// Blockwise barrier and signal-pad kernels.
//
// smr_barrier runs the all-to-all CAS handshake (send 0->1 on every peer's pad,
// consume 1->0 on the own pad) for `rounds` back-to-back rounds; the pads are
// all-zero again after every round, so nothing is reset from the host.
//
// smr_signal_round adds a payload: in every round workgroup (rank r, block b)
// publishes a chunk into rank r's symmetric buffer, handshakes with the other
// ranks' block b, then reads and checksums all chunks of block b.  Chunks
// alternate between two halves of the buffer by round parity; a peer can only
// be one round ahead (it needs this workgroup's next flag to go further), so the
// half being read is never the half being overwritten.
//
// Workgroup id -> (block = id / ws, rank = id % ws): the ws partners of a
// handshake have adjacent ids, and with ws == 8 rank r's workgroups land on
// XCD r, so every flag and every payload chunk crosses an XCD boundary like it
// would cross a link between GPUs.
#include "smr_internal.hpp"

namespace smr {

constexpr int kBarrierThreads = 64;
constexpr int kRoundThreads = 128;   // 2 waves: 16 workgroups fit a CU, so 8 x 304 are co-resident

// True when some workgroup already reported a failure: lets multi-round loops
// stop instead of paying one timeout per remaining round.  Uniform per
// workgroup (thread 0 samples, everybody reads the same LDS word).
__device__ __forceinline__ bool any_failure(uint32_t* status, uint32_t* lds_flag) {
  if (status == nullptr) return false;
  if (threadIdx.x == 0)
    *lds_flag = __hip_atomic_load(&status[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  const uint32_t v = *lds_flag;
  __syncthreads();
  return v != 0u;
}

__global__ __launch_bounds__(kBarrierThreads) void barrier_kernel(
    const uint64_t* __restrict__ signal_pad_ptrs, int rank, int world_size, int rounds,
    int order_memory, uint64_t limit_ticks, uint32_t* status) {
  __shared__ uint32_t failed;
  int block = blockIdx.x;
  if (rank < 0) {
    block = blockIdx.x / world_size;
    rank = blockIdx.x % world_size;
  }
  for (int r = 0; r < rounds; ++r) {
    if (!blockwise_barrier(signal_pad_ptrs, block, rank, world_size, limit_ticks, status,
                           order_memory != 0, order_memory != 0))
      break;
    if ((r & 63) == 63 && any_failure(status, &failed)) break;
  }
}

__global__ __launch_bounds__(kRoundThreads) void signal_round_kernel(
    const uint32_t* __restrict__ src, const uint64_t* __restrict__ buffer_ptrs,
    const uint64_t* __restrict__ signal_pad_ptrs, const uint32_t* __restrict__ expected_base,
    uint32_t* __restrict__ checksums, uint32_t* __restrict__ mismatches, int world_size,
    int num_blocks, int64_t chunk_words, int rounds, uint64_t limit_ticks, uint32_t* status) {
  __shared__ uint32_t failed;
  __shared__ uint32_t wave_sums[kRoundThreads / 64];
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

  const int block = blockIdx.x / world_size;
  const int rank = blockIdx.x % world_size;
  const int64_t chunk_vecs = chunk_words / 4;
  const u32x4* my_src =
      reinterpret_cast<const u32x4*>(src + ((size_t)rank * num_blocks + block) * chunk_words);
  const uint32_t expect0 = chunk_words ? expected_base[block] : 0u;
  const uint32_t per_round = (uint32_t)((uint64_t)world_size * (uint64_t)chunk_words);
  uint32_t last_sum = 0u;

  for (int r = 0; r < rounds; ++r) {
    const size_t half = (size_t)(r & 1) * (size_t)num_blocks * chunk_words;
    // produce
    if (chunk_vecs) {
      u32x4* dst = reinterpret_cast<u32x4*>(reinterpret_cast<uint32_t*>(buffer_ptrs[rank]) + half +
                                            (size_t)block * chunk_words);
      const uint32_t tag = (uint32_t)r;
      for (int64_t i = threadIdx.x; i < chunk_vecs; i += kRoundThreads) {
        u32x4 v = my_src[i];
        v.x += tag; v.y += tag; v.z += tag; v.w += tag;
        uint64_t* d = reinterpret_cast<uint64_t*>(dst + i);
        store_coherent(d, ((uint64_t)v.y << 32) | v.x);
        store_coherent(d + 1, ((uint64_t)v.w << 32) | v.z);
      }
      wait_stores_acknowledged();
    }
    // Publish + wait for all peers' chunks of this block.  The payload travels
    // with agent-coherent stores and loads, so the handshake itself needs no
    // cache write-back or invalidate.
    if (!blockwise_barrier(signal_pad_ptrs, block, rank, world_size, limit_ticks, status, false, false))
      break;
    // consume
    if (chunk_vecs) {
      uint32_t s = 0u;
      for (int p = 0; p < world_size; ++p) {
        const u32x4* peer = reinterpret_cast<const u32x4*>(
            reinterpret_cast<const uint32_t*>(buffer_ptrs[p]) + half + (size_t)block * chunk_words);
        for (int64_t i = threadIdx.x; i < chunk_vecs; i += kRoundThreads) {
          const uint64_t* q = reinterpret_cast<const uint64_t*>(peer + i);
          const uint64_t lo = load_coherent(q), hi = load_coherent(q + 1);
          s += (uint32_t)lo + (uint32_t)(lo >> 32) + (uint32_t)hi + (uint32_t)(hi >> 32);
        }
      }
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
      if ((threadIdx.x & 63) == 0) wave_sums[threadIdx.x >> 6] = s;
      __syncthreads();
      if (threadIdx.x == 0) {
        uint32_t t = 0u;
        for (int w = 0; w < kRoundThreads / 64; ++w) t += wave_sums[w];
        last_sum = t;
        if (t != expect0 + per_round * (uint32_t)r) {
          atomicAdd(mismatches, 1u);
          report(status, SMR_ST_MISMATCH, rank, block, (uint32_t)r);
        }
      }
      __syncthreads();
    }
    if ((r & 15) == 15 && any_failure(status, &failed)) break;
  }
  if (threadIdx.x == 0) checksums[(size_t)rank * num_blocks + block] = last_sum;
}

__global__ void send_signal_kernel(uint32_t* addr, uint64_t limit_ticks, uint32_t* status) {
  if (threadIdx.x == 0 && !send_signal(addr, limit_ticks))
    report(status, SMR_ST_SEND_TIMEOUT, 0u, 0u, 0u);
}

__global__ void wait_signal_kernel(const uint32_t* addr, uint64_t limit_ticks, uint32_t* status) {
  wait_signal(addr, limit_ticks, status, 0u);
}

__global__ void wait_signal_reset_kernel(uint32_t* addr, uint64_t limit_ticks, uint32_t* status) {
  if (threadIdx.x == 0 && !wait_signal_reset(addr, limit_ticks))
    report(status, SMR_ST_WAIT_TIMEOUT, 0u, 0u, 0u);
  __syncthreads();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
}

__global__ void write_value32_kernel(uint32_t* addr, uint32_t value) {
  if (threadIdx.x == 0) __hip_atomic_store(addr, value, __ATOMIC_RELEASE, kScope);
}

}  // namespace smr

extern "C" {

int smr_barrier(const uint64_t* signal_pad_ptrs_dev, int rank, int world_size, int num_blocks,
                int rounds, int order_memory, uint32_t* status, void* stream) {
  using namespace smr;
  if (signal_pad_ptrs_dev == nullptr) return fail(SMR_E_INVALID, "smr_barrier: signal pads are NULL");
  if (world_size < 1 || world_size > SMR_MAX_WORLD_SIZE)
    return fail(SMR_E_INVALID, "smr_barrier: world_size must be 1..8");
  if (rank < -1 || rank >= world_size) return fail(SMR_E_INVALID, "smr_barrier: rank out of range");
  if (num_blocks < 1 || rounds < 0) return fail(SMR_E_INVALID, "smr_barrier: num_blocks/rounds");
  if ((int64_t)num_blocks * world_size > 8192)
    return fail(SMR_E_UNSUPPORTED, "smr_barrier: more than 8192 workgroups cannot be co-resident");
  if (rounds == 0) return 0;
  const unsigned grid = rank < 0 ? (unsigned)num_blocks * world_size : (unsigned)num_blocks;
  hipLaunchKernelGGL(barrier_kernel, dim3(grid), dim3(kBarrierThreads), 0,
                     reinterpret_cast<hipStream_t>(stream), signal_pad_ptrs_dev, rank, world_size,
                     rounds, order_memory, spin_limit_ticks(), status);
  return check_hip(hipGetLastError(), "smr_barrier launch");
}

int smr_signal_round(const uint32_t* src_dev, const uint64_t* buffer_ptrs_dev,
                     const uint64_t* signal_pad_ptrs_dev, const uint32_t* expected_base_dev,
                     uint32_t* checksums_dev, uint32_t* mismatches_dev, int world_size,
                     int num_blocks, int64_t chunk_bytes, int rounds, uint32_t* status,
                     void* stream) {
  using namespace smr;
  if (signal_pad_ptrs_dev == nullptr || checksums_dev == nullptr || mismatches_dev == nullptr)
    return fail(SMR_E_INVALID, "smr_signal_round: null pointer");
  if (world_size < 1 || world_size > SMR_MAX_WORLD_SIZE)
    return fail(SMR_E_INVALID, "smr_signal_round: world_size must be 1..8");
  if (num_blocks < 1 || rounds < 0 || chunk_bytes < 0 || chunk_bytes % 16 != 0)
    return fail(SMR_E_INVALID, "smr_signal_round: num_blocks/rounds/chunk_bytes");
  if (chunk_bytes > 0 && (src_dev == nullptr || buffer_ptrs_dev == nullptr || expected_base_dev == nullptr))
    return fail(SMR_E_INVALID, "smr_signal_round: payload pointers are NULL");
  if ((int64_t)num_blocks * world_size > 4096)
    return fail(SMR_E_UNSUPPORTED, "smr_signal_round: more than 4096 workgroups cannot be co-resident");
  if (rounds == 0) return 0;
  hipLaunchKernelGGL(signal_round_kernel, dim3((unsigned)num_blocks * world_size), dim3(kRoundThreads),
                     0, reinterpret_cast<hipStream_t>(stream), src_dev, buffer_ptrs_dev,
                     signal_pad_ptrs_dev, expected_base_dev, checksums_dev, mismatches_dev,
                     world_size, num_blocks, chunk_bytes / 4, rounds, spin_limit_ticks(), status);
  return check_hip(hipGetLastError(), "smr_signal_round launch");
}

int smr_send_signal(uint32_t* addr_dev, uint32_t* status, void* stream) {
  using namespace smr;
  if (addr_dev == nullptr) return fail(SMR_E_INVALID, "smr_send_signal: addr is NULL");
  hipLaunchKernelGGL(send_signal_kernel, dim3(1), dim3(64), 0, reinterpret_cast<hipStream_t>(stream),
                     addr_dev, spin_limit_ticks(), status);
  return check_hip(hipGetLastError(), "smr_send_signal launch");
}

int smr_wait_signal(const uint32_t* addr_dev, uint32_t* status, void* stream) {
  using namespace smr;
  if (addr_dev == nullptr) return fail(SMR_E_INVALID, "smr_wait_signal: addr is NULL");
  hipLaunchKernelGGL(wait_signal_kernel, dim3(1), dim3(64), 0, reinterpret_cast<hipStream_t>(stream),
                     addr_dev, spin_limit_ticks(), status);
  return check_hip(hipGetLastError(), "smr_wait_signal launch");
}

int smr_wait_signal_reset(uint32_t* addr_dev, uint32_t* status, void* stream) {
  using namespace smr;
  if (addr_dev == nullptr) return fail(SMR_E_INVALID, "smr_wait_signal_reset: addr is NULL");
  hipLaunchKernelGGL(wait_signal_reset_kernel, dim3(1), dim3(64), 0,
                     reinterpret_cast<hipStream_t>(stream), addr_dev, spin_limit_ticks(), status);
  return check_hip(hipGetLastError(), "smr_wait_signal_reset launch");
}

int smr_stream_write_value32(uint32_t* addr_dev, uint32_t value, void* stream) {
  using namespace smr;
  if (addr_dev == nullptr) return fail(SMR_E_INVALID, "smr_stream_write_value32: addr is NULL");
  hipLaunchKernelGGL(write_value32_kernel, dim3(1), dim3(64), 0, reinterpret_cast<hipStream_t>(stream),
                     addr_dev, value);
  return check_hip(hipGetLastError(), "smr_stream_write_value32 launch");
}

}  // extern "C"
