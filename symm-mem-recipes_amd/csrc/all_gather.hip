// All-gather producer with progress flags.
//
// The reference drives copy engines from a side stream: one peer-to-peer copy
// per chunk, then a stream-ordered 32-bit write that raises the chunk's flag.
// On one GPU the same role is played by a deliberately small copy kernel: a few
// workgroups walk the chunks in the reference's order (sources rank+1, ...,
// rank+ws-1, rank), stream every chunk with 128-bit non-temporal loads and
// write-through stores, and the last workgroup to finish a chunk raises its flag.
// "Last" is decided by a per-chunk arrival counter, so the flag is raised once
// all of the chunk's bytes have been written and acknowledged.
//
// The grid is small on purpose: the consumer GEMM owns most compute units, and the
// caller sizes the producer to what the GEMM's grid leaves free.  The stores are
// written through the L2 (agent scope) and a chunk is published by waiting for their
// acknowledgement: releasing cached stores instead costs a cache-wide write-back per
// wave and chunk, which stalled the GEMM next to it (fused M=16384 N=3584 K=8192:
// 860 us with the write-backs, 760 us without).
#include "smr_internal.hpp"

namespace smr {

// 1024-thread workgroups: a producer workgroup then fills one compute unit by
// itself, so "num_workgroups" is also the number of compute units it can occupy
// whichever of the two kernels is dispatched first.
constexpr int kGatherThreads = 1024;
constexpr int kGatherDefaultWorkgroups = 8;
constexpr int kBesideDefaultWorkgroups = 256;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) u32x4 GlobalVec;

// 128-bit store at agent scope: written through the XCD's L2.  The idle slots behind it: the
// hardware reads a 128-bit store's data for two cycles after issue, and a vector instruction
// that writes one of the data registers in that time changes what is stored; the compiler
// spaces its own stores but does not look into assembly.
__device__ __forceinline__ void store_through(GlobalVec* p, u32x4 v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" : : "v"(p), "v"(v) : "memory");
}
// The same with the address as a uniform base and a 32-bit byte offset per lane.
__device__ __forceinline__ void store_through(uint8_t* base, uint32_t offset, u32x4 v) {
  asm volatile("global_store_dwordx4 %0, %1, %2 sc1\n\ts_nop 1" : : "v"(offset), "v"(v), "s"(base) : "memory");
}

// The timetable of a producer that copies beside the GEMM it feeds, in ticks of the 100 MHz
// clock (worked out on the host: a 64-bit division costs the kernel thirty registers, and its
// workgroups have to fit beside the GEMM's).  step = 0: none.
struct Timetable {
  uint64_t step;       // from one rank's chunks to the next rank's (margin taken off)
  uint64_t window;     // one chunk's share of a step
  uint64_t per_trip;   // one trip's (two loads per thread) share of a window
  int lead_ranks;      // ring positions below this one are copied flat out
};

// THREADS = 1024: a workgroup fills a compute unit (the producer beside a GEMM that leaves
// compute units free).  THREADS = 256: one wave per SIMD with a few dozen registers and no LDS -
// a workgroup that fits BESIDE a workgroup of the GEMM on the same compute unit (the GEMM's
// waves hold 424 of a SIMD's 512 registers per lane), so the copy needs no compute units of its
// own, like the copy engines it stands in for.  That form can copy on a timetable: a persistent
// GEMM takes its tiles in ring order, one pass of its grid after the other, so the chunks of the
// ranks whose tiles the first pass holds are due at once and are copied as fast as memory
// delivers them, and every later rank's are due one rank's share of the GEMM's time after
// the rank before it - they are copied two loads per thread at a time, each trip at its time.
// Not as fast as possible, because a copy that runs flat out on the compute unit of a GEMM
// workgroup slows that workgroup down (M=16384 N=3584 K=8192: the GEMM ends 2 % later).
template <int THREADS>
__global__ __launch_bounds__(THREADS) void all_gather_kernel(
    const uint64_t* __restrict__ buffer_ptrs, uint8_t* __restrict__ a_out,
    uint32_t* __restrict__ progress, uint32_t* __restrict__ counters, int rank, int world_size,
    int64_t chunk_vecs, int splits_per_rank, Timetable tt, uint64_t* trace) {
  constexpr int kGatherThreads = THREADS;
  if (trace != nullptr && blockIdx.x == 0 && threadIdx.x == 0) trace[kTraceProducerWords - 1] = wall_clock64();
  const uint64_t t_entry = tt.step != 0 ? wall_clock64() : 0;
  for (int step = 0; step < world_size; ++step) {
    const int src_rank = (rank + step + 1) % world_size;
    for (int split = 0; split < splits_per_rank; ++split) {
      const int idx = src_rank * splits_per_rank + split;
      const int nwg = (int)gridDim.x;
      // (ring position of the source: 1 for the next rank, ..., world_size for the own shard)
      const bool trickle = THREADS == 256 && tt.step != 0 && step + 1 >= tt.lead_ranks;
      // Addresses as a uniform base and a 32-bit byte offset per lane (the host keeps a chunk
      // below 2 GiB): one register per slot in flight instead of four, which is what lets
      // the slim form's workgroups fit beside the GEMM's.
      const uint8_t* src = (const uint8_t*)(uintptr_t)buffer_ptrs[src_rank] + (int64_t)split * chunk_vecs * 16;
      uint8_t* dst = a_out + (int64_t)idx * chunk_vecs * 16;
      const uint32_t chunk_bytes = (uint32_t)chunk_vecs * 16u;
      // 8 independent 16-byte slots per thread per trip: 128 KiB in flight per
      // workgroup, which is what one compute unit needs to stream at its share
      const uint32_t stride = (uint32_t)nwg * kGatherThreads * 16u;
      uint32_t i = ((uint32_t)blockIdx.x * kGatherThreads + threadIdx.x) * 16u;
      auto load = [&](uint32_t off) { return __builtin_nontemporal_load((const GlobalVec*)(uintptr_t)(src + off)); };
      auto store = [&](uint32_t off, u32x4 v) { store_through(dst, off, v); };
      if (trickle) {
        // The timetable: the ranks at ring positions below lead_ranks are in the GEMM's first
        // pass (copied flat out, above); the rank at position r is due a step after the rank
        // before it, so its chunks are spread over [r - lead_ranks, r - lead_ranks + 1) steps
        // from the kernel's start (a step is shortened by an eighth as a margin).  A trip whose
        // time has come already (the first ranks took longer than planned, or the estimate was
        // short) does not wait, so a producer that is behind copies flat out until it is not.
        // Two loads per thread and trip: single loads fall behind the GEMM's need at any pace,
        // and a burst of eight fills the memory pipeline that the GEMM workgroup on the same
        // compute unit feeds its tiles through.
        uint64_t due = t_entry + tt.step * (uint64_t)(step + 1 - tt.lead_ranks) + tt.window * (uint64_t)split;
        for (; i + stride < chunk_bytes; i += 2 * stride) {
          while (wall_clock64() < due) __builtin_amdgcn_s_sleep(8);     // (ends: the clock runs, `due` does not)
          due += tt.per_trip;
          const u32x4 v0 = load(i), v1 = load(i + stride);
          store(i, v0);
          store(i + stride, v1);
        }
      }
      for (; i + 7 * stride < chunk_bytes; i += 8 * stride) {
        u32x4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = load(i + u * stride);
#pragma unroll
        for (int u = 0; u < 8; ++u) store(i + u * stride, v[u]);
      }
      // what is left of the chunk (all of a small one): up to four slots in flight together too -
      // one after the other they were as many trips to memory and back per chunk
      for (; i < chunk_bytes; i += 4 * stride) {
        u32x4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u)
          if (i + u * stride < chunk_bytes) v[u] = load(i + u * stride);
#pragma unroll
        for (int u = 0; u < 4; ++u)
          if (i + u * stride < chunk_bytes) store(i + u * stride, v[u]);
      }
      // publish: the stores went through to where every XCD sees them, so a thread
      // only has to wait for their acknowledgement - no cache-wide write-back, which
      // two thousand waves per chunk would queue up for.  Then the workgroup meets,
      // one thread counts the arrival, and the last arrival raises the flag.
      wait_stores_acknowledged();
      __syncthreads();
      if (threadIdx.x == 0) {
        const uint32_t prev =
            __hip_atomic_fetch_add(&counters[idx], 1u, __ATOMIC_RELAXED, kScope);
        if (prev + 1u == (uint32_t)nwg) {
          __hip_atomic_store(&counters[idx], 0u, __ATOMIC_RELAXED, kScope);
          __hip_atomic_store(&progress[idx], 1u, __ATOMIC_RELAXED, kScope);
          if (trace != nullptr && idx < kTraceProducerWords - 1) trace[idx] = wall_clock64();
        }
      }
    }
  }
}

// The same gather with nobody watching the flags on the way: every thread's slot is
// copied in all chunks at once (one load per chunk in flight together), the stores are
// acknowledged once, and the last workgroup to arrive raises every flag.  Chunk by chunk
// a small shard is one slot per thread and chunk, i.e. one memory round trip after
// another; all at once it is a plain wide copy (8 x 4 MiB ahead of a 73 us GEMM: the
// pair takes 108 us chunk by chunk, 96 us at once).
__global__ __launch_bounds__(kGatherThreads) void all_gather_at_once_kernel(
    const uint64_t* __restrict__ buffer_ptrs, uint8_t* __restrict__ a_out,
    uint32_t* __restrict__ progress, uint32_t* __restrict__ counters, int world_size,
    int64_t chunk_vecs, int splits_per_rank) {
  const int chunks = world_size * splits_per_rank;
  const int64_t stride = (int64_t)gridDim.x * kGatherThreads;
  for (int64_t i = (int64_t)blockIdx.x * kGatherThreads + threadIdx.x; i < chunk_vecs; i += stride) {
    for (int c0 = 0; c0 < chunks; c0 += 8) {
      // (a group past the last chunk is skipped: the condition is the same for every lane)
      u32x4 v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int idx = c0 + u;
        if (idx < chunks) {
          const GlobalVec* src = (const GlobalVec*)(uintptr_t)buffer_ptrs[idx / splits_per_rank] +
                                 (int64_t)(idx % splits_per_rank) * chunk_vecs;
          v[u] = __builtin_nontemporal_load(src + i);
        }
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int idx = c0 + u;
        if (idx < chunks) store_through((GlobalVec*)(uintptr_t)a_out + (int64_t)idx * chunk_vecs + i, v[u]);
      }
    }
  }
  wait_stores_acknowledged();
  __syncthreads();
  if (threadIdx.x == 0) {
    const uint32_t prev = __hip_atomic_fetch_add(&counters[0], 1u, __ATOMIC_RELAXED, kScope);
    if (prev + 1u == gridDim.x) {
      __hip_atomic_store(&counters[0], 0u, __ATOMIC_RELAXED, kScope);
      for (int idx = 0; idx < chunks; ++idx) __hip_atomic_store(&progress[idx], 1u, __ATOMIC_RELAXED, kScope);
    }
  }
}

}  // namespace smr

static int launch_gather(const uint64_t* buffer_ptrs_dev, void* a_out_dev, uint32_t* progress_dev,
                         uint32_t* counters_dev, int rank, int world_size, int64_t shard_bytes,
                         int splits_per_rank, int num_workgroups, void* stream, bool at_once,
                         bool beside = false, int64_t step_us = 0, int lead_ranks = 0) {
  using namespace smr;
  if (buffer_ptrs_dev == nullptr || a_out_dev == nullptr || progress_dev == nullptr ||
      counters_dev == nullptr)
    return fail(SMR_E_INVALID, "smr_all_gather_with_progress: null pointer");
  if (world_size < 1 || world_size > SMR_MAX_WORLD_SIZE || rank < 0 || rank >= world_size)
    return fail(SMR_E_INVALID, "smr_all_gather_with_progress: rank/world_size");
  if (splits_per_rank < 1 || shard_bytes < 0 || shard_bytes % splits_per_rank != 0)
    return fail(SMR_E_INVALID, "smr_all_gather_with_progress: shard must divide into the splits");
  const int64_t chunk_bytes = shard_bytes / splits_per_rank;
  if (chunk_bytes % 16 != 0 || (reinterpret_cast<uintptr_t>(a_out_dev) & 15u))
    return fail(SMR_E_INVALID, "smr_all_gather_with_progress: chunks must be 16-byte multiples");
  if (chunk_bytes > ((int64_t)1 << 31) - ((int64_t)1 << 28))       // (32-bit byte offsets, eight strides of slack)
    return fail(SMR_E_UNSUPPORTED, "smr_all_gather_with_progress: a chunk (shard / splits) beyond 1.75 GiB");
  if (num_workgroups < 0 || num_workgroups > 1024)
    return fail(SMR_E_INVALID, "smr_all_gather_with_progress: num_workgroups must be 0..1024");
  if (step_us < 0 || step_us > 1000000 || lead_ranks < 0)
    return fail(SMR_E_INVALID, "smr_all_gather_beside: step_us must be 0..1,000,000 and lead_ranks >= 0");
  const int nwg = num_workgroups == 0 ? (beside ? kBesideDefaultWorkgroups : kGatherDefaultWorkgroups) : num_workgroups;
  Timetable tt = {0, 0, 0, lead_ranks < 1 ? 1 : lead_ranks};
  if (beside && step_us > 0) {
    const int64_t trips = (chunk_bytes / 16 + 2 * (int64_t)nwg * 256 - 1) / (2 * (int64_t)nwg * 256);
    tt.step = (uint64_t)step_us * 100u * 7 / 8;                 // 100 MHz clock, an eighth of margin
    tt.window = tt.step / (uint64_t)splits_per_rank;
    tt.per_trip = tt.window / (uint64_t)(trips > 0 ? trips : 1);
  }
  if (at_once) {
    hipLaunchKernelGGL(all_gather_at_once_kernel, dim3(nwg), dim3(kGatherThreads), 0,
                       reinterpret_cast<hipStream_t>(stream), buffer_ptrs_dev,
                       reinterpret_cast<uint8_t*>(a_out_dev), progress_dev, counters_dev, world_size,
                       chunk_bytes / 16, splits_per_rank);
    return check_hip(hipGetLastError(), "smr_all_gather launch");
  }
  if (beside)
    hipLaunchKernelGGL(all_gather_kernel<256>, dim3(nwg), dim3(256), 0,
                       reinterpret_cast<hipStream_t>(stream), buffer_ptrs_dev,
                       reinterpret_cast<uint8_t*>(a_out_dev), progress_dev, counters_dev, rank,
                       world_size, chunk_bytes / 16, splits_per_rank, tt, trace_buffer(kTraceProducerWords));
  else
    hipLaunchKernelGGL(all_gather_kernel<kGatherThreads>, dim3(nwg), dim3(kGatherThreads), 0,
                       reinterpret_cast<hipStream_t>(stream), buffer_ptrs_dev,
                       reinterpret_cast<uint8_t*>(a_out_dev), progress_dev, counters_dev, rank,
                       world_size, chunk_bytes / 16, splits_per_rank, tt, trace_buffer(kTraceProducerWords));
  return check_hip(hipGetLastError(), "smr_all_gather_with_progress launch");
}

extern "C" int smr_all_gather_with_progress(const uint64_t* buffer_ptrs_dev, void* a_out_dev,
                                            uint32_t* progress_dev, uint32_t* counters_dev,
                                            int rank, int world_size, int64_t shard_bytes,
                                            int splits_per_rank, int num_workgroups, void* stream) {
  return launch_gather(buffer_ptrs_dev, a_out_dev, progress_dev, counters_dev, rank, world_size,
                       shard_bytes, splits_per_rank, num_workgroups, stream, false);
}

extern "C" int smr_all_gather_at_once(const uint64_t* buffer_ptrs_dev, void* a_out_dev,
                                      uint32_t* progress_dev, uint32_t* counters_dev, int rank,
                                      int world_size, int64_t shard_bytes, int splits_per_rank,
                                      int num_workgroups, void* stream) {
  return launch_gather(buffer_ptrs_dev, a_out_dev, progress_dev, counters_dev, rank, world_size,
                       shard_bytes, splits_per_rank, num_workgroups, stream, true);
}

extern "C" int smr_all_gather_beside(const uint64_t* buffer_ptrs_dev, void* a_out_dev, uint32_t* progress_dev,
                                     uint32_t* counters_dev, int rank, int world_size, int64_t shard_bytes,
                                     int splits_per_rank, int num_workgroups, int64_t step_us, int lead_ranks,
                                     void* stream) {
  return launch_gather(buffer_ptrs_dev, a_out_dev, progress_dev, counters_dev, rank, world_size,
                       shard_bytes, splits_per_rank, num_workgroups, stream, false, true, step_us, lead_ranks);
}
