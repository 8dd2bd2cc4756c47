/*
 * smr_device.h - the device side of the flag protocol, for HIP kernels of other libraries
 * (gfx950).  Header-only, device-only: nothing here touches the host, and nothing of
 * libsmr_gfx950.so needs to be linked.
 *
 * The reference's barrier and flag waits are device functions that other kernels import
 * (symm_mem_recipes/triton_one_shot_all_reduce.py:9 imports blockwise_barrier,
 * symm_mem_recipes/triton_all_gather_matmul.py:17 imports get_flat_tid); these are their
 * counterparts:
 *   smr::blockwise_barrier   symm_mem_recipes/triton_barrier.py:50-153
 *   smr::send_signal         the send half, triton_barrier.py:119-122
 *   smr::wait_signal_reset   the wait half, triton_barrier.py:124-129
 *   smr::wait_signal         symm_mem_recipes/triton_all_gather_matmul.py:72-95
 * (get_tid / get_flat_tid, triton_barrier.py:11-47, are threadIdx.x of a one-dimensional
 * workgroup.)  Differences from the reference, all in the caller's favour: every spin is
 * bounded by `limit_ticks` (ticks of the GPU's constant 100 MHz clock, 0 = unbounded as in the
 * reference) and a spin that expires writes a SMR_ST_* code into `status` (nullable; layout in
 * smr.h) and returns false instead of hanging; waiting lanes back off with s_sleep.
 *
 * Signal pads are zero-initialised uint32 arrays, one per rank; `signal_pad_ptrs` is a device
 * array of world_size uint64 addresses; the slot of (block, peer) is pad[block * world_size +
 * peer], as in triton_barrier.py:100-110.
 */
#ifndef SMR_DEVICE_H_
#define SMR_DEVICE_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "smr.h"

namespace smr {

// ---------------------------------------------------------------- status
__device__ __forceinline__ void report(uint32_t* status, uint32_t code, uint32_t a, uint32_t b,
                                       uint32_t c) {
  if (status == nullptr) return;
  uint32_t expected = 0u;
  if (__hip_atomic_compare_exchange_strong(&status[0], &expected, code, __ATOMIC_RELAXED,
                                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) {
    status[1] = a;
    status[2] = b;
    status[3] = c;
  }
}

// ---------------------------------------------------------------- flag protocol
// All flags live in ordinary device memory of one GPU, so agent scope is the
// widest scope that is ever needed here; a multi-GPU build over xGMI would use
// __HIP_MEMORY_SCOPE_SYSTEM on fine-grained peer mappings with the same code.
constexpr int kScope = __HIP_MEMORY_SCOPE_AGENT;

// ---------------------------------------------------------------- coherent data accesses
// A release fence at agent scope writes back the whole L2 of the XCD and an
// acquire fence invalidates it; with thousands of workgroups handing data over
// through flags those two cache-wide operations queue up behind each other and
// cost more than the hand-over itself.  Data that is handed over through a flag is
// therefore written with agent-scope (write-through) stores and read with
// agent-scope loads, which go to the level where all XCDs agree.  The producer
// then only has to wait until its stores are acknowledged before it raises the
// flag, and the consumer needs nothing but the flag: no write-back, no invalidate.
__device__ __forceinline__ void store_coherent(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, kScope);
}
__device__ __forceinline__ float load_coherent(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, kScope);
}
__device__ __forceinline__ void store_coherent(uint64_t* p, uint64_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, kScope);
}
__device__ __forceinline__ uint64_t load_coherent(const uint64_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, kScope);
}
// All of this thread's stores have been acknowledged (and nothing is moved across
// by the compiler).
__device__ __forceinline__ void wait_stores_acknowledged() {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// Spin helper: true while the caller may keep spinning.
struct SpinClock {
  uint64_t start, limit;
  __device__ __forceinline__ explicit SpinClock(uint64_t limit_ticks)
      : start(limit_ticks ? wall_clock64() : 0), limit(limit_ticks) {}
  __device__ __forceinline__ bool expired() const {
    return limit != 0 && (wall_clock64() - start) > limit;
  }
};

// Back-off between polls of a flag: 64 clocks at first, doubling up to 2048.
// Every poll of an agent-scope flag is a trip to memory, so a tight spin by
// thousands of waiting lanes would starve the very atomics they wait for.
__device__ __forceinline__ void backoff_sleep(uint32_t& level) {
  switch (level) {
    case 0: __builtin_amdgcn_s_sleep(1); break;
    case 1: __builtin_amdgcn_s_sleep(2); break;
    case 2: __builtin_amdgcn_s_sleep(4); break;
    case 3: __builtin_amdgcn_s_sleep(8); break;
    case 4: __builtin_amdgcn_s_sleep(16); break;
    default: __builtin_amdgcn_s_sleep(32); break;
  }
  if (level < 5) ++level;
}

// CAS `from` -> `to` until it succeeds.  Relaxed: the callers put one release
// fence before and one acquire fence after the whole handshake instead of paying
// a cache write-back on every attempt.
__device__ __forceinline__ bool spin_cas(uint32_t* addr, uint32_t from, uint32_t to,
                                         uint64_t limit_ticks) {
  SpinClock clk(limit_ticks);
  uint32_t level = 0;
  for (;;) {
    uint32_t expected = from;
    if (__hip_atomic_compare_exchange_strong(addr, &expected, to, __ATOMIC_RELAXED,
                                             __ATOMIC_RELAXED, kScope))
      return true;
    backoff_sleep(level);
    if (clk.expired()) return false;
  }
}

// Wait-side variant: poll with plain atomic loads and attempt the CAS only once
// the flag shows `from`, so that a waiting lane sends loads, not read-modify-write
// traffic, to memory.  (The transition itself must stay a read-modify-write: a
// plain store by the polling side would leave the line in its own L2, where its
// later polls would keep hitting the stale copy.)
__device__ __forceinline__ bool poll_then_cas(uint32_t* addr, uint32_t from, uint32_t to,
                                              uint64_t limit_ticks) {
  SpinClock clk(limit_ticks);
  uint32_t level = 0;
  for (;;) {
    if (__hip_atomic_load(addr, __ATOMIC_RELAXED, kScope) == from) {
      uint32_t expected = from;
      if (__hip_atomic_compare_exchange_strong(addr, &expected, to, __ATOMIC_RELAXED,
                                               __ATOMIC_RELAXED, kScope))
        return true;
    }
    backoff_sleep(level);
    if (clk.expired()) return false;
  }
}

// Release-CAS 0 -> 1 until it succeeds: publishes everything the calling
// thread (and, through a preceding workgroup barrier, its workgroup) wrote.
__device__ __forceinline__ bool send_signal(uint32_t* addr, uint64_t limit_ticks) {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
  return spin_cas(addr, 0u, 1u, limit_ticks);
}

// The same without the release fence, for data written with store_coherent and
// followed by wait_stores_acknowledged.
__device__ __forceinline__ bool send_signal_relaxed(uint32_t* addr, uint64_t limit_ticks) {
  return spin_cas(addr, 0u, 1u, limit_ticks);
}

// CAS 1 -> 0 until it succeeds (consumes and resets the flag).  Relaxed: the
// caller acquires afterwards, once, for the whole workgroup.
__device__ __forceinline__ bool wait_signal_reset(uint32_t* addr, uint64_t limit_ticks) {
  return poll_then_cas(addr, 1u, 0u, limit_ticks);
}

// Spin (one thread) until *addr == 1; the flag is left set.
__device__ __forceinline__ bool wait_flag_set(const uint32_t* addr, uint64_t limit_ticks) {
  SpinClock clk(limit_ticks);
  uint32_t level = 0;
  for (;;) {
    if (__hip_atomic_load(addr, __ATOMIC_RELAXED, kScope) == 1u) return true;
    backoff_sleep(level);
    if (clk.expired()) return false;
  }
}

// Whole-workgroup wait on a progress flag: thread 0 spins, everyone meets at the
// workgroup barrier, then every wave acquires so that its later loads cannot be
// served from lines cached before the flag was set.
__device__ __forceinline__ void wait_signal(const uint32_t* addr, uint64_t limit_ticks,
                                            uint32_t* status, uint32_t who) {
  if (threadIdx.x == 0) {
    if (!wait_flag_set(addr, limit_ticks)) report(status, SMR_ST_WAIT_TIMEOUT, who, blockIdx.x, 0u);
  }
  __syncthreads();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
}

// Blockwise barrier across the (emulated) ranks for one block index.
//   lane r < ws:         send: CAS 0 -> 1 on pad[r][block*ws + rank]
//   lane ws + r < 2*ws:  wait: until pad[rank][block*ws + r] == 1, then back to 0
// The two halves are independent memory operations, so they run on different
// lanes of the same wave and a round costs one atomic round trip, not two.  Pads
// are all-zero again afterwards.
//
// A wait lane polls with loads and consumes the flag with a read-modify-write whose result
// nobody waits for: only this lane ever takes the slot from 1 to 0, so once it has seen the
// 1 the transition cannot fail, and the workgroup goes on one memory round trip after the
// flag went up - as a CAS 1 -> 0 that finds the flag up does, but a CAS that comes too early
// costs three (CAS, poll, CAS) where this costs two.  The write is acknowledged before this
// lane polls the slot again: the next call starts by waiting for the wave's outstanding
// memory operations, which by then have long returned.  (A second poll in flight half a
// round trip behind the first was measured: the wave waits for both, 0.1 to 0.4 us slower.)
//
// Only the first wave touches memory-ordering machinery: the workgroup barrier in
// front collects every wave's earlier stores, then that one wave releases (when
// `publish` is set: the workgroup wrote data inside this kernel that the peers
// will read), flips the flags and acquires (when `acquire` is set: the workgroup, or
// anybody else on its compute unit or XCD, may have read the peers' data earlier inside
// this kernel, so that stale lines could sit in a cache); the closing workgroup barrier
// hands the acquired view to the other waves, which share its L1 and L2.  A cache
// write-back and an invalidate per wave would otherwise dominate the round.
// After the call every thread sees what the peers wrote before their call.
// Needs at least 2*ws threads.  Returns false (to every thread of the workgroup
// alike) when a spin timed out.
//
// `pads` is anything that yields rank r's pad address as pads[r]: the device table the
// reference passes (const uint64_t*), or SignalPads, the same addresses by value - kernel
// arguments, which saves the first wave a dependent load from memory in front of its atomics.
struct SignalPads {
  uint64_t p[SMR_MAX_WORLD_SIZE];
  __device__ __forceinline__ uint64_t operator[](int r) const {
    uint64_t v = p[0];
#pragma unroll
    for (int i = 1; i < SMR_MAX_WORLD_SIZE; ++i) v = (r == i) ? p[i] : v;
    return v;
  }
};

template <typename Pads>
__device__ __forceinline__ bool blockwise_barrier(const Pads& signal_pad_ptrs,
                                                  uint32_t block_id, int rank, int world_size,
                                                  uint64_t limit_ticks, uint32_t* status,
                                                  bool publish = true, bool acquire = true) {
  __syncthreads();
  const int lane = threadIdx.x;
  int bad = 0;
  if (lane < 64) {
    if (publish) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    // the consuming write of an earlier call on this slot has been performed
    else wait_stores_acknowledged();
    if (lane < 2 * world_size) {
      const bool is_send = lane < world_size;
      const int peer = is_send ? lane : lane - world_size;
      uint32_t* pad = reinterpret_cast<uint32_t*>(signal_pad_ptrs[is_send ? peer : rank]);
      uint32_t* slot = pad + (size_t)block_id * world_size + (is_send ? rank : peer);
      // One loop for both kinds of lane: the wait lane of the rank's own slot
      // depends on the send lane next to it, so neither may spin in a loop of its
      // own while the other is masked off.
      SpinClock clk(limit_ticks);
      uint32_t level = 0;
      bool ok = false;
      for (;;) {
        if (is_send) {
          uint32_t expected = 0u;
          ok = __hip_atomic_compare_exchange_strong(slot, &expected, 1u, __ATOMIC_RELAXED,
                                                    __ATOMIC_RELAXED, kScope);
        } else {
          ok = __hip_atomic_load(slot, __ATOMIC_RELAXED, kScope) == 1u;
        }
        if (ok) break;
        backoff_sleep(level);
        if (clk.expired()) break;
      }
      if (!ok) {
        report(status, is_send ? SMR_ST_SEND_TIMEOUT : SMR_ST_WAIT_TIMEOUT, rank, block_id, peer);
        bad = 1;
      } else if (!is_send) {
        __hip_atomic_fetch_and(slot, 0u, __ATOMIC_RELAXED, kScope);       // consume: 1 -> 0
      }
    }
    if (acquire) __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  }
  bad = __syncthreads_or(bad);
  return bad == 0;
}

}  // namespace smr

#endif /* SMR_DEVICE_H_ */
