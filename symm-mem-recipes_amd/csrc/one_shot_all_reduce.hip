// One-shot all-reduce over the emulated peer buffers of one MI355X.
//
// Every thread owns 16-byte slots (8 bf16 or 4 fp32).  For a slot it issues one
// 128-bit load per peer, all in flight together, then adds the peers into an
// fp32 accumulator that starts at +0, strictly in rank order 0..ws-1 - the
// vector dimension runs across elements, never across ranks, so the result is
// bit-identical to a sequential fp32 sum - and stores one 128-bit result.
// The kernel is bound by HBM bandwidth: (ws + 1) * 16 bytes per slot.
//
// The stores are held back: a thread keeps the results of several slots in registers and
// writes them in one go (8 slots; 64 in the kernel for large messages, which then holds a
// whole 64 MiB launch's results and stores them at the end).  Memory serves eight read
// streams at 6.8 TB/s and a write stream at 6.4 TB/s, but reads with a ninth of writes mixed
// in at 6.0 to 6.3 TB/s: a launch that reads first and writes afterwards pays for the two
// separately.
//
// Role of the workgroups (`layout`):
//   kPlain     grid = nblocks: one rank's share, no handshake
//   kProxy     grid = nblocks: one rank's share behind the handshake; the other ranks'
//              halves of the handshake, which nobody runs in the one-rank emulation, are
//              played by spare lanes of the wave that does the rank's own half
//   kAllRanks  grid = ws*nblocks: workgroup id -> (block = id / ws, rank = id % ws);
//              every emulated rank reduces into its own row of `out`
// In kAllRanks adjacent ids hold the partners of one handshake, so in-order
// dispatch makes every partner resident by the time a later workgroup starts:
// the spins end.
#include <atomic>

#include "smr_internal.hpp"

namespace smr {

enum ReduceLayout : int { kPlain = 0, kProxy = 1, kAllRanks = 2 };

constexpr int kReduceMaxThreads = 1024;
// Launch shape (threads per workgroup, cap on workgroups = barrier blocks per
// rank); smr_set_reduce_launch overrides the defaults.
// Defaults from a sweep on MI355X: one workgroup per compute unit streams best
// (8 contiguous read streams of 1 MiB-strided chunks keep the DRAM pages open);
// 512 threads below 32 MiB per buffer, 256 above.  0 = pick by size.
// Both knobs in one word (threads in the low half, cap in the high half): a launch reads the
// pair once, so a setter on another thread cannot hand it half of an update.
static std::atomic<uint32_t> g_reduce_launch{256u << 16};
struct ReduceLaunch {
  int threads, max_blocks;
};
static ReduceLaunch reduce_launch_knobs() {
  const uint32_t v = g_reduce_launch.load(std::memory_order_relaxed);
  return {(int)(v & 0xFFFFu), (int)(v >> 16)};
}

static int reduce_threads_for(const ReduceLaunch& knobs, int64_t nvec) {
  if (knobs.threads != 0) return knobs.threads;
  return nvec >= (int64_t)(32 << 20) / 16 ? 256 : 512;
}

static int reduce_blocks_for(const ReduceLaunch& knobs, int64_t nvec) {
  if (nvec <= 0) return 0;
  const int threads = reduce_threads_for(knobs, nvec);
  int64_t nb = (nvec + threads - 1) / threads;
  if (nb > knobs.max_blocks) nb = knobs.max_blocks;
  return nb < 1 ? 1 : (int)nb;
}

// The peers' buffer addresses as kernel arguments.  The reference's kernel reads them from a
// table in device memory (triton_one_shot_all_reduce.py:87): a dependent memory round trip
// in front of every thread's first data load, which a launch of a few microseconds notices.
// A host that knows the addresses passes them by value; all-zero = read the device table.
struct PeerPtrs {
  uint64_t p[SMR_MAX_WORLD_SIZE];
};

struct alignas(16) Vec16 {
  uint32_t w[4];
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
// Addresses handed over as integers would otherwise be treated as generic
// (flat) pointers; naming the global address space gives global_load/store.
typedef __attribute__((address_space(1))) u32x4 GlobalVec;

__device__ __forceinline__ Vec16 load_stream(const GlobalVec* p) {
  u32x4 t = __builtin_nontemporal_load(p);
  Vec16 v;
  v.w[0] = t.x; v.w[1] = t.y; v.w[2] = t.z; v.w[3] = t.w;
  return v;
}

__device__ __forceinline__ void store_stream(GlobalVec* p, const Vec16& v) {
  u32x4 t = {v.w[0], v.w[1], v.w[2], v.w[3]};
  __builtin_nontemporal_store(t, p);
}

// One correctly rounded bf16 add, canonical NaN: what add.bf16x2 computes per half
// (triton_one_shot_all_reduce.py:44-47).  The fp32 sum of two bf16 values is exact
// when their exponents differ by at most 16; beyond that the smaller one is less
// than 2^-9 of a bf16 ulp of the larger and no rounding of the fp32 sum can carry
// the result to another bf16, so rounding the fp32 sum once is the bf16 add.
__device__ __forceinline__ float add_bf16_step(float acc, float x) {
  const float s = acc + x;
  const uint32_t u = __float_as_uint(s);
  const uint32_t r = (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
  const uint32_t bits = ((u & 0x7FFFFFFFu) > 0x7F800000u) ? 0x7FFFu : r;
  return __uint_as_float(bits << 16);
}

// KIND follows the dtype codes: 0 bf16 with an fp32 accumulator, 1 fp32, 2 bf16 with
// the accumulator rounded to bf16 after every add.
template <int KIND, int WS>
__device__ __forceinline__ Vec16 sum_in_rank_order(const Vec16 (&v)[WS]) {
  Vec16 o;
  if constexpr (KIND == SMR_DTYPE_BF16_STEPWISE) {
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.0f;
#pragma unroll
    for (int r = 0; r < WS; ++r) {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        acc[2 * k] = add_bf16_step(acc[2 * k], bf16_lo(v[r].w[k]));
        acc[2 * k + 1] = add_bf16_step(acc[2 * k + 1], bf16_hi(v[r].w[k]));
      }
    }
#pragma unroll
    for (int k = 0; k < 4; ++k)
      o.w[k] = (__float_as_uint(acc[2 * k]) >> 16) | (__float_as_uint(acc[2 * k + 1]) & 0xFFFF0000u);
  } else if constexpr (KIND == SMR_DTYPE_BF16) {
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.0f;
#pragma unroll
    for (int r = 0; r < WS; ++r) {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        acc[2 * k] += bf16_lo(v[r].w[k]);
        acc[2 * k + 1] += bf16_hi(v[r].w[k]);
      }
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) o.w[k] = pack_bf16x2(acc[2 * k], acc[2 * k + 1]);
  } else {
    float acc[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[e] = 0.0f;
#pragma unroll
    for (int r = 0; r < WS; ++r) {
#pragma unroll
      for (int k = 0; k < 4; ++k) acc[k] += __uint_as_float(v[r].w[k]);
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) o.w[k] = __float_as_uint(acc[k]);
  }
  return o;
}

// blockwise_barrier for the one-rank emulation: the rank's half of block `block_id`'s handshake
// and, in the same wave and the same loop, the halves of the ws - 1 ranks that nobody runs.
// Lane = role * ws + peer.  Role 0: the rank sends to `peer` (CAS 0 -> 1 on the peer's pad);
// 1: the rank waits for `peer` (own pad); 2: `peer` sends to the rank (the rank's pad, the slot
// role 1 polls); 3: `peer` waits for the rank (the peer's pad, the slot role 0 raised).  One
// loop for all of them, as in blockwise_barrier: every wait depends on a send of a lane
// beside it.  `publish` / `acquire` as there.
template <int WS, typename Pads>
__device__ __forceinline__ bool barrier_with_stand_ins(const Pads& pads, uint32_t block_id, int rank,
                                                       uint64_t limit_ticks, uint32_t* status, bool publish,
                                                       bool acquire) {
  static_assert(4 * WS <= 64, "one wave plays all four roles");
  __syncthreads();
  const int lane = threadIdx.x;
  int bad = 0;
  if (lane < 64) {
    if (publish) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    // the consuming write of an earlier call on this slot has been performed
    else wait_stores_acknowledged();
    const int role = lane / WS, peer = lane % WS;
    if (role < 4 && !(role >= 2 && peer == rank)) {
      const bool is_send = (role & 1) == 0;
      const bool peers_pad = role == 0 || role == 3;          // else the rank's own pad
      uint32_t* pad = reinterpret_cast<uint32_t*>(pads[peers_pad ? peer : rank]);
      uint32_t* slot = pad + (size_t)block_id * WS + (peers_pad ? rank : peer);
      SpinClock clk(limit_ticks);
      uint32_t level = 0;
      bool ok = false;
      for (;;) {
        if (is_send) {
          uint32_t expected = 0u;
          ok = __hip_atomic_compare_exchange_strong(slot, &expected, 1u, __ATOMIC_RELAXED, __ATOMIC_RELAXED, kScope);
        } else {
          ok = __hip_atomic_load(slot, __ATOMIC_RELAXED, kScope) == 1u;
        }
        if (ok) break;
        backoff_sleep(level);
        if (clk.expired()) break;
      }
      if (!ok) {
        if (role < 2) report(status, is_send ? SMR_ST_SEND_TIMEOUT : SMR_ST_WAIT_TIMEOUT, rank, block_id, peer);
        else report(status, is_send ? SMR_ST_SEND_TIMEOUT : SMR_ST_WAIT_TIMEOUT, peer, block_id, rank);
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

// DEFER: results a thread holds back before it stores them (1 = each as it comes: messages of
// one or two slots per thread, and the all-ranks emulation, where holding back gained nothing -
// its time is the handshakes' fences).  The kernel with 64 takes a compute unit's registers
// for 256 threads.
template <int KIND, int WS, bool WRITE_ALL, int DEFER>
__global__ __launch_bounds__(DEFER > 16 ? 256 : kReduceMaxThreads) void one_shot_all_reduce_kernel(
    const uint64_t* __restrict__ buffer_ptrs, PeerPtrs by_value, const uint64_t* __restrict__ signal_pad_ptrs,
    SignalPads pads_by_value, Vec16* __restrict__ out, int64_t nvec, int rank, int layout, int nblocks, int do_barrier,
    uint64_t limit_ticks, uint32_t* status) {
  int block = blockIdx.x;
  const int nthreads = blockDim.x;
  int64_t lo = 0, hi = nvec;             // slots this rank reduces
  if (layout == kAllRanks) {
    block = blockIdx.x / WS;
    rank = blockIdx.x % WS;
    if constexpr (WRITE_ALL) {
      // two-shot: the rank reduces its own slice only and hands it to every peer
      lo = nvec * rank / WS;
      hi = nvec * (rank + 1) / WS;
    } else {
      out += (size_t)rank * nvec;
    }
  }

  // A handshake of this block: between real workgroups (all ranks in one launch), or with
  // stand-ins for the ranks that are not there.
  auto handshake = [&](bool publish, bool acquire) {
    const bool by_val = pads_by_value.p[0] != 0;
    if (layout == kProxy) {
      if (by_val) barrier_with_stand_ins<WS>(pads_by_value, block, rank, limit_ticks, status, publish, acquire);
      else barrier_with_stand_ins<WS>(signal_pad_ptrs, block, rank, limit_ticks, status, publish, acquire);
    } else {
      if (by_val) blockwise_barrier(pads_by_value, block, rank, WS, limit_ticks, status, publish, acquire);
      else blockwise_barrier(signal_pad_ptrs, block, rank, WS, limit_ticks, status, publish, acquire);
    }
  };

  // The peers' buffers were written by earlier kernels: nothing of this kernel to publish.
  // And nothing to invalidate: a launch starts from invalidated caches, and no workgroup reads
  // a peer's line before its own handshake (a line is never shared by two blocks: a block's
  // slots are nthreads * 16 bytes in a row), so no cache can hold a line of the peers' data
  // that is older than the handshake.  The invalidate an acquire stands for cost 1.3 us of a
  // 14 us launch.
  if (do_barrier) handshake(false, false);

  GlobalVec* src[WS];
  if (buffer_ptrs != nullptr) {
#pragma unroll
    for (int r = 0; r < WS; ++r) src[r] = (GlobalVec*)(uintptr_t)buffer_ptrs[r];
  } else {
#pragma unroll
    for (int r = 0; r < WS; ++r) src[r] = (GlobalVec*)(uintptr_t)by_value.p[r];
  }
  GlobalVec* dst = (GlobalVec*)(uintptr_t)out;

  const int64_t stride = (int64_t)nblocks * nthreads;
  if constexpr (DEFER > 1) {
    int64_t i = lo + (int64_t)block * nthreads + threadIdx.x;
    while (i < hi) {
      Vec16 held[DEFER];
      const int64_t first = i;
#pragma unroll
      for (int d = 0; d < DEFER; ++d) {
        if (i < hi) {
          Vec16 v[WS];
#pragma unroll
          for (int r = 0; r < WS; ++r) v[r] = load_stream(src[r] + i);
          held[d] = sum_in_rank_order<KIND, WS>(v);
          i += stride;
        }
      }
      if constexpr (WRITE_ALL) {
        // In place (a slot is read and written by the one thread that owns it), one peer's
        // buffer after the other: eight write streams side by side are slower than one at a
        // time (8 MiB per buffer: 26.7 -> 24.5 us).
#pragma unroll
        for (int r = 0; r < WS; ++r)
#pragma unroll
          for (int d = 0; d < DEFER; ++d)
            if (first + d * stride < hi) store_stream(src[r] + first + d * stride, held[d]);
      } else {
#pragma unroll
        for (int d = 0; d < DEFER; ++d)
          if (first + d * stride < hi) store_stream(dst + first + d * stride, held[d]);
      }
    }
  } else {
    for (int64_t i = lo + (int64_t)block * nthreads + threadIdx.x; i < hi; i += stride) {
      Vec16 v[WS];
#pragma unroll
      for (int r = 0; r < WS; ++r) v[r] = load_stream(src[r] + i);
      Vec16 o = sum_in_rank_order<KIND, WS>(v);
      if constexpr (WRITE_ALL) {
#pragma unroll
        for (int r = 0; r < WS; ++r) store_stream(src[r] + i, o);
      } else {
        store_stream(dst + i, o);
      }
    }
  }
  // Trailing handshake: nobody's buffer is overwritten (or, with write-back, read)
  // before every rank is through; it publishes this workgroup's stores.
  if (do_barrier == 2) handshake(true, true);
}

template <int KIND, int WS>
static int launch_ws(bool write_all, dim3 grid, int threads, hipStream_t s, const uint64_t* bp,
                     const PeerPtrs& pv, const uint64_t* sp, const SignalPads& spv,
                     Vec16* out, int64_t nvec, int rank, int layout, int nblocks, int do_barrier,
                     uint32_t* status) {
  const uint64_t lim = spin_limit_ticks();
#define SMR_REDUCE_LAUNCH(WA, D)                                                                          \
  hipLaunchKernelGGL((one_shot_all_reduce_kernel<KIND, WS, WA, D>), grid, dim3(threads), 0, s, bp, pv, sp, spv, \
                     out, nvec, rank, layout, nblocks, do_barrier, lim, status)
  // Results a thread holds back.  None for one or two slots per thread (nothing to hold back,
  // and the loop that could costs a launch of 5 us a quarter of a microsecond) and for the
  // all-ranks emulation; 64 beyond 16 slots per thread in workgroups of at most 256 threads
  // (the kernel is compiled for 256), but not for the stepwise sum (an order of magnitude more
  // arithmetic per slot: 64 unrolled copies are more code than the compiler keeps in
  // registers); otherwise 8.  Write-back to all peers, as many bytes written as read, has less
  // to gain: 9 % at 8 MiB per buffer, 4 % at 16 and 64 MiB.
  const int64_t per_thread = (nvec + (int64_t)nblocks * threads - 1) / ((int64_t)nblocks * threads);
  const bool deep = KIND != SMR_DTYPE_BF16_STEPWISE && threads <= 256 && per_thread > 16;
  const int held = (layout == kAllRanks || per_thread <= 2) ? 1 : (deep ? 64 : 8);
  if (held == 1) {
    if (write_all) SMR_REDUCE_LAUNCH(true, 1);
    else SMR_REDUCE_LAUNCH(false, 1);
  } else if (held == 8) {
    if (write_all) SMR_REDUCE_LAUNCH(true, 8);
    else SMR_REDUCE_LAUNCH(false, 8);
  } else if constexpr (KIND != SMR_DTYPE_BF16_STEPWISE) {
    if (write_all) SMR_REDUCE_LAUNCH(true, 64);
    else SMR_REDUCE_LAUNCH(false, 64);
  }
#undef SMR_REDUCE_LAUNCH
  return check_hip(hipGetLastError(), "smr_one_shot_all_reduce launch");
}

template <int KIND>
static int launch_dtype(int ws, bool write_all, dim3 grid, int threads, hipStream_t s, const uint64_t* bp,
                        const PeerPtrs& pv, const uint64_t* sp, const SignalPads& spv, Vec16* out, int64_t nvec, int rank, int layout,
                        int nblocks, int do_barrier, uint32_t* status) {
#define SMR_WS_CASE(W)                                                                          \
  case W:                                                                                       \
    return launch_ws<KIND, W>(write_all, grid, threads, s, bp, pv, sp, spv, out, nvec, rank, layout, nblocks, \
                              do_barrier, status);
  switch (ws) {
    SMR_WS_CASE(1) SMR_WS_CASE(2) SMR_WS_CASE(3) SMR_WS_CASE(4)
    SMR_WS_CASE(5) SMR_WS_CASE(6) SMR_WS_CASE(7) SMR_WS_CASE(8)
  }
#undef SMR_WS_CASE
  return fail(SMR_E_INVALID, "smr_one_shot_all_reduce: world_size must be 1..8");
}

}  // namespace smr

// Validation and launch behind both entry points: the peers' addresses come either from the
// device table (`buffer_ptrs_dev`) or, by value, from the host array `buffer_ptrs_host`.
static int reduce_entry(const uint64_t* buffer_ptrs_dev, const uint64_t* buffer_ptrs_host,
                        const uint64_t* signal_pad_ptrs_dev, const uint64_t* signal_pad_ptrs_host, void* out, int64_t numel, int dtype, int rank,
                        int world_size, int write_all, int barrier_mode, uint32_t* status, void* stream) {
  using namespace smr;
  if (dtype != SMR_DTYPE_BF16 && dtype != SMR_DTYPE_FP32 && dtype != SMR_DTYPE_BF16_STEPWISE)
    return fail(SMR_E_INVALID, "smr_one_shot_all_reduce: dtype must be bf16 (0), fp32 (1) or stepwise bf16 (2)");
  if (world_size < 1 || world_size > SMR_MAX_WORLD_SIZE)
    return fail(SMR_E_INVALID, "smr_one_shot_all_reduce: world_size must be 1..8");
  if (rank < -1 || rank >= world_size)
    return fail(SMR_E_INVALID, "smr_one_shot_all_reduce: rank out of range");
  const int per_vec = dtype == SMR_DTYPE_FP32 ? 4 : 8;
  if (numel < 0 || numel % per_vec != 0)
    return fail(SMR_E_INVALID, "smr_one_shot_all_reduce: The number of elements must be 128-bit aligned.");
  if (buffer_ptrs_dev == nullptr && buffer_ptrs_host == nullptr)
    return fail(SMR_E_INVALID, "smr_one_shot_all_reduce: the buffer address table is NULL");
  PeerPtrs pv = {};
  if (buffer_ptrs_host != nullptr) {
    for (int r = 0; r < world_size; ++r) {
      if (buffer_ptrs_host[r] == 0 || (buffer_ptrs_host[r] & 15u))
        return fail(SMR_E_INVALID, "smr_one_shot_all_reduce_addrs: buffer addresses must be non-zero and 16-byte aligned");
      pv.p[r] = buffer_ptrs_host[r];
    }
  }
  if (barrier_mode != SMR_BARRIER_NONE && barrier_mode != SMR_BARRIER_PROXY && barrier_mode != SMR_BARRIER_BOTH)
    return fail(SMR_E_INVALID, "smr_one_shot_all_reduce: unknown barrier_mode");
  if (barrier_mode != SMR_BARRIER_NONE && signal_pad_ptrs_dev == nullptr && signal_pad_ptrs_host == nullptr)
    return fail(SMR_E_INVALID, "smr_one_shot_all_reduce: signal pads required for the barrier");
  SignalPads spv = {};
  if (signal_pad_ptrs_host != nullptr && barrier_mode != SMR_BARRIER_NONE) {
    for (int r = 0; r < world_size; ++r) {
      if (signal_pad_ptrs_host[r] == 0 || (signal_pad_ptrs_host[r] & 3u))
        return fail(SMR_E_INVALID, "smr_one_shot_all_reduce_addrs: signal pad addresses must be non-zero and 4-byte aligned");
      spv.p[r] = signal_pad_ptrs_host[r];
    }
  }
  if (write_all && rank < 0 && barrier_mode != SMR_BARRIER_BOTH)
    return fail(SMR_E_INVALID, "smr_one_shot_all_reduce: the two-shot form (all ranks, write-back) needs SMR_BARRIER_BOTH");
  if (!write_all && out == nullptr)
    return fail(SMR_E_INVALID, "smr_one_shot_all_reduce: out is NULL");
  if (out != nullptr && (reinterpret_cast<uintptr_t>(out) & 15u))
    return fail(SMR_E_INVALID, "smr_one_shot_all_reduce: out must be 16-byte aligned");
  if (numel == 0) return 0;

  const ReduceLaunch knobs = reduce_launch_knobs();       // one consistent pair for the whole call
  const int64_t nvec = numel / per_vec;
  const int nblocks = reduce_blocks_for(knobs, nvec);
  const int threads = reduce_threads_for(knobs, nvec);
  const int do_barrier = barrier_mode == SMR_BARRIER_BOTH ? 2 : (barrier_mode != SMR_BARRIER_NONE ? 1 : 0);
  int layout = kPlain;
  unsigned grid = (unsigned)nblocks;
  if (rank < 0) {
    layout = kAllRanks;
    grid = (unsigned)nblocks * (unsigned)world_size;
  } else if (do_barrier) {
    layout = kProxy;
  }
  hipStream_t s = reinterpret_cast<hipStream_t>(stream);
  Vec16* o = reinterpret_cast<Vec16*>(out);
  const uint64_t* table = buffer_ptrs_host != nullptr ? nullptr : buffer_ptrs_dev;
  if (dtype == SMR_DTYPE_BF16)
    return launch_dtype<SMR_DTYPE_BF16>(world_size, write_all != 0, dim3(grid), threads, s, table, pv,
                                        signal_pad_ptrs_dev, spv, o, nvec, rank, layout, nblocks, do_barrier, status);
  if (dtype == SMR_DTYPE_BF16_STEPWISE)
    return launch_dtype<SMR_DTYPE_BF16_STEPWISE>(world_size, write_all != 0, dim3(grid), threads, s, table, pv,
                                                 signal_pad_ptrs_dev, spv, o, nvec, rank, layout, nblocks, do_barrier,
                                                 status);
  return launch_dtype<SMR_DTYPE_FP32>(world_size, write_all != 0, dim3(grid), threads, s, table, pv,
                                      signal_pad_ptrs_dev, spv, o, nvec, rank, layout, nblocks, do_barrier, status);
}

extern "C" {

int smr_set_reduce_launch(int threads, int max_blocks) {
  if (max_blocks == 0) max_blocks = 256;
  if (threads != 0 && (threads < 64 || threads > smr::kReduceMaxThreads || (threads & 63) != 0))
    return smr::fail(SMR_E_INVALID, "smr_set_reduce_launch: threads must be a multiple of 64 in 64..1024");
  if (max_blocks < 1 || max_blocks > 4096)
    return smr::fail(SMR_E_INVALID, "smr_set_reduce_launch: max_blocks must be 1..4096");
  smr::g_reduce_launch.store((uint32_t)threads | ((uint32_t)max_blocks << 16), std::memory_order_relaxed);
  return 0;
}

int smr_reduce_num_blocks(int64_t numel, int dtype) {
  const int per_vec = dtype == SMR_DTYPE_FP32 ? 4 : 8;
  if (numel <= 0) return 0;
  return smr::reduce_blocks_for(smr::reduce_launch_knobs(), numel / per_vec);
}

int smr_one_shot_all_reduce(const uint64_t* buffer_ptrs_dev, const uint64_t* signal_pad_ptrs_dev,
                            void* out, int64_t numel, int dtype, int rank, int world_size,
                            int write_all, int barrier_mode, uint32_t* status, void* stream) {
  return reduce_entry(buffer_ptrs_dev, nullptr, signal_pad_ptrs_dev, nullptr, out, numel, dtype, rank, world_size,
                      write_all, barrier_mode, status, stream);
}

int smr_one_shot_all_reduce_addrs(const uint64_t* buffer_ptrs_host, const uint64_t* signal_pad_ptrs_host,
                                  void* out, int64_t numel, int dtype, int rank, int world_size,
                                  int write_all, int barrier_mode, uint32_t* status, void* stream) {
  if (buffer_ptrs_host == nullptr)
    return smr::fail(SMR_E_INVALID, "smr_one_shot_all_reduce_addrs: buffer_ptrs_host is NULL");
  return reduce_entry(nullptr, buffer_ptrs_host, nullptr, signal_pad_ptrs_host, out, numel, dtype, rank, world_size,
                      write_all, barrier_mode, status, stream);
}

}  // extern "C"
