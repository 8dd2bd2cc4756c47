// One-shot all-reduce over the emulated peer buffers of one MI355X.
//
// Every thread owns 16-byte slots (8 bf16 or 4 fp32).  For a slot it issues one
// 128-bit load per peer, all in flight together, then adds the peers into an
// fp32 accumulator that starts at +0, strictly in rank order 0..ws-1 - the
// vector dimension runs across elements, never across ranks, so the result is
// bit-identical to a sequential fp32 sum - and stores one 128-bit result.
// The kernel is bound by HBM bandwidth: (ws + 1) * 16 bytes per slot.
//
// Role of the workgroups (`layout`):
//   kPlain     grid = nblocks: one rank's share, no handshake
//   kProxy     grid = nproxy + nblocks: the first nproxy workgroups play the other
//              ranks' halves of the handshake (8 lanes per block, no arithmetic)
//              and are dispatched first, so they are resident and spinning by
//              the time the rank's own workgroups arrive behind the barrier
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

template <int KIND, int WS, bool WRITE_ALL>
__global__ __launch_bounds__(kReduceMaxThreads) void one_shot_all_reduce_kernel(
    const uint64_t* __restrict__ buffer_ptrs, PeerPtrs by_value, const uint64_t* __restrict__ signal_pad_ptrs,
    SignalPads pads_by_value, Vec16* __restrict__ out, int64_t nvec, int rank, int layout, int nblocks, int do_barrier,
    uint64_t limit_ticks, uint32_t* status) {
  int block = blockIdx.x;
  const int nthreads = blockDim.x;
  int64_t lo = 0, hi = nvec;             // slots this rank reduces
  if (layout == kProxy) {
    const int per_proxy = nthreads >> 3;
    const int nproxy = (nblocks + per_proxy - 1) / per_proxy;
    if ((int)blockIdx.x < nproxy) {
      // Peer proxies: 8 lanes per block, lane j stands in for rank j's block b.
      const int b = blockIdx.x * per_proxy + (threadIdx.x >> 3);
      const int j = threadIdx.x & 7;
      if (b < nblocks && j < WS && j != rank) {
        const bool by_val = pads_by_value.p[0] != 0;
        uint32_t* to_rank = reinterpret_cast<uint32_t*>(by_val ? pads_by_value[rank] : signal_pad_ptrs[rank]) + (size_t)b * WS + j;
        uint32_t* from_rank = reinterpret_cast<uint32_t*>(by_val ? pads_by_value[j] : signal_pad_ptrs[j]) + (size_t)b * WS + rank;
        // one round per handshake of the rank's block (leading, and trailing if asked for)
        for (int round = 0; round < do_barrier; ++round) {
          // (a proxy publishes nothing: the peers' data are the work of earlier kernels)
          if (!send_signal_relaxed(to_rank, limit_ticks)) {
            report(status, SMR_ST_SEND_TIMEOUT, j, b, rank);
            break;
          }
          if (!wait_signal_reset(from_rank, limit_ticks)) {
            report(status, SMR_ST_WAIT_TIMEOUT, j, b, rank);
            break;
          }
        }
      }
      return;
    }
    block = blockIdx.x - nproxy;
  } else if (layout == kAllRanks) {
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

  // The peers' buffers were written by earlier kernels: nothing of this kernel to publish.
  // And nothing to invalidate: a launch starts from invalidated caches, and no workgroup reads
  // a peer's line before its own handshake (a line is never shared by two blocks: a block's
  // slots are nthreads * 16 bytes in a row), so no cache can hold a line of the peers' data
  // that is older than the handshake.  The invalidate an acquire stands for cost 1.3 us of a
  // 14 us launch.
  if (do_barrier) {
    if (pads_by_value.p[0] != 0) blockwise_barrier(pads_by_value, block, rank, WS, limit_ticks, status, false, false);
    else blockwise_barrier(signal_pad_ptrs, block, rank, WS, limit_ticks, status, false, false);
  }

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
  // Trailing handshake: nobody's buffer is overwritten (or, with write-back, read)
  // before every rank is through; it publishes this workgroup's stores.
  if (do_barrier == 2) {
    if (pads_by_value.p[0] != 0) blockwise_barrier(pads_by_value, block, rank, WS, limit_ticks, status, true, true);
    else blockwise_barrier(signal_pad_ptrs, block, rank, WS, limit_ticks, status, true, true);
  }
}

template <int KIND, int WS>
static int launch_ws(bool write_all, dim3 grid, int threads, hipStream_t s, const uint64_t* bp,
                     const PeerPtrs& pv, const uint64_t* sp, const SignalPads& spv,
                     Vec16* out, int64_t nvec, int rank, int layout, int nblocks, int do_barrier,
                     uint32_t* status) {
  const uint64_t lim = spin_limit_ticks();
  if (write_all)
    hipLaunchKernelGGL((one_shot_all_reduce_kernel<KIND, WS, true>), grid, dim3(threads), 0, s,
                       bp, pv, sp, spv, out, nvec, rank, layout, nblocks, do_barrier, lim, status);
  else
    hipLaunchKernelGGL((one_shot_all_reduce_kernel<KIND, WS, false>), grid, dim3(threads), 0, s,
                       bp, pv, sp, spv, out, nvec, rank, layout, nblocks, do_barrier, lim, status);
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
    const int per_proxy = threads / 8;
    grid = (unsigned)nblocks + (unsigned)((nblocks + per_proxy - 1) / per_proxy);
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
