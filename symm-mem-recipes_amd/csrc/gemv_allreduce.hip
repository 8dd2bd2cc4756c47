// Split-K GEMV + all-reduce through signal-pad flags, emulated ranks on one GPU.
//
//   out[b, n] = bf16( ((0 + p_0[b,n]) + p_1[b,n]) + ... + p_{ws-1}[b,n] ),
//   p_r = x[:, shard r] @ W[shard r, :]   (fp32)
//
// The job is bound by reading W once (K*N*2 bytes).  W is row-major [K, N], so a
// row is N contiguous bf16: TPR threads cover a row segment with one 128-bit load
// each, and the 256/TPR thread groups of a workgroup stride over the K rows of
// their share, two rows at a time, with 4 to 16 independent loads in flight per
// thread.  x (at most 8 rows) is staged in LDS as pairs of consecutive k,
// transposed to [k/2][batch]; a byte permute pairs W[k][j] with W[k+1][j], and one
// v_dot2c_f32_bf16 per column and batch row does both multiply-adds (half the
// vector instructions of convert-and-FMA, which is what a batch of 8 was bound by).
//
// Workgroup id -> (sender = rank * sub + sub-shard, column block), column block
// fastest.  Every workgroup writes its fp32 partial, waits until the stores are
// acknowledged, raises flag[column block][sender] and counts itself in the column
// block's arrival word.  The workgroup that arrives last knows that every partial is in
// place: it consumes all flags (CAS 1 -> 0, so flags and arrival word are zero again on
// exit) and adds the partials in sender order, i.e. rank by rank.  Nobody spins on a
// flag that is not up yet, and the end of the kernel is two memory round trips behind the
// last partial instead of four.  The partials travel with agent-coherent stores and
// loads, so no cache write-back or invalidate surrounds the flags.
#include <atomic>
#include <cstdio>
#include <mutex>

#include "smr_internal.hpp"

namespace smr {

constexpr int kGemvThreads = 256;
constexpr int kGemvKChunk = 1024;            // K rows of x staged in LDS at a time

// Launch shape: TPR threads cover one row segment of TPR*8 columns (TPR*16
// contiguous bytes); the K rows of a rank's shard may be split into `sub`
// sub-shards, one workgroup each, when the column blocks alone do not fill the
// chip.  Measured on MI355X at K = N = 8192: 16 threads per segment (512
// workgroups, 64 of them combining) beat 64-thread segments at every batch size.
// smr_set_gemv_launch overrides.
// Both knobs in one word (threads per row in the low half, sub-shards in the high half), so
// that a launch reads a consistent pair with one load whoever sets them meanwhile.
static std::atomic<uint32_t> g_gemv_launch{16u};   // sub-shards 0 = pick so that >= 256 workgroups run
struct GemvLaunch {
  int tpr, sub;
  bool mfma;      // batches above 2 on the matrix cores (bit 15 of the low half set = off)
};
static GemvLaunch gemv_launch_knobs() {
  const uint32_t v = g_gemv_launch.load(std::memory_order_relaxed);
  return {(int)(v & 0x7FFFu), (int)(v >> 16), (v & 0x8000u) == 0};
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) u32x4 GlobalVec;
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

// What follows the multiplication, shared by both kernels.  `red` holds the four waves'
// partial sums as fp32 [wave][BR][kCols]; the workgroup adds them (wave order), writes its
// partial, raises its flag and counts itself in, and the workgroup that arrives last at the
// column block combines the partials of all senders in sender order.
template <int BR, int kCols>
__device__ __forceinline__ void publish_and_combine(const float* red, float* __restrict__ partials,
                                                    uint32_t* __restrict__ flags, uint16_t* __restrict__ out,
                                                    int batch, int N, int cblk, int sender, int senders,
                                                    uint64_t limit_ticks, uint32_t* status) {
  const int tid = threadIdx.x;
  auto red_at = [&](int w, int b, int c) { return red[((size_t)w * BR + b) * kCols + c]; };
  for (int c = tid; c < kCols; c += kGemvThreads) {
    const int col = cblk * kCols + c;
    if (col < N) {
      for (int b = 0; b < batch; ++b) {
        const float p = ((red_at(0, b, c) + red_at(1, b, c)) + red_at(2, b, c)) + red_at(3, b, c);
        store_coherent(&partials[((int64_t)sender * batch + b) * N + col], p);
      }
    }
  }

  // publish the partial: it was written through, so once every thread's stores
  // are acknowledged and the workgroup has met, one thread raises the flag (nobody waits
  // for that: the raise is a store-like atomic without a return value) and counts the
  // workgroup in; the count comes back and tells whether it was the last
  wait_stores_acknowledged();
  __syncthreads();
  uint32_t* my_flags = flags + (size_t)cblk * (senders + 1);
  __shared__ uint32_t arrived;
  if (tid == 0) {
    __hip_atomic_fetch_or(my_flags + sender, 1u, __ATOMIC_RELAXED, kScope);
    arrived = __hip_atomic_fetch_add(my_flags + senders, 1u, __ATOMIC_RELAXED, kScope);
  }
  __syncthreads();
  if (arrived + 1u != (uint32_t)senders) return;

  // Last arrival of the column block.  The last wave consumes the flags (all raised by now,
  // or a moment from landing: the wait is the protocol's bounded CAS 1 -> 0) and clears the
  // arrival word, while the other waves already add the partials in rank order (sub-shards
  // of a rank in order inside it).
  constexpr int kCombiners = kGemvThreads - 64;
  if (tid >= kCombiners) {
    const int lane = tid - kCombiners;
    for (int f = lane; f < senders; f += 64)
      if (!wait_signal_reset(my_flags + f, limit_ticks)) report(status, SMR_ST_WAIT_TIMEOUT, f, cblk, 0u);
    if (lane == 0) __hip_atomic_store(my_flags + senders, 0u, __ATOMIC_RELAXED, kScope);
    return;
  }
  // All of a thread's outputs at once: their partials are fetched eight senders at a time
  // (independent loads, a few dozen in flight per thread - one output after the other would
  // be one memory round trip after the other), then added strictly in sender order; the +0
  // terms that pad the last group cannot change a sum that starts from +0.
  constexpr int kOutputs = (8 * kCols + kCombiners - 1) / kCombiners;    // per thread at batch 8
  const int64_t plane = (int64_t)batch * N;
  const float* p[kOutputs];
  float a[kOutputs];
#pragma unroll
  for (int e = 0; e < kOutputs; ++e) {
    const int idx = tid + e * kCombiners;
    const int b = idx / kCols, col = cblk * kCols + idx % kCols;
    p[e] = (idx < batch * kCols && col < N) ? partials + (int64_t)b * N + col : nullptr;
    a[e] = 0.0f;
  }
  for (int r0 = 0; r0 < senders; r0 += 8) {
    float v[kOutputs][8];
#pragma unroll
    for (int e = 0; e < kOutputs; ++e)
#pragma unroll
      for (int u = 0; u < 8; ++u)
        v[e][u] = (p[e] != nullptr && r0 + u < senders) ? load_coherent(p[e] + (int64_t)(r0 + u) * plane) : 0.0f;
#pragma unroll
    for (int e = 0; e < kOutputs; ++e)
#pragma unroll
      for (int u = 0; u < 8; ++u) a[e] += v[e][u];
  }
#pragma unroll
  for (int e = 0; e < kOutputs; ++e)
    if (p[e] != nullptr) out[p[e] - partials] = (uint16_t)f32_to_bf16_bits(a[e]);
}

template <int B, int TPR>
__global__ __launch_bounds__(kGemvThreads) void gemv_allreduce_kernel(
    const uint16_t* __restrict__ x, const uint8_t* __restrict__ w, float* __restrict__ partials,
    uint32_t* __restrict__ flags, uint16_t* __restrict__ out, int batch, int K, int N,
    int world_size, int sub, uint64_t limit_ticks, uint32_t* status) {
  // Row pairs in flight per thread (two 128-bit loads each): fewer for larger
  // batches, whose 8*B accumulators would otherwise leave one wave per SIMD
  constexpr int kGemvUnroll = B >= 8 ? 2 : (B >= 4 ? 4 : 8);
  constexpr int kCols = TPR * 8;                         // columns per workgroup
  constexpr int kKGroups = kGemvThreads / TPR;           // row groups per workgroup
  constexpr int kKGroupsPerWave = 64 / TPR;
  // x staging and the cross-wave reduction never live at the same time: one buffer
  constexpr int kXsWords = kGemvKChunk / 2 * B, kRedFloats = (kGemvThreads / 64) * B * kCols;
  __shared__ __attribute__((aligned(16))) float smem[kXsWords > kRedFloats ? kXsWords : kRedFloats];
  // x as bf16 pairs of consecutive k: word [k/2][batch] = x[batch][k] | x[batch][k+1] << 16
  uint32_t (*xp)[B] = reinterpret_cast<uint32_t (*)[B]>(smem);
  float (*red)[B][kCols] = reinterpret_cast<float (*)[B][kCols]>(smem);

  // Column block fastest: workgroups with neighbouring ids read neighbouring 1 KiB
  // segments of the same rows, so the workgroups in flight together sweep whole
  // rows of W instead of segments that lie a power-of-two stride apart.
  const int senders = world_size * sub;
  const int cblocks = gridDim.x / senders;
  const int cblk = blockIdx.x % cblocks;
  const int sender = blockIdx.x / cblocks;               // rank-major, sub-shard-minor
  const int rank = sender / sub;
  const int tid = threadIdx.x;
  const int col_t = tid % TPR;
  const int kg = tid / TPR;
  const int col0 = cblk * kCols + col_t * 8;
  const bool col_ok = col0 < N;
  const int ks = K / world_size;                         // rows per rank
  const int kss = (ks + sub - 1) / sub;                  // rows per sub-shard
  const int k_begin = rank * ks + (sender % sub) * kss;
  int k_end = k_begin + kss;
  if (k_end > (rank + 1) * ks) k_end = (rank + 1) * ks;
  const int64_t row_bytes = (int64_t)N * 2;

  float acc[B][8];
#pragma unroll
  for (int b = 0; b < B; ++b)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[b][j] = 0.0f;

  for (int k0 = k_begin; k0 < k_end; k0 += kGemvKChunk) {
    const int kc = (k_end - k0) < kGemvKChunk ? (k_end - k0) : kGemvKChunk;
    // stage x[:, k0 .. k0+kc) as pairs, transposed to [k/2][batch]; zero past the end
#pragma unroll
    for (int b = 0; b < B; ++b) {
#pragma unroll
      for (int i = 0; i < kGemvKChunk / 2 / kGemvThreads; ++i) {
        const int kp = tid + i * kGemvThreads;
        const int k = 2 * kp;
        uint32_t lo = 0, hi = 0;
        if (b < batch && k < kc) lo = x[(int64_t)b * K + k0 + k];
        if (b < batch && k + 1 < kc) hi = x[(int64_t)b * K + k0 + k + 1];
        xp[kp][b] = lo | (hi << 16);
      }
    }
    __syncthreads();
    if (col_ok) {
      const __attribute__((address_space(1))) uint8_t* wp =
          (const __attribute__((address_space(1))) uint8_t*)(uintptr_t)(w + (int64_t)k0 * row_bytes +
                                                                      (int64_t)col0 * 2);
      const int pairs = (kc + 1) >> 1;
      for (int p = kg; p < pairs; p += kKGroups * kGemvUnroll) {
        u32x4 w0[kGemvUnroll], w1[kGemvUnroll];
#pragma unroll
        for (int u = 0; u < kGemvUnroll; ++u) {
          // rows past the end are re-read from the last valid row; their x is 0
          const int k = 2 * (p + u * kKGroups);
          const int r0 = k < kc ? k : kc - 1, r1 = k + 1 < kc ? k + 1 : kc - 1;
          w0[u] = __builtin_nontemporal_load((const GlobalVec*)(wp + (int64_t)r0 * row_bytes));
          w1[u] = __builtin_nontemporal_load((const GlobalVec*)(wp + (int64_t)r1 * row_bytes));
        }
#pragma unroll
        for (int u = 0; u < kGemvUnroll; ++u) {
          const int pp = p + u * kKGroups;
          const int pr = pp < kGemvKChunk / 2 ? pp : kGemvKChunk / 2 - 1;   // (its x words are 0 there)
          // (W[k][j], W[k+1][j]) as one bf16 pair per column: two byte permutes per word
          uint32_t wq[8];
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            wq[2 * q] = __builtin_amdgcn_perm(w1[u][q], w0[u][q], 0x05040100u);
            wq[2 * q + 1] = __builtin_amdgcn_perm(w1[u][q], w0[u][q], 0x07060302u);
          }
#pragma unroll
          for (int b = 0; b < B; ++b) {
            const bf16x2 xb = __builtin_bit_cast(bf16x2, pp < pairs ? xp[pr][b] : 0u);
#pragma unroll
            for (int j = 0; j < 8; ++j)
              acc[b][j] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, wq[j]), xb, acc[b][j], false);
          }
        }
      }
    }
    __syncthreads();
  }

  // combine the row groups: those of one wave by lane shuffles, the waves through LDS
#pragma unroll
  for (int b = 0; b < B; ++b)
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float v = acc[b][j];
#pragma unroll
      for (int off = TPR; off < 64; off <<= 1) v += __shfl_xor(v, off, 64);
      acc[b][j] = v;
    }
  if ((tid & 63) < TPR) {
#pragma unroll
    for (int b = 0; b < B; ++b)
#pragma unroll
      for (int j = 0; j < 8; ++j) red[tid >> 6][b][col_t * 8 + j] = acc[b][j];
  }
  __syncthreads();
  static_assert(kKGroupsPerWave * (kGemvThreads / 64) == kKGroups, "row groups = per wave x waves");
  publish_and_combine<B, kCols>(&red[0][0][0], partials, flags, out, batch, N, cblk, sender, senders, limit_ticks, status);
}

// ---------------------------------------------------------------------------
// The same job on the matrix cores, for batches whose multiply-adds would otherwise bind
// the kernel (8 rows of x: 33 us on the vector ALUs against 26 us for one row).
//
// v_mfma_f32_16x16x32_bf16 wants both operands with K running inside a lane; W has N
// running inside a row.  A wave therefore puts each 32 x 128 tile of W (32 K rows of its
// column block) into its own 8 KiB of LDS as it comes - row r at r * 256 bytes, the eight
// 32-byte column blocks of a row rotated by r so that the reads below spread over the
// banks - and reads it back transposed with ds_read_b64_tr_b16: within 16 lanes, lane i
// supplies the address of a 4-element chunk, and receives element i & 3 of the chunks of
// lanes i >> 2, 4 + (i >> 2), 8 + (i >> 2), 12 + (i >> 2).  With lane i pointing at row
// 4 * G + (i >> 2) (G = lane / 16), column 4 * (i & 3), that is column i of rows 4 * G .. + 3:
// half an operand.  The MFMA's K index is ours to assign, as long as x uses the same
// assignment: position jj of lane group G stands for tile row 16 * (jj >> 2) + 4 * G + (jj & 3).
// x (padded to 16 rows, the MFMA's M) is the other operand, straight from its LDS copy; the
// result fragment D[b][n] has the batch row in (lane / 16) * 4 + register and the column in
// lane % 16, so only the lanes below 32 carry real rows.
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) bf16x4 LdsBf16x4;
typedef __attribute__((address_space(3))) u32x4 LdsVec;
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) u32x2 LdsVec2;

constexpr int kMfmaCols = 128;                 // columns per workgroup: 8 blocks of 16
constexpr int kMfmaTileRows = 32;              // K rows per MFMA

// Needs whole tiles and 8-byte aligned pieces of x: the K rows of a workgroup a multiple of 32.
__global__ __launch_bounds__(kGemvThreads) void gemv_allreduce_mfma_kernel(
    const uint16_t* __restrict__ x, const uint8_t* __restrict__ w, float* __restrict__ partials,
    uint32_t* __restrict__ flags, uint16_t* __restrict__ out, int batch, int K, int N,
    int world_size, int sub, uint64_t limit_ticks, uint32_t* status) {
  constexpr int kTileBytes = kMfmaTileRows * kMfmaCols * 2;      // 8 KiB, also one wave's [16][128] fp32 sums
  __shared__ __attribute__((aligned(16))) uint8_t smem[4 * kTileBytes];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint32_t lds_tile = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) void*)smem + wave * kTileBytes;

  const int senders = world_size * sub;
  const int cblocks = gridDim.x / senders;
  const int cblk = blockIdx.x % cblocks;
  const int sender = blockIdx.x / cblocks;
  const int rank = sender / sub;
  const int ks = K / world_size;
  const int kss = ks / sub;                      // (a multiple of 32: the host checks)
  const int k_begin = rank * ks + (sender % sub) * kss;
  const int64_t row_bytes = (int64_t)N * 2;

  // this lane's 16 bytes of a tile row: columns 8c .. 8c+7 of the column block (clamped into
  // the matrix: the columns past N feed results that are never stored)
  const int c = lane & 15, rsub = lane >> 4;
  int col = cblk * kMfmaCols + c * 8;
  if (col > N - 8) col = N - 8;
  const int G = lane >> 4, i = lane & 15;
  const __attribute__((address_space(1))) uint8_t* wp =
      (const __attribute__((address_space(1))) uint8_t*)(uintptr_t)(w + (int64_t)k_begin * row_bytes + (int64_t)col * 2);
  // x: batch row i (zero beyond the batch), K positions 4G .. 4G+3 and 16 + 4G .. 16 + 4G+3 of a tile
  typedef __attribute__((address_space(1))) u32x2 GlobalVec2;
  const GlobalVec2* xp = (const GlobalVec2*)(uintptr_t)(x + (int64_t)(i < batch ? i : 0) * K + k_begin + 4 * G);
  const bool x_row = i < batch;

  f32x4 acc[8];
#pragma unroll
  for (int nb = 0; nb < 8; ++nb) acc[nb] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

  struct Tile {
    u32x4 v[8];
    u32x2 xlo, xhi;
  };
  const int ntiles = kss / kMfmaTileRows;
  auto load_tile = [&](Tile& tl, int t) {
#pragma unroll
    for (int u = 0; u < 8; ++u)
      tl.v[u] = __builtin_nontemporal_load((const GlobalVec*)(wp + (int64_t)(t * kMfmaTileRows + 4 * u + rsub) * row_bytes));
    tl.xlo = u32x2{0u, 0u};
    tl.xhi = u32x2{0u, 0u};
    if (x_row) {
      tl.xlo = xp[t * (kMfmaTileRows / 4)];
      tl.xhi = xp[t * (kMfmaTileRows / 4) + 4];
    }
  };
  auto multiply_tile = [&](const Tile& tl) {
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int r = 4 * u + rsub;
      *reinterpret_cast<LdsVec*>((uintptr_t)(lds_tile + r * 256 + ((((c >> 1) + r) & 7) << 5) + ((c & 1) << 4))) = tl.v[u];
    }
    const u32x4 xw = {tl.xlo.x, tl.xlo.y, tl.xhi.x, tl.xhi.y};
    const bf16x8 xf = __builtin_bit_cast(bf16x8, xw);
#pragma unroll
    for (int nb = 0; nb < 8; ++nb) {
      const int r0 = 4 * G + (i >> 2), r1 = 16 + r0;
      const bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
          reinterpret_cast<LdsBf16x4*>((uintptr_t)(lds_tile + r0 * 256 + (((nb + r0) & 7) << 5) + ((i & 3) << 3))));
      const bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
          reinterpret_cast<LdsBf16x4*>((uintptr_t)(lds_tile + r1 * 256 + (((nb + r1) & 7) << 5) + ((i & 3) << 3))));
      const bf16x8 wf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      acc[nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xf, wf, acc[nb], 0, 0, 0);
    }
  };
  // two tiles in turn: the next tile's loads are in flight while this one is multiplied
  Tile ta, tb;
  int t = wave;
  if (t < ntiles) load_tile(ta, t);
  while (t < ntiles) {
    const int t1 = t + 4;
    if (t1 < ntiles) load_tile(tb, t1);
    multiply_tile(ta);
    if (t1 >= ntiles) break;
    t = t1 + 4;
    if (t < ntiles) load_tile(ta, t);
    multiply_tile(tb);
  }

  // the wave's sums, [16 rows][128 columns] fp32, into its own tile buffer (nobody else's)
  float* red = reinterpret_cast<float*>(smem);
#pragma unroll
  for (int nb = 0; nb < 8; ++nb)
#pragma unroll
    for (int e = 0; e < 4; ++e) red[((size_t)wave * 16 + 4 * G + e) * kMfmaCols + nb * 16 + i] = acc[nb][e];
  __syncthreads();
  publish_and_combine<16, kMfmaCols>(red, partials, flags, out, batch, N, cblk, sender, senders, limit_ticks, status);
}

static int gemv_sub_for(const GemvLaunch& knobs, int N, int K, int world_size) {
  if (knobs.sub > 0) return knobs.sub;
  const int cols = knobs.tpr * 8;
  const int cblocks = (N + cols - 1) / cols;
  int sub = 1;
  while (sub < 8 && cblocks * world_size * sub < 256 && (K / world_size) / (sub * 2) >= 64) sub *= 2;
  return sub;
}

// Words [0, n) of `p` set to zero: a kernel, not a memset, so that a caller who captures
// the launch into a graph records kernel nodes only.
__global__ void gemv_clear_words_kernel(uint32_t* p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0u;
}

// Scratch of smr_gemv_allreduce_static: the flags, then the fp32 partials.  One copy per GPU the
// library runs on, held until the process ends.
constexpr int kStaticFlagWords = 4096;                               // one per workgroup at most
constexpr int64_t kStaticPartialBytes = (int64_t)4 << 20;
constexpr int64_t kStaticScratchBytes = kStaticFlagWords * 4 + kStaticPartialBytes;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// The device address of `scratch` on the current GPU.  The array's name is only a handle on
// the host; every GPU has its own copy at its own address, looked up once per device.
constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static unsigned char* g_scratch_ptr[kMaxDevices] = {};

static int static_scratch(unsigned char** out) {
  int dev = -1;
  if (int rc = check_hip(hipGetDevice(&dev), "smr_gemv_allreduce_static: hipGetDevice")) return rc;
  if (dev < 0 || dev >= kMaxDevices) return fail(SMR_E_UNSUPPORTED, "smr_gemv_allreduce_static: device index beyond 63");
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    if (int rc = check_hip(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)),
                           "smr_gemv_allreduce_static: hipGetSymbolAddress"))
      return rc;
    if (p == nullptr) return fail(SMR_E_INVALID, "smr_gemv_allreduce_static: no address for the scratch array");
    g_scratch_ptr[dev] = static_cast<unsigned char*>(p);
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

// Validation and launch shared by the entry points.  `flag_capacity` (words) and
// `partial_capacity` (bytes) bound what the kernel may touch of the two scratch arrays; a
// problem that needs more returns `too_small`.
static int launch_gemv(const char* who, const void* x_dev, const void* w_dev, float* partials_dev,
                       uint32_t* flags_dev, int64_t flag_capacity, int64_t partial_capacity, int too_small,
                       void* out_dev, int batch, int K, int N, int world_size, uint32_t* status, void* stream,
                       bool clear_flags) {
  char msg[160];
  auto bad = [&](int code, const char* what) {
    snprintf(msg, sizeof(msg), "%s: %s", who, what);
    return fail(code, msg);
  };
  if (x_dev == nullptr || w_dev == nullptr || partials_dev == nullptr || flags_dev == nullptr ||
      out_dev == nullptr)
    return bad(SMR_E_INVALID, "null pointer");
  if (world_size < 1 || world_size > SMR_MAX_WORLD_SIZE) return bad(SMR_E_INVALID, "world_size must be 1..8");
  if (batch < 1 || batch > 8) return bad(SMR_E_UNSUPPORTED, "batch must be 1..8");
  if (K <= 0 || N <= 0 || K % world_size != 0) return bad(SMR_E_INVALID, "K must split evenly over the ranks");
  if (N % 8 != 0 || (reinterpret_cast<uintptr_t>(w_dev) & 15u))
    return bad(SMR_E_UNSUPPORTED, "N must be a multiple of 8 and W 16-byte aligned");
  const GemvLaunch knobs = gemv_launch_knobs();          // one consistent pair for the whole call
  const int sub = gemv_sub_for(knobs, N, K, world_size);
  const int cblocks = (N + knobs.tpr * 8 - 1) / (knobs.tpr * 8);
  const int64_t grid64 = (int64_t)cblocks * world_size * sub;
  if (grid64 > 4096) return bad(SMR_E_UNSUPPORTED, "more than 4096 workgroups cannot be co-resident");
  const unsigned grid = (unsigned)grid64;
  const int64_t flag_words = (int64_t)cblocks * (world_size * sub + 1);
  if (flag_words > flag_capacity) return bad(too_small, "the flag array is too small (smr_gemv_flag_words)");
  if ((int64_t)world_size * sub * batch * N * 4 > partial_capacity)
    return bad(too_small, "the partial sums exceed their array (senders * batch * N * 4 bytes)");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const uint16_t* x = reinterpret_cast<const uint16_t*>(x_dev);
  const uint8_t* w = reinterpret_cast<const uint8_t*>(w_dev);
  uint16_t* out = reinterpret_cast<uint16_t*>(out_dev);
  const uint64_t lim = spin_limit_ticks();
  if (clear_flags) {
    hipLaunchKernelGGL(gemv_clear_words_kernel, dim3(((unsigned)flag_words + 255) / 256), dim3(256), 0, st, flags_dev,
                       (int)flag_words);
    if (int rc = check_hip(hipGetLastError(), who)) return rc;
  }
#define SMR_GEMV_LAUNCH(BP, TPR)                                                                   \
  hipLaunchKernelGGL((gemv_allreduce_kernel<BP, TPR>), dim3(grid), dim3(kGemvThreads), 0, st, x, w, \
                     partials_dev, flags_dev, out, batch, K, N, world_size, sub, lim, status)
#define SMR_GEMV_BATCH(TPR)                                                                        \
  do {                                                                                             \
    if (batch == 1) SMR_GEMV_LAUNCH(1, TPR);                                                       \
    else if (batch == 2) SMR_GEMV_LAUNCH(2, TPR);                                                  \
    else if (batch <= 4) SMR_GEMV_LAUNCH(4, TPR);                                                  \
    else SMR_GEMV_LAUNCH(8, TPR);                                                                  \
  } while (0)
  // (the matrix-core kernel works in whole 32-row tiles and reads x in 8-byte pieces)
  const bool whole_tiles = (K / world_size) % sub == 0 && ((K / world_size) / sub) % 32 == 0 &&
                           (reinterpret_cast<uintptr_t>(x_dev) & 7u) == 0;
  if (knobs.tpr == 16 && batch > 2 && knobs.mfma && whole_tiles)
    hipLaunchKernelGGL(gemv_allreduce_mfma_kernel, dim3(grid), dim3(kGemvThreads), 0, st, x, w, partials_dev,
                       flags_dev, out, batch, K, N, world_size, sub, lim, status);
  else if (knobs.tpr == 16) SMR_GEMV_BATCH(16);
  else SMR_GEMV_BATCH(64);
#undef SMR_GEMV_BATCH
#undef SMR_GEMV_LAUNCH
  return check_hip(hipGetLastError(), who);
}

}  // namespace smr

extern "C" {

int smr_set_gemv_launch(int threads_per_row, int sub_shards) {
  using namespace smr;
  if (threads_per_row == 0) threads_per_row = 16;
  if (threads_per_row != 16 && threads_per_row != 64)
    return fail(SMR_E_INVALID, "smr_set_gemv_launch: threads_per_row must be 16 or 64");
  if (sub_shards < 0 || sub_shards > 8)
    return fail(SMR_E_INVALID, "smr_set_gemv_launch: sub_shards must be 0..8");
  // (the matrix-core switch shares the word: keep it)
  uint32_t old = g_gemv_launch.load(std::memory_order_relaxed), want;
  do {
    want = (uint32_t)threads_per_row | (old & 0x8000u) | ((uint32_t)sub_shards << 16);
  } while (!g_gemv_launch.compare_exchange_weak(old, want, std::memory_order_relaxed));
  return 0;
}

int smr_set_gemv_matrix_cores(int on) {
  using namespace smr;
  uint32_t old = g_gemv_launch.load(std::memory_order_relaxed), want;
  do {
    want = on ? (old & ~0x8000u) : (old | 0x8000u);
  } while (!g_gemv_launch.compare_exchange_weak(old, want, std::memory_order_relaxed));
  return 0;
}

int smr_gemv_flag_blocks(int N) {
  const int cols = smr::gemv_launch_knobs().tpr * 8;
  return N <= 0 ? 0 : (N + cols - 1) / cols;
}

int smr_gemv_flag_words(int N, int K, int world_size) {
  if (N <= 0 || K <= 0 || world_size < 1 || world_size > SMR_MAX_WORLD_SIZE) return 0;
  const smr::GemvLaunch knobs = smr::gemv_launch_knobs();
  const int cols = knobs.tpr * 8;
  return ((N + cols - 1) / cols) * (world_size * smr::gemv_sub_for(knobs, N, K, world_size) + 1);
}

int smr_gemv_senders(int N, int K, int world_size) {
  if (N <= 0 || K <= 0 || world_size < 1 || world_size > SMR_MAX_WORLD_SIZE) return 0;
  return world_size * smr::gemv_sub_for(smr::gemv_launch_knobs(), N, K, world_size);
}

int smr_gemv_allreduce(const void* x_dev, const void* w_dev, float* partials_dev, int64_t partials_bytes,
                       uint32_t* flags_dev, int64_t flag_words, void* out_dev, int batch, int K, int N,
                       int world_size, uint32_t* status, void* stream) {
  return smr::launch_gemv("smr_gemv_allreduce", x_dev, w_dev, partials_dev, flags_dev, flag_words, partials_bytes,
                          SMR_E_INVALID, out_dev, batch, K, N, world_size, status, stream, false);
}

int smr_gemv_allreduce_static(const void* x_dev, const void* w_dev, void* out_dev, int batch, int K, int N,
                              int world_size, uint32_t* status, void* stream) {
  using namespace smr;
  unsigned char* base = nullptr;
  if (int rc = static_scratch(&base)) return rc;
  uint32_t* flags = reinterpret_cast<uint32_t*>(base);
  float* partials = reinterpret_cast<float*>(base + kStaticFlagWords * 4);
  // The array keeps whatever the last call left: a call that timed out may have left flags
  // up, so they are cleared (by a kernel) ahead of every launch.
  return launch_gemv("smr_gemv_allreduce_static", x_dev, w_dev, partials, flags, kStaticFlagWords,
                     kStaticPartialBytes, SMR_E_UNSUPPORTED, out_dev, batch, K, N, world_size, status, stream, true);
}

int64_t smr_gemv_static_scratch_bytes(void) { return smr::kStaticPartialBytes; }

}  // extern "C"
