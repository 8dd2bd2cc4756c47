// Flag-gated bf16 GEMM for the all-gather matmul:  C[M,N] = A[M,K] * B[N,K]^T.
//
// Shape of the kernel (MI355X / gfx950, 256 CUs in 8 XCDs, 160 KiB LDS per CU):
//   * persistent grid, one 256-thread workgroup per CU; a workgroup computes
//     BM x BN output tiles (256x256 by default), 4 waves in a 2x2 arrangement, so
//     a wave owns a (BM/2)x(BN/2) block held in fp32 accumulators and built from
//     v_mfma_f32_16x16x32_bf16 (the 32x32x16 form computes the same in as many cycles
//     but draws more power, and the clock of a GEMM this size is power-limited);
//   * both operands are K-contiguous, so a tile's K-slab (rows x 64 bf16 = 128 B
//     per row) is brought straight from global memory into LDS with 128-bit
//     direct-to-LDS loads (no staging registers).  LDS is a ring of five slots that
//     hold one slab each (2.5 slab pairs): while one pair is multiplied, up to three
//     slabs are landing, and only half of a pair's bytes are ever due within one
//     pair's time;
//   * an LDS row is 8 chunks of 16 B; chunk c of row r is stored at position
//     c ^ row_swizzle(r), which keeps the 128-bit fragment reads free of bank
//     conflicts;
//   * the MFMA is issued with the B fragment as its first operand, so a lane
//     ends up with 4 consecutive output columns of one row; the epilogue turns 32
//     rows at a time through LDS and stores whole rows;
//   * tiles are walked in the ready order of the all-gather: all tiles of the
//     local comm block first, then the comm blocks in ring order; a tile of a
//     non-local comm block first waits for that block's progress flag.  Within
//     one pass over the grid, XCD x (workgroups with id % 8 == x) takes a
//     contiguous run of the tile order - a patch about as wide as it is high - so
//     the workgroups that share an L2 also share A rows and B columns;
//   * a fused launch gathers the peers' shards itself (CopyJob): extra workgroups of the
//     same grid only copy, and a GEMM workgroup that finds its tile's chunk missing copies
//     along instead of spinning;
//   * the same kernel in e4m3fn (run_tile_fp8): the bytes move the same way, the
//     tile is built from v_mfma_f32_16x16x128_f8f6f4.
#include <atomic>
#include <type_traits>

#include "smr_internal.hpp"

namespace smr {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void LdsVoid;

constexpr int kGemmThreads = 256;
constexpr int kBK = 64;          // K extent of one slab (128 bytes per row)
constexpr int kRowBytes = kBK * 2;

struct GemmSchedule {
  int M, N, K;
  int rank, world_size, comm_block_m;
  int BM, BN;
  int grid;                      // persistent workgroups, a multiple of 8
  int steps;                     // trips of the busiest workgroup (passes over the tile order)
  int group_m;                   // row tiles per group of the tile order; divides the comm block's
  int acquire;                   // invalidate the caches behind every flag wait (smr_set_ag_matmul_acquire)
};

struct TileRef {
  int row0, col0;                // output tile origin
  int comm_block;                // progress flag index
  int local;                     // rows come from the local shard, no wait
  int a_row;                     // first row inside the source (shard-relative when local)
};

__host__ __device__ inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// Tile visited by workgroup `wg` in trip `step` of the grid; false when it has none in that trip.
// The comm blocks are visited in ring order starting at the local one, in passes of `grid`
// tiles; within a pass XCD x (workgroups with id % 8 == x) takes a contiguous run of the tile
// order.  The tile order is comm block (ring order), then group of row tiles, then column
// tile, then row tile: an XCD's run is then a patch about as wide as it is high, and
// the workgroups that share an L2 load the fewest distinct A and B slabs.
__host__ __device__ inline bool tile_for(const GemmSchedule& s, int wg, int step, TileRef& t) {
  const int cb_tiles_m = s.comm_block_m / s.BM;
  const int n_comm = s.M / s.comm_block_m;
  const int per_rank = n_comm / s.world_size;
  const int first_local = s.rank * per_rank;
  const int tn = ceil_div(s.N, s.BN);
  const int tiles_per_cb = cb_tiles_m * tn;
  const int total = n_comm * tiles_per_cb;
  const int start = step * s.grid;
  if (start >= total) return false;
  const int cnt = (total - start) < s.grid ? (total - start) : s.grid;
  const int per_xcd = (cnt + 7) >> 3;
  const int slot = wg >> 3;
  if (slot >= per_xcd) return false;
  const int in_pass = (wg & 7) * per_xcd + slot;
  if (in_pass >= cnt) return false;
  const int lin = start + in_pass;
  const int pos = lin / tiles_per_cb;
  const int rem = lin - pos * tiles_per_cb;
  // inside a comm block: groups of group_m row tiles, column by column inside a group
  const int per_group = s.group_m * tn;
  const int group = rem / per_group;
  const int in_group = rem - group * per_group;
  const int tile_n = in_group / s.group_m;
  const int tile_m = group * s.group_m + (in_group - tile_n * s.group_m);
  const int cb = (first_local + pos) % n_comm;
  t.comm_block = cb;
  t.row0 = cb * s.comm_block_m + tile_m * s.BM;
  t.col0 = tile_n * s.BN;
  t.local = (cb / per_rank) == s.rank;
  t.a_row = t.local ? t.row0 - first_local * s.comm_block_m : t.row0;
  return true;
}

// First tile of workgroup `wg` at or after trip `step`; advances `step` to that trip.
// False when the workgroup is done.
__host__ __device__ inline bool next_tile(const GemmSchedule& s, int wg, int& step, TileRef& t) {
  for (; step < s.steps; ++step)
    if (tile_for(s, wg, step, t)) return true;
  return false;
}

// Position swizzle of an LDS row: chunk c of slab row r is stored at position
// c ^ row_swizzle(r).  A 128-bit LDS read is served 16 lanes at a time, lanes
// 8g..8g+7 together with lanes 32+8g..32+8g+7, and those 16 lanes must fall into 16
// different 16-byte columns of the 256-byte bank row (two slab rows).  In a fragment
// read they are 8 consecutive rows at two chunks that differ by 2, so the 4 rows of
// equal parity must differ in swizzle bits 0 and 2: bits 0,1 = row bits 1,2 and
// bit 2 = row bit 2 ^ row bit 3.
__host__ __device__ inline int row_swizzle(int r) {
  return ((r >> 1) & 3) | ((((r >> 2) ^ (r >> 3)) & 1) << 2);
}

typedef __attribute__((address_space(3))) const bf16x8 LdsFrag;

__device__ __forceinline__ uint32_t lds_offset_of(const void* p) {
  return (uint32_t)(uintptr_t)(LdsVoid*)p;
}
__device__ __forceinline__ bf16x8 lds_read_frag(uint32_t addr) {
  return *reinterpret_cast<LdsFrag*>((uintptr_t)addr);
}
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void lds_write_b64(uint32_t addr, u32x2 v) {
  *reinterpret_cast<__attribute__((address_space(3))) u32x2*>((uintptr_t)addr) = v;
}
__device__ __forceinline__ u32x4 lds_read_b128(uint32_t addr) {
  return *reinterpret_cast<__attribute__((address_space(3))) const u32x4*>((uintptr_t)addr);
}

// A pointer that is the same in every lane, said so that it is kept in scalar
// registers (the tile loads take their base address from there).
__device__ __forceinline__ const uint8_t* uniform_ptr(const uint8_t* p) {
  const uint64_t v = (uint64_t)(uintptr_t)p;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
  return (const uint8_t*)(uintptr_t)(((uint64_t)hi << 32) | lo);
}

// One wave instruction of a direct-to-LDS tile load: 64 lanes x 16 B land at
// lds_dst + lane*16 (one 8-row group, 1 KiB); `voff` is the lane's byte offset
// from the uniform global base.
//
// Issued through inline assembly so that the compiler does not count these loads:
// it cannot tell which LDS bytes they write, so it would make every later
// fragment read wait for all of them.  All waits on these loads are explicit s_waitcnt vmcnt in the
// kernel (loads return in order, so "vmcnt(n)" leaves the n youngest in flight).
__device__ __forceinline__ void load_group(const uint8_t* base, uint32_t voff, uint32_t lds_dst) {
  // scalar base + 32-bit per-lane offset: no 64-bit address arithmetic per lane
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_dst), "v"(voff), "s"(base)
               : "memory", "m0");
}

// D += A x B on a 16x16x32 bf16 fragment pair, the accumulator named as an accumulation
// register.  Through the builtin the register allocator is free to keep an accumulator in
// either register file, and with 256 of them next to 128 fragment registers it would, on
// details of code far from the loop, park some in vector registers and move them back and
// forth inside the K loop (every result still right, 9 % slower).  The compiler still sees
// the operands, so the waits for the fragment reads that feed them are its own.
__device__ __forceinline__ void mfma_bf16(f32x4& acc, const bf16x8& first, const bf16x8& second) {
  asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(first), "v"(second));
}

// An MFMA with one tile load (see load_group) behind it, as one piece of assembly.  With one
// wave per SIMD every instruction between two MFMAs costs an issue slot, and a K loop trip
// carries sixteen loads: written apart from the MFMA each of them is a destination address
// computed into a register, that register moved into M0, an idle slot (M0 must be written one
// slot ahead of the load that uses it) and the load.  Here the M0 write stands ahead of the
// MFMA, which is the slot in between, and the loads of one slab after the first (FIRST = false)
// advance M0 by one load group (1 KiB) where it stands: two instructions per load instead of
// four.  M0 is live from one load of a slab to the next, which the compiler is not told; it has
// no use for M0 in these loops, and the ISA test fails if anything but this assembly names it.
template <bool FIRST>
__device__ __forceinline__ void mfma_bf16_load(f32x4& acc, const bf16x8& first, const bf16x8& second,
                                               const uint8_t* base, uint32_t voff, uint32_t lds_dst) {
  if constexpr (FIRST)
    asm volatile("s_mov_b32 m0, %3\n\tv_mfma_f32_16x16x32_bf16 %0, %1, %2, %0\n\tglobal_load_lds_dwordx4 %4, %5"
                 : "+a"(acc)
                 : "v"(first), "v"(second), "s"(lds_dst), "v"(voff), "s"(base)
                 : "memory", "m0");
  else
    asm volatile("s_addk_i32 m0, 0x400\n\tv_mfma_f32_16x16x32_bf16 %0, %1, %2, %0\n\tglobal_load_lds_dwordx4 %3, %4"
                 : "+a"(acc)
                 : "v"(first), "v"(second), "v"(voff), "s"(base)
                 : "memory", "m0", "scc");
}

// LDS holds a ring of five slots.  A K-slab of A and a K-slab of B take one slot each,
// in the order A0 B0 A1 B1 A2 ..., so slab number i lives in slot i % 5: the two slabs
// of the K step being multiplied, and up to three slabs that are landing.
constexpr int kRingSlots = 5;

template <int BM, int BN>
struct GemmTile {
  static constexpr int WM = BM / 2, WN = BN / 2;        // wave tile (2 x 2 waves)
  static constexpr int FM = WM / 16, FN = WN / 16;      // 16x16 fragments per wave tile
  static constexpr int GA = BM / 32, GB = BN / 32;      // 8-row load groups per wave and slab
  // BN <= BM in every configuration; a slot takes the larger slab.
  static constexpr int kSlotBytes = BM * kRowBytes;
  static constexpr int kLdsBytes = kRingSlots * kSlotBytes;
  static_assert(BN <= BM, "slot size is the A slab");
};

// Everything a tile needs that does not depend on the tile shape.
struct TileContext {
  int lane, wave;
  uint32_t row_stride;           // bytes between rows of A and of B
  int nk;                        // K-slabs
  uint32_t lds0;                 // LDS byte offset of the ring
  int N;
  uint8_t* c;
  uint64_t* tr;                  // trace record of this tile or null
};

// The first four slabs of a tile (A0 B0 A1 B1), global -> ring slots 0..3, no wait.
// Issued either at the start of the tile or, for every tile but a workgroup's first,
// by the previous tile between its K loop and its epilogue, so that the loads fly
// while the previous tile's results are being stored.  Slabs past the end of K repeat
// the last one; nobody reads them.
template <int BM, int BN>
__device__ __forceinline__ void issue_prologue(const TileContext& cx, const uint8_t* a_rows,
                                               const uint8_t* b_rows, int b_last) {
  using T = GemmTile<BM, BN>;
  const uint8_t* a_base = uniform_ptr(a_rows);
  const uint8_t* b_base = uniform_ptr(b_rows);
  constexpr int GA = T::GA, GB = T::GB;
  int ln = cx.lane;
  asm volatile("" : "+v"(ln));
  const int u = (ln & 7) ^ row_swizzle(ln >> 3);
#pragma unroll
  for (int idx = 0; idx < 4; ++idx) {
    const int k = (idx >> 1) < cx.nk ? (idx >> 1) : cx.nk - 1;
    const uint32_t dst = cx.lds0 + idx * T::kSlotBytes;
    if ((idx & 1) == 0) {
      const uint8_t* ak = a_base + (int64_t)k * kRowBytes;
#pragma unroll
      for (int j = 0; j < GA; ++j) {
        const int q = cx.wave * GA + j;
        load_group(ak, (uint32_t)(q * 8 + (ln >> 3)) * cx.row_stride + (uint32_t)((u ^ ((q & 1) << 2)) << 4),
                   dst + q * 1024);
      }
    } else {
      const uint8_t* bk = b_base + (int64_t)k * kRowBytes;
#pragma unroll
      for (int j = 0; j < GB; ++j) {
        const int q = cx.wave * GB + j;
        int r = q * 8 + (ln >> 3);
        r = r < b_last ? r : b_last;
        load_group(bk, (uint32_t)r * cx.row_stride + (uint32_t)((u ^ ((q & 1) << 2)) << 4), dst + q * 1024);
      }
    }
  }
}

// One output tile: C[row0 .. +BM, col0 .. +BN] = A rows (at a_base) x B rows (at b_base)^T.
// `preloaded`: the tile's first four slabs are already on their way into LDS.
// `between` runs after the K loop, when LDS is free again, and before the results
// are stored: the place to start the next tile's loads.
template <int BM, int BN, typename Between>
__device__ __forceinline__ void run_tile(const TileContext& cx, const TileRef& tile,
                                         const uint8_t* a_rows, const uint8_t* b_rows,
                                         bool preloaded, Between&& between) {
  using T = GemmTile<BM, BN>;
  const uint8_t* a_base = uniform_ptr(a_rows);
  const uint8_t* b_base = uniform_ptr(b_rows);
  constexpr int WM = T::WM, WN = T::WN, FM = T::FM, FN = T::FN, GA = T::GA, GB = T::GB;
  constexpr uint32_t kSlot = T::kSlotBytes;
  const int lane = cx.lane, wave = cx.wave;
  const int wm = wave >> 1, wn = wave & 1;
  const uint32_t row_stride = cx.row_stride;
  const int nk = cx.nk;
  const uint32_t lds0 = cx.lds0;
  uint64_t* tr = cx.tr;
  uint8_t* c = cx.c;
  struct { int N; } s = {cx.N};

  // The per-lane addresses below are recomputed for every tile from a laundered
  // copy of the lane id: kept loop-invariant they would stay live across the
  // register-hungry epilogue, be spilled there, and be reloaded from scratch
  // in the middle of the K loop.
  int ln = lane;
  asm volatile("" : "+v"(ln));
  // ---- per-lane fragment read addresses.  A 16x16x32 MFMA operand is 16 rows x 32
  // K: lane l holds row l & 15 and the 8 K values (one 16-byte chunk) number
  // l >> 4 of the four, so K step kk (0 or 1) wants chunk 4*kk + (l >> 4) of row
  // w*W + f*16 + (l & 15), whose swizzle depends on l & 15 only: one address per
  // operand and K step, the fragment row f is an immediate offset.  The addresses
  // point into the slots of the slab pair being read (slots 0 and 1 at first) and
  // move around the ring by a uniform amount once per slab pair.
  uint32_t a_fr[2], b_fr[2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) {
    const int pos = (4 * kk + (ln >> 4)) ^ row_swizzle(ln & 15);
    a_fr[kk] = lds0 + (uint32_t)((wm * WM + (ln & 15)) * kRowBytes + (pos << 4));
    b_fr[kk] = lds0 + kSlot + (uint32_t)((wn * WN + (ln & 15)) * kRowBytes + (pos << 4));
  }
  uint32_t a_at = 0, b_at = kSlot;       // ring offsets of the slab pair being read

  // ---- per-lane global offsets of the tile loads.  Load group q = wave*G + j holds
  // rows q*8 .. q*8+7; lane l carries row q*8 + (l >> 3) and the chunk whose swizzled
  // position is (l & 7): chunk = (l & 7) ^ row_swizzle(q*8 + (l >> 3)).
  const int u = (ln & 7) ^ row_swizzle(ln >> 3);
  uint32_t a_off[GA];
#pragma unroll
  for (int j = 0; j < GA; ++j) {
    const int q = wave * GA + j;
    a_off[j] = (uint32_t)(q * 8 + (ln >> 3)) * row_stride + (uint32_t)((u ^ ((q & 1) << 2)) << 4);
  }
  // rows of B past the last column are clamped: they feed outputs that are never stored
  const int b_last = s.N - 1 - tile.col0;
  uint32_t b_off[GB];
#pragma unroll
  for (int j = 0; j < GB; ++j) {
    const int q = wave * GB + j;
    int r = q * 8 + (ln >> 3);
    r = r < b_last ? r : b_last;
    b_off[j] = (uint32_t)r * row_stride + (uint32_t)((u ^ ((q & 1) << 2)) << 4);
  }

  f32x4 acc[FN][FM];
#pragma unroll
  for (int ni = 0; ni < FN; ++ni)
#pragma unroll
    for (int mi = 0; mi < FM; ++mi)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[ni][mi][e] = 0.0f;

  auto read_frags = [&](bf16x8 (&af)[FM], bf16x8 (&bf)[FN], int kk) {
#pragma unroll
    for (int mi = 0; mi < FM; ++mi)
      af[mi] = lds_read_frag(a_fr[kk] + mi * (16 * kRowBytes));
#pragma unroll
    for (int ni = 0; ni < FN; ++ni)
      bf[ni] = lds_read_frag(b_fr[kk] + ni * (16 * kRowBytes));
  };

  // Prologue: four slabs in flight, then the first fragments.  The wait is for
  // everything: loads and the previous tile's stores do not retire in one order.
  if (!preloaded) issue_prologue<BM, BN>(cx, a_base, b_base, b_last);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  // A slab pair is two K steps of 32.  Fragment double buffer: while the MFMAs
  // of one K step run, the fragments of the next are read.  The workgroup
  // barrier sits between the two K steps of a slab pair, right after its last
  // fragment reads: from there on both of its slots are free.
  bf16x8 af0[FM], bf0[FN], af1[FM], bf1[FN];
  read_frags(af0, bf0, 0);

  // The loads of a slab pair's 64 KiB are spread over its MFMAs: a burst would
  // fill the memory pipeline's queue, and a wave that cannot issue its load
  // cannot issue the MFMA behind it either.
  //   * the first K step of slab pair kt carries the loads of A slab kt+2, into
  //     the slot that B slab kt-1 left at the previous barrier (slot 4 at
  //     kt = 0): they have until the barrier of pair kt+1, more than a slab
  //     pair away;
  //   * the first half of the second K step, behind the barrier, carries the
  //     loads of B slab kt+2 into the slot A slab kt has just left: due at the
  //     next barrier, three quarters of a slab pair from now at the least.
  //     Only half of a slab pair's bytes are ever on that short deadline,
  //     which the 2.5 slab pairs of LDS buy.
  // Past the end of K the loads repeat the last slab (into a slot nobody reads
  // any more) rather than being branched around: one code path keeps the
  // accumulators in place across the whole loop body.  All loops below have
  // constant trip counts, so they unroll fully and every array index is a
  // compile-time constant; the instruction order is the program order.
  constexpr int kMfma = FM * FN, kReads = FM + FN;
  static_assert(kMfma % GA == 0 && (kMfma / 2) % GB == 0, "one load per MFMA at most");
  // the fragment reads of the next K step go under the first three quarters of the
  // MFMAs, so that the last of them has returned when that step starts
  constexpr int kReadSpan = kMfma * 3 / 4;
  auto first_step = [&](const uint8_t* ak, uint32_t la) {
#pragma unroll
    for (int ni = 0; ni < FN; ++ni) {
#pragma unroll
      for (int mi = 0; mi < FM; ++mi) {
        const int slot = ni * FM + mi;
        // (GA divides kMfma: at most one load per MFMA, group g at MFMA g * kMfma / GA)
        if (slot % (kMfma / GA) != 0) mfma_bf16(acc[ni][mi], bf0[ni], af0[mi]);
        else if (slot == 0) mfma_bf16_load<true>(acc[ni][mi], bf0[ni], af0[mi], ak, a_off[0], la);
        else mfma_bf16_load<false>(acc[ni][mi], bf0[ni], af0[mi], ak, a_off[slot / (kMfma / GA)], 0);
#pragma unroll
        for (int r = 0; r < FM; ++r)
          if (r * kReadSpan / kReads == slot)
            af1[r] = lds_read_frag(a_fr[1] + r * (16 * kRowBytes));
#pragma unroll
        for (int r = 0; r < FN; ++r)
          if ((FM + r) * kReadSpan / kReads == slot)
            bf1[r] = lds_read_frag(b_fr[1] + r * (16 * kRowBytes));
        __builtin_amdgcn_sched_barrier(0);     // keep this interleaving
      }
    }
  };
  auto second_step = [&](int kt) {
    const int kb = kt + 2 < nk ? kt + 2 : nk - 1;
    const uint8_t* bk = b_base + (int64_t)kb * kRowBytes;
    const uint32_t lb = lds0 + a_at + wave * (GB * 1024);
    // the next slab pair sits two slots further round the ring
    const uint32_t a_to = a_at + 2 * kSlot < kRingSlots * kSlot ? a_at + 2 * kSlot : a_at + 2 * kSlot - kRingSlots * kSlot;
    const uint32_t b_to = b_at + 2 * kSlot < kRingSlots * kSlot ? b_at + 2 * kSlot : b_at + 2 * kSlot - kRingSlots * kSlot;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      a_fr[kk] += a_to - a_at;
      b_fr[kk] += b_to - b_at;
    }
    a_at = a_to;
    b_at = b_to;
#pragma unroll
    for (int ni = 0; ni < FN; ++ni) {
#pragma unroll
      for (int mi = 0; mi < FM; ++mi) {
        const int slot = ni * FM + mi;
        // (group g at MFMA g * (kMfma / 2) / GB: the first half of the step)
        if (slot >= kMfma / 2 || slot % (kMfma / 2 / GB) != 0) mfma_bf16(acc[ni][mi], bf1[ni], af1[mi]);
        else if (slot == 0) mfma_bf16_load<true>(acc[ni][mi], bf1[ni], af1[mi], bk, b_off[0], lb);
        else mfma_bf16_load<false>(acc[ni][mi], bf1[ni], af1[mi], bk, b_off[slot / (kMfma / 2 / GB)], 0);
#pragma unroll
        for (int r = 0; r < FM; ++r)
          if (r * kReadSpan / kReads == slot)
            af0[r] = lds_read_frag(a_fr[0] + r * (16 * kRowBytes));
#pragma unroll
        for (int r = 0; r < FN; ++r)
          if ((FM + r) * kReadSpan / kReads == slot)
            bf0[r] = lds_read_frag(b_fr[0] + r * (16 * kRowBytes));
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  for (int kt = 0; kt < nk; ++kt) {
    const int ka = kt + 2 < nk ? kt + 2 : nk - 1;
    const uint8_t* ak = a_base + (int64_t)ka * kRowBytes;
    // four slots on from A slab kt = one slot back = where B slab kt-1 was
    const uint32_t a_dst = a_at >= kSlot ? a_at - kSlot : a_at + (kRingSlots - 1) * kSlot;
    first_step(ak, lds0 + a_dst + wave * (GA * 1024));
    // Wait for this wave's own loads of B slab kt+1 (and everything older) before
    // the barrier; the compiler does not count them (see load_group).  The GA
    // loads of A slab kt+2, issued last, may stay in flight: loads return in order.
    static_assert(GA == 8 || GA == 4, "explicit vmcnt below");
    if constexpr (GA == 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    __syncthreads();     // slab pair kt fully read by everyone; pair kt+1 has landed
    second_step(kt);
  }
  // The repeated loads of the last K steps must not land on top of the next
  // tile's first slabs.  (The MFMAs are assembly the compiler does not time: the explicit
  // idle slots cover the distance the last of them needs before its result may be read.)
  asm volatile("s_waitcnt vmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");
  __syncthreads();       // the next tile's prologue overwrites the ring
  if (tr != nullptr) tr[2] = wall_clock64();
  between();

  // Epilogue.  D[n][m]: a lane holds row m = lane & 15 of a 16x16 fragment and the 4
  // consecutive columns (lane >> 4)*4 .. +3.  Stored from there, a wave instruction
  // would touch 16 rows with 32 bytes each.  Instead each wave turns 32 rows of its
  // tile at a time through its own quarter of ring slot 4 (the only slot the next
  // tile's early loads leave alone) and stores whole rows: 16 bytes per lane, WN*2
  // contiguous bytes per row.  Chunk c of row r sits at position
  // c ^ (r mod chunks-per-row), which keeps both sides free of bank conflicts.
  // The region is private to the wave and a wave's LDS operations execute in
  // order, so no barrier is needed.
  constexpr int kChunks = WN / 8;                 // 16-byte chunks per wave-tile row
  constexpr int kRowsPerStore = 64 / kChunks;
  // (a row of 14 chunks - the 224-wide tile - is 224 bytes: consecutive rows start 32 bytes
  // apart in the 256-byte bank row by themselves, and no position swizzle is needed)
  constexpr bool kPow2 = (kChunks & (kChunks - 1)) == 0;
  static_assert(32 % kRowsPerStore == 0, "whole store instructions per band");
  const uint32_t turn = lds0 + (kRingSlots - 1) * kSlot + wave * (32 * WN * 2);
  const int rd_row = ln / kChunks, rd_chunk = ln % kChunks;
  const bool rd_lane = rd_row < kRowsPerStore;    // 64 lanes = 4 rows of 14 chunks and 8 lanes over
#pragma unroll
  for (int band = 0; band < FM / 2; ++band) {
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      const int wr_row = sub * 16 + (ln & 15);
#pragma unroll
      for (int ni = 0; ni < FN; ++ni) {
        const f32x4 d = acc[ni][band * 2 + sub];
        u32x2 v;
        v.x = pack_bf16x2(d[0], d[1]);
        v.y = pack_bf16x2(d[2], d[3]);
        const int chunk = ni * 2 + (ln >> 5);
        const int pos = kPow2 ? ((chunk ^ wr_row) & (kChunks - 1)) : chunk;
        lds_write_b64(turn + wr_row * (WN * 2) + (pos << 4) + ((ln >> 4) & 1) * 8, v);
      }
    }
#pragma unroll
    for (int i = 0; i < 32 / kRowsPerStore; ++i) {
      const int r = i * kRowsPerStore + (rd_lane ? rd_row : 0);
      const int pos = kPow2 ? ((rd_chunk ^ r) & (kChunks - 1)) : rd_chunk;
      const u32x4 v = lds_read_b128(turn + r * (WN * 2) + (pos << 4));
      const int m = tile.row0 + wm * WM + band * 32 + r;
      const int n = tile.col0 + wn * WN + rd_chunk * 8;
      if (rd_lane && n < s.N) *reinterpret_cast<u32x4*>(c + ((int64_t)m * s.N + n) * 2) = v;
    }
    // one 32-row band at a time: keeps the accumulator read-out from flooding
    // the vector registers
    __builtin_amdgcn_sched_barrier(0);
  }
}

// ---------------------------------------------------------------------------
// The same tile with e4m3fn operands and result (the reference's FP8_OUTPUT switch,
// triton_all_gather_matmul.py:115,123,188).  A row of a slab is still 128 bytes, now
// 128 K values; everything that moves bytes (the ring, the loads, the swizzle, the
// waits) is the bf16 tile's.  The MFMA is v_mfma_f32_16x16x128_f8f6f4 (without scales:
// both operands e4m3fn as they are): it computes what the 32x32x64 form computes in as
// many cycles and draws less power, as with bf16 - a loop of nothing but MFMAs on
// N(0, 0.5) operands runs 7 to 9 % faster with it, and this kernel's clock is
// power-limited too.  An operand fragment is 16 rows x 128 K, one whole slab row per
// fragment row: lane l holds row l & 15 and the 32 bytes number l >> 4 of the four
// (chunks 2 * (l >> 4) and the one after it).  Both operands use the same lane -> K
// mapping, which is all the sum over K needs.  The 8 lanes x 2 that an LDS read serves
// together are 8 consecutive rows at two chunks that differ by 4; row_swizzle separates
// those as well (four distinct values in bits 0,1 over the rows of one parity, bit 2
// left to the chunk).
//
// One K step is a whole slab pair, and a fragment is 8 registers, so the fragments cannot
// all be double-buffered: the A fragments are (two sets, taken in turn by trip parity),
// the B fragments are one set whose halves are refilled while the other half is in use.
// A trip's MFMAs go B row by B row; the workgroup barrier stands in the middle:
//   first half   MFMAs with B fragments 0 .. FN/2-1; B fragments FN/2 .. FN-1 of this
//                slab pair are read; loads of A slab kt+2 are issued
//   barrier      slab pair kt is read by everyone, pair kt+1 has landed
//   second half  MFMAs with B fragments FN/2 .. FN-1; the other set of A fragments and
//                B fragments 0 .. FN/2-1 are read from pair kt+1; loads of B slab kt+2
typedef int i32x8 __attribute__((ext_vector_type(8)));

// Four fp32 values to e4m3fn, round to nearest even, finite values beyond the range to the
// largest finite one (+-448), NaN kept: cvt.rn.satfinite.  The conversion instruction does all
// of that by itself while the wave's overflow mode bit is set (set_fp8_saturation, around a
// tile's epilogue); without the bit a finite value beyond 464 becomes NaN, and clamping by hand with NaN
// passed through was nine vector instructions per pair instead of one - 2 us of a tile's epilogue.
// (An infinite input would still give NaN; an fp32 sum of products of e4m3fn values cannot get
// there: 448 * 448 * K stays finite for any K an int can hold.)
__device__ __forceinline__ uint32_t pack_fp8x4(float a, float b, float c, float d) {
  int w = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
  w = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, w, true);
  return (uint32_t)w;
}
// MODE.FP16_OVFL (bit 23 of hardware register 1).  Only around the conversions: with the bit
// set the MFMAs read a NaN operand (0x7F, 0xFF) as a number, and a NaN in A or B would no longer
// reach the result.
__device__ __forceinline__ void set_fp8_saturation(bool on) {
  if (on) __builtin_amdgcn_s_setreg((0 << 11) | (23 << 6) | 1, 1);
  else __builtin_amdgcn_s_setreg((0 << 11) | (23 << 6) | 1, 0);
}

// D += A x B on a 16x16x128 e4m3fn fragment pair; the accumulator named as an accumulation
// register for the reason given at mfma_bf16.
__device__ __forceinline__ void mfma_fp8(f32x4& acc, const i32x8& first, const i32x8& second) {
  asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+a"(acc) : "v"(first), "v"(second));
}

template <int P>
struct Parity {
  static constexpr int value = P;
};

template <int BM, int BN, typename Between>
__device__ __forceinline__ void run_tile_fp8(const TileContext& cx, const TileRef& tile,
                                             const uint8_t* a_rows, const uint8_t* b_rows,
                                             bool preloaded, Between&& between) {
  using T = GemmTile<BM, BN>;
  const uint8_t* a_base = uniform_ptr(a_rows);
  const uint8_t* b_base = uniform_ptr(b_rows);
  constexpr int WM = T::WM, WN = T::WN, FM = T::FM, FN = T::FN, GA = T::GA, GB = T::GB;
  constexpr uint32_t kSlot = T::kSlotBytes;
  const int lane = cx.lane, wave = cx.wave;
  const int wm = wave >> 1, wn = wave & 1;
  const uint32_t row_stride = cx.row_stride;
  const int nk = cx.nk;
  const uint32_t lds0 = cx.lds0;
  uint64_t* tr = cx.tr;
  uint8_t* c = cx.c;
  struct { int N; } s = {cx.N};

  int ln = lane;
  asm volatile("" : "+v"(ln));
  // fragment read addresses: first and second chunk of the lane's 32 bytes
  uint32_t a_fr[2], b_fr[2];
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const int pos = (2 * (ln >> 4) + q) ^ row_swizzle(ln & 15);
    a_fr[q] = lds0 + (uint32_t)((wm * WM + (ln & 15)) * kRowBytes + (pos << 4));
    b_fr[q] = lds0 + kSlot + (uint32_t)((wn * WN + (ln & 15)) * kRowBytes + (pos << 4));
  }
  uint32_t a_at = 0, b_at = kSlot;

  const int u = (ln & 7) ^ row_swizzle(ln >> 3);
  uint32_t a_off[GA];
#pragma unroll
  for (int j = 0; j < GA; ++j) {
    const int q = wave * GA + j;
    a_off[j] = (uint32_t)(q * 8 + (ln >> 3)) * row_stride + (uint32_t)((u ^ ((q & 1) << 2)) << 4);
  }
  const int b_last = s.N - 1 - tile.col0;
  uint32_t b_off[GB];
#pragma unroll
  for (int j = 0; j < GB; ++j) {
    const int q = wave * GB + j;
    int r = q * 8 + (ln >> 3);
    r = r < b_last ? r : b_last;
    b_off[j] = (uint32_t)r * row_stride + (uint32_t)((u ^ ((q & 1) << 2)) << 4);
  }

  f32x4 acc[FN][FM];
#pragma unroll
  for (int ni = 0; ni < FN; ++ni)
#pragma unroll
    for (int mi = 0; mi < FM; ++mi)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[ni][mi][e] = 0.0f;

  // one 128-bit read = half a fragment (q = 0 or 1) of fragment row f
  auto read_half = [&](i32x8& dst, uint32_t (&fr)[2], int f, int q) __attribute__((always_inline)) {
    const u32x4 v = lds_read_b128(fr[q] + f * (16 * kRowBytes));
    dst[4 * q + 0] = (int)v.x;
    dst[4 * q + 1] = (int)v.y;
    dst[4 * q + 2] = (int)v.z;
    dst[4 * q + 3] = (int)v.w;
  };

  if (!preloaded) issue_prologue<BM, BN>(cx, a_base, b_base, b_last);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  constexpr int HN = FN / 2;                      // B fragments per half of a trip
  constexpr int kHalf = FM * HN;                  // MFMAs per half
  i32x8 af[2][FM], bf[FN];
#pragma unroll
  for (int f = 0; f < FM; ++f)
#pragma unroll
    for (int q = 0; q < 2; ++q) read_half(af[0][f], a_fr, f, q);
#pragma unroll
  for (int f = 0; f < HN; ++f)
#pragma unroll
    for (int q = 0; q < 2; ++q) read_half(bf[f], b_fr, f, q);

  // Reads under the MFMAs, in the order they are needed.  First half: the FN reads of B
  // fragments HN .. FN-1, under the first three quarters.  Second half: B fragment 0 and
  // the A fragments of the next trip's first row first, then the other B fragments; the
  // last read is issued an eighth of a half before its end.
  constexpr int kReads1 = 2 * HN, kSpan1 = kHalf * 3 / 4;
  constexpr int kReads2 = 2 * (FM + HN), kSpan2 = kHalf * 7 / 8;
  auto trip = [&](auto parity, int kt) __attribute__((always_inline)) {
    constexpr int P = decltype(parity)::value;
    const int ka = kt + 2 < nk ? kt + 2 : nk - 1;
    const uint8_t* ak = a_base + (int64_t)ka * kRowBytes;
    // four slots on from A slab kt = one slot back = where B slab kt-1 was
    const uint32_t a_dst = a_at >= kSlot ? a_at - kSlot : a_at + (kRingSlots - 1) * kSlot;
    const uint32_t la = lds0 + a_dst + wave * (GA * 1024);
#pragma unroll
    for (int ni = 0; ni < HN; ++ni) {
#pragma unroll
      for (int mi = 0; mi < FM; ++mi) {
        const int slot = ni * FM + mi;
        mfma_fp8(acc[ni][mi], bf[ni], af[P][mi]);
#pragma unroll
        for (int r = 0; r < kReads1; ++r)
          if (r * kSpan1 / kReads1 == slot) read_half(bf[HN + (r >> 1)], b_fr, HN + (r >> 1), r & 1);
        // (an MFMA of this kind takes twice as long as a bf16 one: issue slots are not short here, and
        // the loads fused into the MFMAs' assembly, as in the bf16 tile, measured 0.5 to 0.9 % slower)
#pragma unroll
        for (int g = 0; g < GA; ++g)
          if (g * kHalf / GA == slot) load_group(ak, a_off[g], la + g * 1024);
        __builtin_amdgcn_sched_barrier(0);     // keep this interleaving
      }
    }
    // Wait for this wave's own loads of B slab kt+1 (and everything older) before the
    // barrier; the GA loads of A slab kt+2, issued last, may stay in flight.
    static_assert(GA == 8 || GA == 4, "explicit vmcnt below");
    if constexpr (GA == 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
    __syncthreads();     // slab pair kt fully read by everyone; pair kt+1 has landed

    const int kb = kt + 2 < nk ? kt + 2 : nk - 1;
    const uint8_t* bk = b_base + (int64_t)kb * kRowBytes;
    const uint32_t lb = lds0 + a_at + wave * (GB * 1024);
    // the next slab pair sits two slots further round the ring
    const uint32_t a_to = a_at + 2 * kSlot < kRingSlots * kSlot ? a_at + 2 * kSlot : a_at + 2 * kSlot - kRingSlots * kSlot;
    const uint32_t b_to = b_at + 2 * kSlot < kRingSlots * kSlot ? b_at + 2 * kSlot : b_at + 2 * kSlot - kRingSlots * kSlot;
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      a_fr[q] += a_to - a_at;
      b_fr[q] += b_to - b_at;
    }
    a_at = a_to;
    b_at = b_to;
#pragma unroll
    for (int ni = 0; ni < HN; ++ni) {
#pragma unroll
      for (int mi = 0; mi < FM; ++mi) {
        const int slot = ni * FM + mi;
        mfma_fp8(acc[HN + ni][mi], bf[HN + ni], af[P][mi]);
#pragma unroll
        for (int g = 0; g < GB; ++g)
          if (g * (kHalf / 2) / GB == slot) load_group(bk, b_off[g], lb + g * 1024);
#pragma unroll
        for (int r = 0; r < kReads2; ++r)
          if (r * kSpan2 / kReads2 == slot) {
            // order: B fragment 0, all A fragments, B fragments 1 .. HN-1
            if (r < 2) read_half(bf[0], b_fr, 0, r & 1);
            else if (r < 2 + 2 * FM) read_half(af[1 - P][(r - 2) >> 1], a_fr, (r - 2) >> 1, r & 1);
            else read_half(bf[(r - 2 * FM) >> 1], b_fr, (r - 2 * FM) >> 1, r & 1);
          }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  // Two trips per turn of the loop, one for each set of A fragments; an odd last trip
  // stands behind the loop (an exit in the middle of the loop would leave the compiler with
  // two places the accumulators can come from, and it then keeps two copies of them).
  int kt = 0;
  for (; kt + 1 < nk; kt += 2) {
    trip(Parity<0>{}, kt);
    trip(Parity<1>{}, kt + 1);
  }
  if (kt < nk) trip(Parity<0>{}, kt);
  // The repeated loads of the last K steps must not land on top of the next tile's first
  // slabs, and the last MFMAs (assembly the compiler does not time) must be through before
  // their results are read.
  asm volatile("s_waitcnt vmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");
  __syncthreads();
  if (tr != nullptr) tr[2] = wall_clock64();
  between();

  // Epilogue.  D[n][m]: a lane holds row m = lane & 15 of a 16x16 fragment and the 4
  // consecutive columns (lane >> 4)*4 .. +3: one 32-bit word of e4m3fn.  32 rows at a
  // time go through the wave's quarter of ring slot 4 (WN bytes per row, chunk c of row
  // r at position c ^ (r >> 1), modulo the chunks of a row) and leave as whole rows, 16
  // bytes per lane.
  constexpr int kChunks = WN / 16;                // 16-byte chunks per wave-tile row
  constexpr int kRowsPerStore = 64 / kChunks;
  const uint32_t turn = lds0 + (kRingSlots - 1) * kSlot + wave * (32 * WN);
  const int rd_row = ln / kChunks, rd_chunk = ln % kChunks;
  set_fp8_saturation(true);
#pragma unroll
  for (int band = 0; band < FM / 2; ++band) {
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      const int wr_row = sub * 16 + (ln & 15);
#pragma unroll
      for (int ni = 0; ni < FN; ++ni) {
        const f32x4 d = acc[ni][band * 2 + sub];
        const uint32_t w = pack_fp8x4(d[0], d[1], d[2], d[3]);
        const uint32_t addr = turn + wr_row * WN + (((ni ^ (wr_row >> 1)) & (kChunks - 1)) << 4) + (ln >> 4) * 4;
        *reinterpret_cast<__attribute__((address_space(3))) uint32_t*>((uintptr_t)addr) = w;
      }
    }
#pragma unroll
    for (int i = 0; i < 32 / kRowsPerStore; ++i) {
      const int r = i * kRowsPerStore + rd_row;
      const u32x4 v = lds_read_b128(turn + r * WN + (((rd_chunk ^ (r >> 1)) & (kChunks - 1)) << 4));
      const int m = tile.row0 + wm * WM + band * 32 + r;
      const int n = tile.col0 + wn * WN + rd_chunk * 16;
      if (n < s.N) *reinterpret_cast<u32x4*>(c + (int64_t)m * s.N + n) = v;
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  set_fp8_saturation(false);
}

// The gather done by the launch itself.  The reference's copy engines deliver every chunk and
// cost no SMs (triton_all_gather_matmul.py:41-55); on one GPU the copy runs on compute units,
// and here it runs inside the GEMM's own launch: workgroups [gemm_grid, gridDim.x) do nothing
// but copy, in the reference's chunk order, and a GEMM workgroup whose next tile's chunk is
// not there yet copies along instead of spinning.  One launch, one stream, no flag fill.
//
// Every chunk is cut into 64 KiB pieces that are taken by ticket until none is left, so
// nothing depends on which workgroups are running: a copy-only workgroup that is dispatched
// late (another kernel holds its compute unit) finds the pieces gone, and if none of them
// ever runs the GEMM's workgroups copy everything themselves, only later.  Pieces are written
// through to memory; whoever completes a chunk's count raises its flag.
//
// State (uint32 words, zero before the first launch): flags[chunks], tickets[chunks],
// finished[chunks], exits[1].  The last workgroup to leave zeroes all of it, so the next
// launch - or the next replay of a captured graph - starts from zero again with no fill.
struct CopyJob {
  const uint64_t* buffer_ptrs;   // the ranks' shard addresses (device array); nullptr = this launch copies nothing
  uint8_t* a_out;                // the gathered operand
  uint32_t* flags;               // progress flags, one per chunk
  uint32_t* tickets;             // next piece of a chunk
  uint32_t* finished;            // pieces of a chunk that are in place
  uint32_t* exits;               // workgroups that are through
  int64_t chunk_vecs;            // 16-byte vectors per chunk
  int pieces;                    // per chunk
  int chunks, splits, rank, world_size;
  int gemm_grid;                 // workgroups from here on only copy
};

typedef __attribute__((address_space(1))) u32x4 GlobalVec;
typedef __attribute__((address_space(3))) uint32_t LdsWord;
constexpr int kPullInFlight = 16;                               // 128-bit loads per thread and piece
constexpr int kPullPieceVecs = kGemmThreads * kPullInFlight;    // 64 KiB

// One value from thread 0 to the whole workgroup through the first word of the tile ring
// (not in use where this is called: before a tile's first loads).
template <typename F>
__device__ __forceinline__ uint32_t from_thread0(uint32_t lds0, F&& f) {
  LdsWord* slot = reinterpret_cast<LdsWord*>((uintptr_t)lds0);
  if (threadIdx.x == 0) *slot = f();
  __syncthreads();
  const uint32_t v = *slot;
  __syncthreads();
  return v;
}

// Takes pieces of chunk `c` by ticket and copies them until none is left.  SETS = 2 keeps two
// pieces in flight (a copy-only workgroup has the registers; 128 KiB per compute unit is what
// a streaming copy needs), SETS = 1 one (a GEMM workgroup between two tiles).
template <int SETS>
__device__ __forceinline__ void copy_pieces(const CopyJob& job, int c, uint32_t lds0, uint64_t* trace) {
  const GlobalVec* src = (const GlobalVec*)(uintptr_t)job.buffer_ptrs[c / job.splits] +
                         (int64_t)(c % job.splits) * job.chunk_vecs;
  GlobalVec* dst = (GlobalVec*)(uintptr_t)job.a_out + (int64_t)c * job.chunk_vecs;
  const uint32_t pieces = (uint32_t)job.pieces;
  auto draw = [&]() -> uint32_t {
    return from_thread0(lds0, [&]() { return __hip_atomic_fetch_add(&job.tickets[c], 1u, __ATOMIC_RELAXED, kScope); });
  };
  auto load = [&](u32x4 (&v)[kPullInFlight], uint32_t t) {
    const int64_t i0 = (int64_t)t * kPullPieceVecs + threadIdx.x;
#pragma unroll
    for (int u = 0; u < kPullInFlight; ++u) {
      const int64_t i = i0 + u * kGemmThreads;
      v[u] = __builtin_nontemporal_load(src + (i < job.chunk_vecs ? i : job.chunk_vecs - 1));
    }
  };
  auto store = [&](const u32x4 (&v)[kPullInFlight], uint32_t t) {
    const int64_t i0 = (int64_t)t * kPullPieceVecs + threadIdx.x;
#pragma unroll
    for (int u = 0; u < kPullInFlight; ++u) {
      const int64_t i = i0 + u * kGemmThreads;
      // (the idle slots: the hardware reads a 128-bit store's data for two cycles after issue, a
      // vector instruction that writes one of these registers right behind the store changes what
      // is stored, and the compiler, which spaces its own stores, does not look into assembly)
      if (i < job.chunk_vecs)
        asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" : : "v"(dst + i), "v"(v[u]) : "memory");
    }
  };
  uint32_t mine = 0;
  u32x4 v0[kPullInFlight];
  uint32_t t0 = draw();
  if (t0 < pieces) load(v0, t0);
  if constexpr (SETS == 2) {
    u32x4 v1[kPullInFlight];
    while (t0 < pieces) {
      // the next ticket is drawn, and its piece's loads issued, while this piece's are in flight
      const uint32_t t1 = draw();
      if (t1 < pieces) load(v1, t1);
      store(v0, t0);
      ++mine;
      if (t1 >= pieces) break;
      t0 = draw();
      if (t0 < pieces) load(v0, t0);
      store(v1, t1);
      ++mine;
    }
  } else {
    while (t0 < pieces) {
      const uint32_t t1 = draw();
      store(v0, t0);
      ++mine;
      t0 = t1;
      if (t0 < pieces) load(v0, t0);
    }
  }
  // A wait the compiler can see (the builtin, not assembly text): its own count of loads in
  // flight is per register and joins all paths, so behind the loop above it takes the piece
  // registers for possibly still being loaded - and would put its wait for them where they are
  // next written, which is in the middle of a K loop (every direct-to-LDS load drained once per
  // trip: the 256x128 and 128x128 kernels ran 30 % slower that way).
  __builtin_amdgcn_s_waitcnt(0x0F70);      // vmcnt(0), the other counters left alone
  if (mine == 0) return;
  // written through: once acknowledged the pieces are where every XCD reads them
  wait_stores_acknowledged();
  __syncthreads();
  if (threadIdx.x == 0) {
    const uint32_t prev = __hip_atomic_fetch_add(&job.finished[c], mine, __ATOMIC_RELAXED, kScope);
    if (prev + mine == pieces) {
      __hip_atomic_store(&job.flags[c], 1u, __ATOMIC_RELAXED, kScope);
      if (trace != nullptr && c < kTraceProducerWords - 1) trace[c] = wall_clock64();
    }
  }
}

// A workgroup is through: the last one puts the launch's state back to zero.
__device__ __forceinline__ void leave(const CopyJob& job) {
  if (threadIdx.x != 0) return;
  // this thread's own last flag store has landed before the workgroup counts as gone: the
  // zeroing below must not be overtaken by it
  wait_stores_acknowledged();
  const uint32_t prev = __hip_atomic_fetch_add(job.exits, 1u, __ATOMIC_RELAXED, kScope);
  if (prev + 1u != gridDim.x) return;
  // every other workgroup's last access to these words lies before its count above
  for (int c = 0; c < job.chunks; ++c) {
    __hip_atomic_store(&job.flags[c], 0u, __ATOMIC_RELAXED, kScope);
    __hip_atomic_store(&job.tickets[c], 0u, __ATOMIC_RELAXED, kScope);
    __hip_atomic_store(&job.finished[c], 0u, __ATOMIC_RELAXED, kScope);
  }
  __hip_atomic_store(job.exits, 0u, __ATOMIC_RELAXED, kScope);
}

template <int BM, int BN, bool FP8 = false>
__global__ __launch_bounds__(kGemmThreads, 1) void ag_matmul_kernel(
    const uint8_t* __restrict__ a_shard, const uint8_t* __restrict__ a_out,
    const uint8_t* __restrict__ b_nk, uint8_t* __restrict__ c, const uint32_t* progress,
    GemmSchedule s, uint64_t limit_ticks, uint32_t* status, uint64_t* trace, CopyJob job) {
  __shared__ __attribute__((aligned(1024))) uint8_t lds[GemmTile<BM, BN>::kLdsBytes];
  const uint32_t lds0 = lds_offset_of(lds);

  // Copy-only workgroups of a fused launch: the chunks in the reference's order (sources
  // rank+1, ..., rank+ws-1, rank: triton_all_gather_matmul.py:43-44), then out.
  if (job.buffer_ptrs != nullptr && (int)blockIdx.x >= job.gemm_grid) {
    if (trace != nullptr && (int)blockIdx.x == job.gemm_grid && threadIdx.x == 0)
      trace[kTraceProducerWords - 1] = wall_clock64();
    for (int step = 0; step < job.world_size; ++step) {
      const int src_rank = (job.rank + step + 1) % job.world_size;
      for (int split = 0; split < job.splits; ++split)
        copy_pieces<2>(job, src_rank * job.splits + split, lds0, trace);
    }
    leave(job);
    return;
  }

  TileContext cx;
  cx.lane = threadIdx.x & 63;
  cx.wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  cx.row_stride = (uint32_t)s.K * (FP8 ? 1u : 2u);        // K values per row, 1 or 2 bytes each
  cx.nk = (int)(cx.row_stride / kRowBytes);
  cx.lds0 = lds0;
  cx.N = s.N;
  cx.c = c;

  // Source rows of a tile: the local shard, or the gathered buffer once the comm
  // block's flag is up.
  auto a_rows_of = [&](const TileRef& t) -> const uint8_t* {
    if (t.local) return a_shard + (int64_t)t.a_row * cx.row_stride;
    if (progress != nullptr) {
      const uint32_t* flag = progress + t.comm_block;
      // A launch that gathers for itself: if the chunk is not there, take part in copying it.
      bool up = false;
      if (job.buffer_ptrs != nullptr) {
        up = from_thread0(lds0, [&]() { return __hip_atomic_load(flag, __ATOMIC_RELAXED, kScope) == 1u ? 1u : 0u; }) != 0u;
        if (!up) copy_pieces<1>(job, t.comm_block, lds0, trace);
      }
      // Thread 0 polls the flag past the caches, the workgroup meets, and only then are the
      // rows' loads issued.  No cache is invalidated here: a line of this comm block can sit
      // in this compute unit's L1 or this XCD's L2 only if somebody read or wrote it since
      // the kernel began (the dispatch itself starts from invalidated caches), nobody reads
      // a comm block's rows before its flag, and whoever wrote them (a producer, or this
      // launch's own copying) wrote whole lines through to memory and saw them
      // acknowledged before the flag went up.  The invalidate an acquire fence stands for
      // would throw out the XCD's shared A and B lines at every tile instead: 2 % of the
      // fused launch.  smr_set_ag_matmul_acquire(1) puts the fence back.
      if (s.acquire) {
        wait_signal(flag, limit_ticks, status, t.comm_block);
      } else if (!up) {
        if (threadIdx.x == 0 && !wait_flag_set(flag, limit_ticks))
          report(status, SMR_ST_WAIT_TIMEOUT, t.comm_block, blockIdx.x, 0u);
        __syncthreads();
      }
    }
    return a_out + (int64_t)t.a_row * cx.row_stride;
  };

  const uint64_t t_entry = trace != nullptr ? wall_clock64() : 0;
  TileRef tile;
  int step = 0;
  bool have = next_tile(s, blockIdx.x, step, tile);
  const uint8_t* a_base = nullptr;
  const uint8_t* b_base = nullptr;
  if (have) {
    a_base = a_rows_of(tile);
    b_base = b_nk + (int64_t)tile.col0 * cx.row_stride;
  }
  bool preloaded = false;
  for (int trip = 0; have; ++trip) {
    cx.tr = nullptr;
    if (trace != nullptr && trip < kTraceSteps && blockIdx.x < 256 && threadIdx.x == 0) {
      cx.tr = trace + kTraceProducerWords + ((size_t)blockIdx.x * kTraceSteps + trip) * 4;
      cx.tr[0] = cx.tr[1] = wall_clock64();
      if (trip == 0) cx.tr[0] = t_entry;
    }
    TileRef next;
    bool have_next = false;
    const uint8_t* a_next = nullptr;
    const uint8_t* b_next = nullptr;
    // Between this tile's K loop and its stores: pick the next tile, wait for its
    // flag if it has one, and start its first loads.
    auto between = [&]() {
      ++step;
      have_next = next_tile(s, blockIdx.x, step, next);
      if (!have_next) return;
      a_next = a_rows_of(next);
      b_next = b_nk + (int64_t)next.col0 * cx.row_stride;
      issue_prologue<BM, BN>(cx, a_next, b_next, s.N - 1 - next.col0);
    };
    if constexpr (FP8) run_tile_fp8<BM, BN>(cx, tile, a_base, b_base, preloaded, between);
    else run_tile<BM, BN>(cx, tile, a_base, b_base, preloaded, between);
    if (cx.tr != nullptr) cx.tr[3] = wall_clock64();
    have = have_next;
    tile = next;
    a_base = a_next;
    b_base = b_next;
    preloaded = true;
  }
  if (job.buffer_ptrs != nullptr) leave(job);
}

// Tile shape: the largest the flags' granularity allows, stepped down while the
// problem has too few tiles to occupy more than half of the compute units.
static int pick_tile(int M, int N, int comm_block_m, int& BM, int& BN, int cus = 256, bool wide_ok = false) {
  if (comm_block_m % 256 == 0) {
    BM = 256;
    BN = N >= 256 ? 256 : 128;
    // 256x224 tiles when they fill every compute unit in whole passes and 256x256 tiles do not
    // (M=16384 N=3584: 1024 tiles = 4 passes of 256 against 896 tiles = 4 passes of 224):
    // the same number of passes, each an eighth shorter.  Only for a launch that has the
    // whole GPU (bf16, no copy beside it).
    if (wide_ok && N % 224 == 0 && cus % 8 == 0) {
      const int t224 = (M / 256) * (N / 224), t256 = (M / 256) * ceil_div(N, 256);
      if (t224 % cus == 0 && (int64_t)ceil_div(t224, cus) * 224 < (int64_t)ceil_div(t256, cus) * 256) {
        BN = 224;
        return 0;
      }
    }
    if (BN == 256 && (M / 256) * ceil_div(N, 256) * 2 <= cus) BN = 128;
    if (BN == 128 && (M / 256) * ceil_div(N, 128) * 2 <= cus) BM = 128;
  } else if (comm_block_m % 128 == 0) {
    BM = 128;
    BN = 128;
  } else {
    return -1;
  }
  return 0;
}

static int validate(int M, int N, int K, int rank, int world_size, int comm_block_m, const char** why) {
  *why = nullptr;
  if (world_size < 1 || world_size > SMR_MAX_WORLD_SIZE || rank < 0 || rank >= world_size)
    *why = "smr_ag_matmul: rank/world_size";
  else if (M <= 0 || N <= 0 || K <= 0)
    *why = "smr_ag_matmul: empty shape";
  else if (comm_block_m <= 0 || M % comm_block_m != 0 || (M / comm_block_m) % world_size != 0)
    *why = "smr_ag_matmul: M must be world_size * splits * comm_block_m";
  if (*why) return SMR_E_INVALID;
  if (K % kBK != 0)
    *why = "smr_ag_matmul: K must be a multiple of 64";
  else if (N % 8 != 0)
    *why = "smr_ag_matmul: N must be a multiple of 8";
  else if (comm_block_m % 128 != 0)
    *why = "smr_ag_matmul: rows per progress flag must be a multiple of 128";
  if (*why) return SMR_E_UNSUPPORTED;
  return 0;
}

// Compute units of the current device (cached per device: a process may drive several parts).
static int cu_count() {
  constexpr int kMaxDevices = 64;
  static std::atomic<int> cached[kMaxDevices];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return 256;
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 256;
    cached[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

// Persistent grid: the fewest workgroups (a multiple of 8, one per XCD slot) that
// still finish in the minimum number of passes.  A gated launch leaves at least
// kReservedCus compute units to the producer: a workgroup of this kernel fills a
// compute unit's register file, so a producer that arrives late would otherwise
// find no room while the consumers spin on its flags.
constexpr int kReservedCus = 8;

static int total_steps(const GemmSchedule& s) {
  return ceil_div((s.M / s.BM) * ceil_div(s.N, s.BN), s.grid);
}

// Coarse model of a fused launch, for splitting the compute units between the GEMM and the
// copy and for choosing between the fused launch and copy-then-multiply.  Its constants are
// fitted to launches timed on MI355X (24 problems from M=1024 to M=32768, bf16 and e4m3fn, both
// forms of each): a GEMM workgroup sustains 6.5 TFLOP/s on 256x256 tiles next to the copy (6.6
// without it, 4.6 on narrower tiles, twice that in e4m3fn) plus 6 us per tile; a copy-only
// workgroup moves 25 GB/s (bytes read plus bytes written) while the GEMM runs; while workgroups
// wait for a chunk everybody copies at 12 GB/s apiece, and three fifths of such a wait show in
// the launch's duration; a fused launch costs 18 us on top (the first pieces' way through
// tickets, loads, write-through stores and flags), copy-then-multiply 10 us for its two launches.
struct FusedEstimate {
  double gemm_us, copy_us, total_us;
  int producer_wgs;
};
constexpr int kMaxProducerWgs = 128;
constexpr double kCopyOnlyBytesPerUs = 25.0e3, kWaiterBytesPerUs = 12.0e3, kWaitShows = 0.6, kFusedFixedUs = 18.0;
static double model_tile_us(int BM, int BN, int K, int elem_bytes, bool beside_copy) {
  double rate = BM == 256 && BN >= 224 ? (beside_copy ? 6.5e6 : 6.6e6) : 4.6e6;      // FLOP per us
  if (elem_bytes == 1) rate = BM == 256 && BN == 256 ? (beside_copy ? 14.2e6 : 14.0e6) : 9.2e6;
  return 2.0 * BM * BN * K / rate + 6.0;
}
static FusedEstimate estimate_fused(const GemmSchedule& s, int cus, int grid, int elem_bytes = 2) {
  const double tile_us = model_tile_us(s.BM, s.BN, s.K, elem_bytes, true);
  const int tiles = (s.M / s.BM) * ceil_div(s.N, s.BN);
  const int tiles_per_cb = (s.comm_block_m / s.BM) * ceil_div(s.N, s.BN);
  const int n_comm = s.M / s.comm_block_m, per_rank = n_comm / s.world_size;
  FusedEstimate e;
  e.producer_wgs = cus - grid < kMaxProducerWgs ? cus - grid : kMaxProducerWgs;
  if (e.producer_wgs < 1) e.producer_wgs = 1;
  const double chunk_bytes = 2.0 * elem_bytes * s.comm_block_m * s.K;         // read and written
  const double remote_bytes = chunk_bytes * (n_comm - per_rank);
  const int passes = ceil_div(tiles, grid);
  // Pass by pass, tiles in ring order: a pass starts when the chunks it touches are in place;
  // what is missing then is copied by the copy-only workgroups and the workgroups that wait.
  double now = kFusedFixedUs, copied = 0.0;
  for (int pass = 0; pass < passes; ++pass) {
    const int first = pass * grid;
    const int last = (tiles < first + grid ? tiles : first + grid) - 1;
    double need = (last / tiles_per_cb + 1 - per_rank) * chunk_bytes;
    if (need > remote_bytes) need = remote_bytes;
    if (copied < need) {
      const int first_missing = (per_rank + (int)(copied / chunk_bytes)) * tiles_per_cb;
      const int waiting = last + 1 - (first > first_missing ? first : first_missing);
      // (with that many at it at once the copy-only workgroups move no more than the others)
      now += kWaitShows * (need - copied) / ((e.producer_wgs + (waiting > 0 ? waiting : 0)) * kWaiterBytesPerUs);
      copied = need;
    }
    now += tile_us;
    copied += e.producer_wgs * kCopyOnlyBytesPerUs * tile_us;
    if (copied > remote_bytes) copied = remote_bytes;
  }
  e.gemm_us = passes * tile_us;
  e.copy_us = remote_bytes / (e.producer_wgs * kCopyOnlyBytesPerUs);
  e.total_us = now;
  return e;
}

// Process-wide tuning knobs.  Each is one atomic word, read once per call by make_schedule,
// so a setter on another thread changes a whole launch or none of it.
static std::atomic<int> g_acquire_after_flag{0};
static std::atomic<int> g_grid_limit{0};                     // smr_set_ag_matmul_grid_limit: 0 = none

// How a launch shares the GPU: not gated at all; gated with compute units left free for a
// producer kernel; gated by somebody who needs no compute units of his own (copy engines, or
// the producer whose workgroups fit beside this kernel's: smr_all_gather_beside).
enum GateKind : int { kUngated = 0, kGatedShare = 1, kGatedWhole = 2 };

static GemmSchedule make_schedule(int M, int N, int K, int rank, int world_size, int comm_block_m,
                                  int cus, int gated, int elem_bytes = 2) {
  GemmSchedule s;
  s.M = M; s.N = N; s.K = K;
  s.rank = rank; s.world_size = world_size; s.comm_block_m = comm_block_m;
  s.acquire = g_acquire_after_flag.load(std::memory_order_relaxed);
  const int grid_limit = g_grid_limit.load(std::memory_order_relaxed);
  int max_grid = ((gated == kGatedShare ? cus - kReservedCus : cus) / 8) * 8;
  if (grid_limit > 0 && grid_limit < max_grid) max_grid = grid_limit / 8 * 8;
  if (max_grid < 8) max_grid = 8;
  pick_tile(M, N, comm_block_m, s.BM, s.BN, max_grid, gated != kGatedShare && elem_bytes == 2);
  const int tn = (N + s.BN - 1) / s.BN;
  const int total = (M / s.BM) * tn;
  const int passes = (total + max_grid - 1) / max_grid;
  const int need = ((total + passes - 1) / passes + 7) / 8 * 8;
  s.grid = need < max_grid ? need : max_grid;
  if (gated == kGatedShare) {
    // The producer runs on the compute units this grid leaves free, and a small or
    // skinny problem is over before a narrow producer has copied the shards.  Take
    // the grid (a multiple of 8) for which the later of the two - the GEMM's passes,
    // or the last chunk's arrival plus the tiles that wait for it - comes earliest;
    // among equals the smallest grid.
    const FusedEstimate base = estimate_fused(s, cus, s.grid, elem_bytes);
    double best = base.total_us;
    for (int g = 8; g <= max_grid; g += 8) {
      const double t = estimate_fused(s, cus, g, elem_bytes).total_us;
      if (t < best * 0.97) {             // only for a clear gain: the model is coarse
        best = t;
        s.grid = g;
      }
    }
  }
  // Rows per group: the divisor of the comm block's row tiles for which an XCD's run of
  // a full pass touches the fewest slabs (rows of the patch + columns of the patch).
  {
    const int cb_tiles_m = comm_block_m / s.BM;
    const int per_xcd = ceil_div(total < s.grid ? total : s.grid, 8);
    int best_cost = 1 << 30;
    s.group_m = cb_tiles_m;
    for (int g = 1; g <= cb_tiles_m; ++g) {
      if (cb_tiles_m % g != 0) continue;
      const int rows = g < per_xcd ? g : per_xcd;
      const int cost = rows + ceil_div(per_xcd, g);
      if (cost < best_cost || (cost == best_cost && g > s.group_m)) {
        best_cost = cost;
        s.group_m = g;
      }
    }
  }
  s.steps = total_steps(s);
  return s;
}

}  // namespace smr

extern "C" {

// What a fused launch adds to the GEMM's: who copies (see CopyJob).
struct FusedArgs {
  const uint64_t* buffer_ptrs_dev;
  uint32_t* state_dev;           // flags, tickets, finished, exits
  int producer_wgs;              // copy-only workgroups; 0 = the plan's
};

static int launch_gemm(int elem_bytes, const void* a_shard_dev, const void* a_out_dev, const void* b_nk_dev,
                       void* c_dev, const uint32_t* progress_dev, int M, int N, int K, int rank,
                       int world_size, int comm_block_m, int whole_gpu, uint32_t* status, void* stream,
                       const FusedArgs* fused) {
  using namespace smr;
  if (a_shard_dev == nullptr || a_out_dev == nullptr || b_nk_dev == nullptr || c_dev == nullptr)
    return fail(SMR_E_INVALID, elem_bytes == 1 ? "smr_ag_matmul_fp8: null pointer" : "smr_ag_matmul: null pointer");
  if ((reinterpret_cast<uintptr_t>(a_shard_dev) | reinterpret_cast<uintptr_t>(a_out_dev) |
       reinterpret_cast<uintptr_t>(b_nk_dev) | reinterpret_cast<uintptr_t>(c_dev)) & 15u)
    return fail(SMR_E_INVALID, elem_bytes == 1 ? "smr_ag_matmul_fp8: operands must be 16-byte aligned"
                                               : "smr_ag_matmul: operands must be 16-byte aligned");
  const int cus = cu_count();
  const int gate = fused != nullptr ? kGatedShare : (progress_dev == nullptr ? kUngated : (whole_gpu ? kGatedWhole : kGatedShare));
  const GemmSchedule s = make_schedule(M, N, K, rank, world_size, comm_block_m, cus, gate, elem_bytes);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const uint8_t* a0 = reinterpret_cast<const uint8_t*>(a_shard_dev);
  const uint8_t* a1 = reinterpret_cast<const uint8_t*>(a_out_dev);
  const uint8_t* b = reinterpret_cast<const uint8_t*>(b_nk_dev);
  uint8_t* c = reinterpret_cast<uint8_t*>(c_dev);
  const uint64_t lim = spin_limit_ticks();
  uint64_t* tb = trace_buffer(kTraceProducerWords + kTraceGemmWords);
  CopyJob job = {};
  unsigned grid = (unsigned)s.grid;
  if (fused != nullptr) {
    const int splits = (M / world_size) / comm_block_m;
    const int chunks = world_size * splits;
    const int64_t chunk_bytes = (int64_t)comm_block_m * K * elem_bytes;
    job.buffer_ptrs = fused->buffer_ptrs_dev;
    job.a_out = const_cast<uint8_t*>(a1);
    job.flags = fused->state_dev;
    job.tickets = fused->state_dev + chunks;
    job.finished = fused->state_dev + 2 * chunks;
    job.exits = fused->state_dev + 3 * chunks;
    job.chunk_vecs = chunk_bytes / 16;
    job.pieces = (int)((job.chunk_vecs + kPullPieceVecs - 1) / kPullPieceVecs);
    job.chunks = chunks;
    job.splits = splits;
    job.rank = rank;
    job.world_size = world_size;
    job.gemm_grid = s.grid;
    int producers = fused->producer_wgs > 0 ? fused->producer_wgs
                                            : estimate_fused(s, cus, s.grid, elem_bytes).producer_wgs;
    // a workgroup of this kernel fills a compute unit: more of them than there are compute
    // units would only queue up behind the GEMM's
    if (producers > cus - s.grid) producers = cus - s.grid;
    // Never none: the GEMM's workgroups copy only the chunks their own tiles wait for and read
    // the local rows from the shard itself, so the local shard reaches a_out through a
    // copy-only workgroup.  Pieces are taken by ticket, so one that is dispatched late (a part
    // with fewer compute units than the grid) still finds whatever is left.
    if (producers < 1) producers = 1;
    grid += (unsigned)producers;
    progress_dev = job.flags;
  }
  if (elem_bytes == 1 && s.BM == 256 && s.BN == 256)
    hipLaunchKernelGGL((ag_matmul_kernel<256, 256, true>), dim3(grid), dim3(kGemmThreads), 0, st, a0, a1, b,
                       c, progress_dev, s, lim, status, tb, job);
  else if (elem_bytes == 1 && s.BM == 256)
    hipLaunchKernelGGL((ag_matmul_kernel<256, 128, true>), dim3(grid), dim3(kGemmThreads), 0, st, a0, a1, b,
                       c, progress_dev, s, lim, status, tb, job);
  else if (elem_bytes == 1)
    hipLaunchKernelGGL((ag_matmul_kernel<128, 128, true>), dim3(grid), dim3(kGemmThreads), 0, st, a0, a1, b,
                       c, progress_dev, s, lim, status, tb, job);
  else if (s.BM == 256 && s.BN == 256)
    hipLaunchKernelGGL((ag_matmul_kernel<256, 256>), dim3(grid), dim3(kGemmThreads), 0, st, a0, a1, b,
                       c, progress_dev, s, lim, status, tb, job);
  else if (s.BM == 256 && s.BN == 224)
    hipLaunchKernelGGL((ag_matmul_kernel<256, 224>), dim3(grid), dim3(kGemmThreads), 0, st, a0, a1, b,
                       c, progress_dev, s, lim, status, tb, job);
  else if (s.BM == 256)
    hipLaunchKernelGGL((ag_matmul_kernel<256, 128>), dim3(grid), dim3(kGemmThreads), 0, st, a0, a1, b,
                       c, progress_dev, s, lim, status, tb, job);
  else
    hipLaunchKernelGGL((ag_matmul_kernel<128, 128>), dim3(grid), dim3(kGemmThreads), 0, st, a0, a1, b,
                       c, progress_dev, s, lim, status, tb, job);
  return check_hip(hipGetLastError(), "smr_ag_matmul launch");
}

static int validate_fp8(int M, int N, int K, int rank, int world_size, int comm_block_m, const char** why);

int smr_ag_matmul(const void* a_shard_dev, const void* a_out_dev, const void* b_nk_dev, void* c_dev,
                  const uint32_t* progress_dev, int M, int N, int K, int rank, int world_size,
                  int comm_block_m, int whole_gpu, uint32_t* status, void* stream) {
  using namespace smr;
  const char* why;
  if (int rc = validate(M, N, K, rank, world_size, comm_block_m, &why)) return fail(rc, why);
  return launch_gemm(2, a_shard_dev, a_out_dev, b_nk_dev, c_dev, progress_dev, M, N, K, rank, world_size,
                     comm_block_m, whole_gpu, status, stream, nullptr);
}

int smr_ag_matmul_fused_state_words(int world_size, int splits_per_rank) {
  if (world_size < 1 || world_size > SMR_MAX_WORLD_SIZE || splits_per_rank < 1) return 0;
  return 3 * world_size * splits_per_rank + 1;
}

int smr_ag_matmul_fused(const void* a_shard_dev, void* a_out_dev, const void* b_nk_dev, void* c_dev,
                        uint32_t* state_dev, const uint64_t* buffer_ptrs_dev, int elem_bytes, int M, int N,
                        int K, int rank, int world_size, int comm_block_m, int producer_workgroups,
                        uint32_t* status, void* stream) {
  using namespace smr;
  const char* why;
  if (elem_bytes != 1 && elem_bytes != 2)
    return fail(SMR_E_INVALID, "smr_ag_matmul_fused: elem_bytes must be 2 (bf16) or 1 (e4m3fn)");
  if (int rc = elem_bytes == 1 ? validate_fp8(M, N, K, rank, world_size, comm_block_m, &why)
                               : validate(M, N, K, rank, world_size, comm_block_m, &why))
    return fail(rc, why);
  if (state_dev == nullptr || buffer_ptrs_dev == nullptr)
    return fail(SMR_E_INVALID, "smr_ag_matmul_fused: state and buffer_ptrs are required");
  if (((int64_t)comm_block_m * K * elem_bytes) % 16 != 0)
    return fail(SMR_E_INVALID, "smr_ag_matmul_fused: chunks must be 16-byte multiples");
  if (producer_workgroups < 0 || producer_workgroups > 1024)
    return fail(SMR_E_INVALID, "smr_ag_matmul_fused: producer_workgroups must be 0..1024");
  const FusedArgs fa = {buffer_ptrs_dev, state_dev, producer_workgroups};
  return launch_gemm(elem_bytes, a_shard_dev, a_out_dev, b_nk_dev, c_dev, nullptr, M, N, K, rank, world_size,
                     comm_block_m, 0, status, stream, &fa);
}

static void fill_plan(int M, int N, int K, int world_size, int comm_block_m, int elem_bytes, int32_t* out5);

static int validate_fp8(int M, int N, int K, int rank, int world_size, int comm_block_m, const char** why) {
  if (int rc = smr::validate(M, N, K, rank, world_size, comm_block_m, why)) return rc;
  if (K % 128 != 0)
    *why = "smr_ag_matmul_fp8: K must be a multiple of 128";
  else if (N % 16 != 0)
    *why = "smr_ag_matmul_fp8: N must be a multiple of 16";
  return *why ? SMR_E_UNSUPPORTED : 0;
}

int smr_ag_matmul_fp8(const void* a_shard_dev, const void* a_out_dev, const void* b_nk_dev, void* c_dev,
                      const uint32_t* progress_dev, int M, int N, int K, int rank, int world_size,
                      int comm_block_m, int whole_gpu, uint32_t* status, void* stream) {
  using namespace smr;
  const char* why;
  if (int rc = validate_fp8(M, N, K, rank, world_size, comm_block_m, &why)) return fail(rc, why);
  return launch_gemm(1, a_shard_dev, a_out_dev, b_nk_dev, c_dev, progress_dev, M, N, K, rank, world_size,
                     comm_block_m, whole_gpu, status, stream, nullptr);
}

int smr_set_ag_matmul_acquire(int on) {
  smr::g_acquire_after_flag.store(on ? 1 : 0, std::memory_order_relaxed);
  return 0;
}

int smr_ag_matmul_plan_fp8(int M, int N, int K, int world_size, int comm_block_m, int32_t* out5) {
  using namespace smr;
  const char* why;
  if (int rc = validate_fp8(M, N, K, 0, world_size, comm_block_m, &why)) return fail(rc, why);
  if (out5 == nullptr) return fail(SMR_E_INVALID, "smr_ag_matmul_plan_fp8: out5 is NULL");
  fill_plan(M, N, K, world_size, comm_block_m, 1, out5);
  return 0;
}

int smr_set_ag_matmul_grid_limit(int workgroups) {
  if (workgroups < 0) return smr::fail(SMR_E_INVALID, "smr_set_ag_matmul_grid_limit: negative");
  smr::g_grid_limit.store(workgroups, std::memory_order_relaxed);
  return 0;
}

// The model's time for the ungated GEMM with the whole GPU: passes of the grid times a tile.
static double model_ungated_us(int M, int N, int K, int world_size, int comm_block_m, int elem_bytes) {
  using namespace smr;
  const GemmSchedule u = make_schedule(M, N, K, 0, world_size, comm_block_m, cu_count(), kUngated, elem_bytes);
  const int tiles = (M / u.BM) * ceil_div(N, u.BN);
  // (fitted with the rest of the model: a last pass that fills at most half of the grid counts as half a pass)
  const double passes = ceil_div(2 * tiles, u.grid) * 0.5;
  // (the tile model is that of a launch which leaves compute units idle; with all of them busy
  // the part settles at a lower clock: a workgroup's rate drops by 6 %)
  const double clock = u.grid > cu_count() - kReservedCus ? 0.94 : 1.0;
  return passes * ((model_tile_us(u.BM, u.BN, K, elem_bytes, false) - 6.0) / clock + 6.0);
}

// Fills the plan of a fused launch: {GEMM grid, producer workgroups, estimated
// microseconds fused, estimated microseconds copy-then-multiply, sequential}.
static void fill_plan(int M, int N, int K, int world_size, int comm_block_m, int elem_bytes, int32_t* out5) {
  using namespace smr;
  const int cus = cu_count();
  const GemmSchedule s = make_schedule(M, N, K, 0, world_size, comm_block_m, cus, kGatedShare, elem_bytes);
  const FusedEstimate e = estimate_fused(s, cus, s.grid, elem_bytes);
  // The alternative for a problem too small to hide the copy behind: copy with the
  // whole GPU, then multiply with the whole GPU.
  // (all chunks at once, the own shard included: read + write at what a copy reaches on the part)
  const double gather_us = 2.0 * elem_bytes * M * K / 4.8e6 + 4.0;
  const double seq_us = gather_us + model_ungated_us(M, N, K, world_size, comm_block_m, elem_bytes) + 10.0;
  out5[0] = s.grid;
  out5[1] = e.producer_wgs;
  out5[2] = (int32_t)(e.total_us + 0.5);
  out5[3] = (int32_t)(seq_us + 0.5);
  // (where the two estimates are close the launches decide: timed at the reference's nine problems, the
  // bf16 model is a few per cent hard on the fused launch of two passes and the e4m3fn model as much too
  // kind to the fused launch of the narrow problems)
  out5[4] = seq_us < e.total_us * (elem_bytes == 1 ? 1.05 : 0.98) ? 1 : 0;
}

int smr_ag_matmul_plan(int M, int N, int K, int world_size, int comm_block_m, int32_t* out5) {
  using namespace smr;
  const char* why;
  if (int rc = validate(M, N, K, 0, world_size, comm_block_m, &why)) return fail(rc, why);
  if (out5 == nullptr) return fail(SMR_E_INVALID, "smr_ag_matmul_plan: out5 is NULL");
  fill_plan(M, N, K, world_size, comm_block_m, 2, out5);
  return 0;
}

int smr_ag_matmul_pace(int M, int N, int K, int world_size, int comm_block_m, int elem_bytes, int32_t* out2) {
  using namespace smr;
  const char* why;
  if (elem_bytes != 1 && elem_bytes != 2) return fail(SMR_E_INVALID, "smr_ag_matmul_pace: elem_bytes must be 1 or 2");
  if (int rc = elem_bytes == 1 ? validate_fp8(M, N, K, 0, world_size, comm_block_m, &why)
                               : validate(M, N, K, 0, world_size, comm_block_m, &why))
    return fail(rc, why);
  if (out2 == nullptr) return fail(SMR_E_INVALID, "smr_ag_matmul_pace: out2 is NULL");
  // the launch a producer without compute units of its own feeds: gated, the whole GPU
  const GemmSchedule g = make_schedule(M, N, K, 0, world_size, comm_block_m, cu_count(), kGatedWhole, elem_bytes);
  const int per_rank = (M / world_size / g.BM) * ceil_div(N, g.BN);       // tiles of one rank's rows
  const int passes = ceil_div(per_rank * world_size, g.grid);
  if (passes <= 1) {                                  // every tile starts at once: nothing to spread
    out2[0] = 0;
    out2[1] = world_size;
    return 0;
  }
  out2[0] = (int32_t)(model_ungated_us(M, N, K, world_size, comm_block_m, elem_bytes) / world_size + 0.5);
  out2[1] = ceil_div(g.grid, per_rank);               // ranks whose tiles the first pass touches
  return 0;
}

int smr_ag_matmul_grid(int M, int N, int K, int world_size, int comm_block_m, int gated) {
  using namespace smr;
  const char* why;
  if (int rc = validate(M, N, K, 0, world_size, comm_block_m, &why)) return fail(rc, why);
  if (gated < 0 || gated > 2) return fail(SMR_E_INVALID, "smr_ag_matmul_grid: gated must be 0, 1 or 2");
  return make_schedule(M, N, K, 0, world_size, comm_block_m, cu_count(), gated).grid;
}

int smr_ag_matmul_schedule(int M, int N, int K, int rank, int world_size, int comm_block_m,
                           int gated, int32_t* out_records, int max_tiles) {
  using namespace smr;
  const char* why;
  if (int rc = validate(M, N, K, rank, world_size, comm_block_m, &why)) return fail(rc, why);
  // host-only: the schedule of a 256-CU part, the one the kernels are tuned for
  if (gated < 0 || gated > 2) return fail(SMR_E_INVALID, "smr_ag_matmul_schedule: gated must be 0, 1 or 2");
  const GemmSchedule s = make_schedule(M, N, K, rank, world_size, comm_block_m, 256, gated);
  int count = 0;
  for (int wg = 0; wg < s.grid; ++wg) {
    TileRef t;
    // the same walk as the kernel's
    for (int step = 0; next_tile(s, wg, step, t); ++step) {
      if (out_records != nullptr && count < max_tiles) {
        int32_t* rec = out_records + (size_t)count * 8;
        rec[0] = wg;
        rec[1] = step;
        rec[2] = t.row0;
        rec[3] = t.col0;
        rec[4] = s.BM;
        rec[5] = s.BN;
        rec[6] = t.comm_block;
        rec[7] = t.local;
      }
      ++count;
    }
  }
  return count;
}

}  // extern "C"
