// Split-K GEMV + all-reduce through signal-pad flags, emulated ranks on one GPU.
//
//   out[b, n] = bf16( ((0 + p_0[b,n]) + p_1[b,n]) + ... + p_{ws-1}[b,n] ),
//   p_r = x[:, shard r] @ W[shard r, :]   (fp32)
//
// The job is bound by reading W once (K*N*2 bytes).  W is row-major [K, N], so a
// row is N contiguous bf16: 16 threads cover 128 columns with one 128-bit load
// each, and the 16 thread groups of a workgroup stride over the shard's K rows,
// 8 independent loads in flight per thread.  x (at most 8 rows) is staged in LDS
// as fp32, transposed to [k][batch] so a k step reads its batch values with one
// or two broadcast 128-bit LDS reads.
//
// Workgroup id -> (column block = id / ws, rank = id % ws).  Every workgroup
// writes its fp32 partial, releases, and raises flag[column block][rank]
// (CAS 0 -> 1).  The workgroup of rank 0 then consumes the ws flags of its column
// block (CAS 1 -> 0, so the flags are zero again on exit), acquires, and adds
// the partials in rank order.
#include "smr_device.hpp"

namespace smr {

constexpr int kGemvThreads = 256;
constexpr int kGemvCols = 128;               // columns per workgroup
constexpr int kGemvTpr = kGemvCols / 8;      // threads per row segment (16)
constexpr int kGemvKGroups = kGemvThreads / kGemvTpr;   // 16
constexpr int kGemvUnroll = 8;
constexpr int kGemvKChunk = 1024;            // K rows of x staged in LDS at a time

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(1))) u32x4 GlobalVec;

template <int B>
__global__ __launch_bounds__(kGemvThreads) void gemv_allreduce_kernel(
    const uint16_t* __restrict__ x, const uint8_t* __restrict__ w, float* __restrict__ partials,
    uint32_t* __restrict__ flags, uint16_t* __restrict__ out, int batch, int K, int N,
    int world_size, uint64_t limit_ticks, uint32_t* status) {
  __shared__ __attribute__((aligned(16))) float xs[kGemvKChunk][B];
  __shared__ float red[kGemvThreads / 64][B][kGemvCols];

  const int cblk = blockIdx.x / world_size;
  const int rank = blockIdx.x % world_size;
  const int tid = threadIdx.x;
  const int col_t = tid % kGemvTpr;
  const int kg = tid / kGemvTpr;
  const int col0 = cblk * kGemvCols + col_t * 8;
  const bool col_ok = col0 < N;
  const int ks = K / world_size;
  const int k_begin = rank * ks, k_end = k_begin + ks;
  const int64_t row_bytes = (int64_t)N * 2;

  float acc[B][8];
#pragma unroll
  for (int b = 0; b < B; ++b)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[b][j] = 0.0f;

  for (int k0 = k_begin; k0 < k_end; k0 += kGemvKChunk) {
    const int kc = (k_end - k0) < kGemvKChunk ? (k_end - k0) : kGemvKChunk;
    for (int i = tid; i < kc * B; i += kGemvThreads) {
      const int b = i / kc, k = i - b * kc;
      xs[k][b] = b < batch ? bf16_lo((uint32_t)x[(int64_t)b * K + k0 + k]) : 0.0f;
    }
    __syncthreads();
    if (col_ok) {
      const GlobalVec* wp = (const GlobalVec*)(uintptr_t)(w + (int64_t)k0 * row_bytes + (int64_t)col0 * 2);
      for (int k = kg; k < kc; k += kGemvKGroups * kGemvUnroll) {
        u32x4 wv[kGemvUnroll];
#pragma unroll
        for (int u = 0; u < kGemvUnroll; ++u) {
          const int kk = k + u * kGemvKGroups;
          if (kk < kc)
            wv[u] = __builtin_nontemporal_load(
                (const GlobalVec*)((const __attribute__((address_space(1))) uint8_t*)wp + (int64_t)kk * row_bytes));
          else
            wv[u] = u32x4{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int u = 0; u < kGemvUnroll; ++u) {
          const int kk = k + u * kGemvKGroups;
          const int ksafe = kk < kc ? kk : 0;      // wv is zero past the end
          float wf[8];
          wf[0] = bf16_lo(wv[u].x); wf[1] = bf16_hi(wv[u].x);
          wf[2] = bf16_lo(wv[u].y); wf[3] = bf16_hi(wv[u].y);
          wf[4] = bf16_lo(wv[u].z); wf[5] = bf16_hi(wv[u].z);
          wf[6] = bf16_lo(wv[u].w); wf[7] = bf16_hi(wv[u].w);
#pragma unroll
          for (int b = 0; b < B; ++b) {
            const float xb = xs[ksafe][b];
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[b][j] = __builtin_fmaf(xb, wf[j], acc[b][j]);
          }
        }
      }
    }
    __syncthreads();
  }

  // combine the 16 k groups: 4 per wave by lane shuffles, then 4 waves through LDS
#pragma unroll
  for (int b = 0; b < B; ++b)
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float v = acc[b][j];
      v += __shfl_xor(v, 16, 64);
      v += __shfl_xor(v, 32, 64);
      acc[b][j] = v;
    }
  if ((tid & 63) < kGemvTpr) {
#pragma unroll
    for (int b = 0; b < B; ++b)
#pragma unroll
      for (int j = 0; j < 8; ++j) red[tid >> 6][b][col_t * 8 + j] = acc[b][j];
  }
  __syncthreads();
  const int col = cblk * kGemvCols + tid;
  if (tid < kGemvCols && col < N) {
    for (int b = 0; b < batch; ++b) {
      const float p = ((red[0][b][tid] + red[1][b][tid]) + red[2][b][tid]) + red[3][b][tid];
      partials[((int64_t)rank * batch + b) * N + col] = p;
    }
  }

  // publish the partial: every wave releases, the workgroup meets, one send
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
  __syncthreads();
  uint32_t* my_flags = flags + (size_t)cblk * world_size;
  if (tid == 0 && !send_signal(my_flags + rank, limit_ticks))
    report(status, SMR_ST_SEND_TIMEOUT, rank, cblk, 0u);
  if (rank != 0) return;

  // rank 0 of the column block: consume all ws flags, then add in rank order
  int bad = 0;
  if (tid < world_size && !wait_signal_reset(my_flags + tid, limit_ticks)) {
    report(status, SMR_ST_WAIT_TIMEOUT, tid, cblk, 0u);
    bad = 1;
  }
  bad = __syncthreads_or(bad);
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
  if (bad) return;
  if (tid < kGemvCols && col < N) {
    for (int b = 0; b < batch; ++b) {
      float a = 0.0f;
      for (int r = 0; r < world_size; ++r) a += partials[((int64_t)r * batch + b) * N + col];
      out[(int64_t)b * N + col] = (uint16_t)f32_to_bf16_bits(a);
    }
  }
}

}  // namespace smr

extern "C" {

int smr_gemv_flag_blocks(int N) { return N <= 0 ? 0 : (N + smr::kGemvCols - 1) / smr::kGemvCols; }

int smr_gemv_allreduce(const void* x_dev, const void* w_dev, float* partials_dev, uint32_t* flags_dev,
                       void* out_dev, int batch, int K, int N, int world_size, uint32_t* status,
                       void* stream) {
  using namespace smr;
  if (x_dev == nullptr || w_dev == nullptr || partials_dev == nullptr || flags_dev == nullptr ||
      out_dev == nullptr)
    return fail(SMR_E_INVALID, "smr_gemv_allreduce: null pointer");
  if (world_size < 1 || world_size > SMR_MAX_WORLD_SIZE)
    return fail(SMR_E_INVALID, "smr_gemv_allreduce: world_size must be 1..8");
  if (batch < 1 || batch > 8) return fail(SMR_E_UNSUPPORTED, "smr_gemv_allreduce: batch must be 1..8");
  if (K <= 0 || N <= 0 || K % world_size != 0)
    return fail(SMR_E_INVALID, "smr_gemv_allreduce: K must split evenly over the ranks");
  if (N % 8 != 0 || (reinterpret_cast<uintptr_t>(w_dev) & 15u))
    return fail(SMR_E_UNSUPPORTED, "smr_gemv_allreduce: N must be a multiple of 8 and W 16-byte aligned");
  const unsigned grid = (unsigned)smr_gemv_flag_blocks(N) * (unsigned)world_size;
  if (grid > 4096u)
    return fail(SMR_E_UNSUPPORTED, "smr_gemv_allreduce: more than 4096 workgroups cannot be co-resident");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const uint16_t* x = reinterpret_cast<const uint16_t*>(x_dev);
  const uint8_t* w = reinterpret_cast<const uint8_t*>(w_dev);
  uint16_t* out = reinterpret_cast<uint16_t*>(out_dev);
  const uint64_t lim = spin_limit_ticks();
#define SMR_GEMV_LAUNCH(BP)                                                                        \
  hipLaunchKernelGGL((gemv_allreduce_kernel<BP>), dim3(grid), dim3(kGemvThreads), 0, st, x, w,     \
                     partials_dev, flags_dev, out, batch, K, N, world_size, lim, status)
  if (batch == 1) SMR_GEMV_LAUNCH(1);
  else if (batch == 2) SMR_GEMV_LAUNCH(2);
  else if (batch <= 4) SMR_GEMV_LAUNCH(4);
  else SMR_GEMV_LAUNCH(8);
#undef SMR_GEMV_LAUNCH
  return check_hip(hipGetLastError(), "smr_gemv_allreduce launch");
}

}  // extern "C"
