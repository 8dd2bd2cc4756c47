// CPU model of the fused launch's copy protocol.  The copy functions of ag_matmul.hip are
// compiled for the host (FRAGMENT is cut from the source by the test) and run with one host
// thread per GPU thread: copy-only workgroups walk the chunks in the reference's order while
// "waiting GEMM workgroups" take pieces of chunks in another order, then everybody leaves.
// Checked: every byte copied exactly where it belongs, no access outside the buffers (also by
// AddressSanitizer), every chunk's flag raised, the state array zero again at the end.
//
//   harness rows row_vecs world_size splits copy_workgroups helper_workgroups
#include <atomic>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <pthread.h>
#include <thread>
#include <vector>
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
#define __device__
#define __forceinline__ inline __attribute__((always_inline))
#define kScope 5 /* system scope: any valid scope will do on the host */
constexpr int kGemmThreads = 256;
constexpr int kTraceProducerWords = 64;
struct Dim { uint32_t x; };
static thread_local Dim threadIdx, blockIdx;
static Dim gridDim;
static thread_local pthread_barrier_t* wg_barrier;
static thread_local uint32_t* wg_lds;
static void __syncthreads() { pthread_barrier_wait(wg_barrier); }
static uint32_t* lds_ptr(uint32_t off) { return wg_lds + off / 4; }
static uint64_t wall_clock64() { return 1; }
static void wait_stores_acknowledged() {}
static const u32x4* g_src_lo; static const u32x4* g_src_hi; static u32x4* g_dst_lo; static u32x4* g_dst_hi;
static void out_of_bounds(const char* what, long at) { fprintf(stderr, "%s out of bounds at vector %ld\n", what, at); abort(); }
static void store_checked(u32x4* p, const u32x4& v) { if (p < g_dst_lo || p >= g_dst_hi) out_of_bounds("store", (long)(p - g_dst_lo)); *p = v; }
static u32x4 load_checked(const u32x4* p) { if (p < g_src_lo || p >= g_src_hi) out_of_bounds("load", (long)(p - g_src_lo)); return *p; }
namespace smr {
#include FRAGMENT
}
using namespace smr;

int main(int argc, char** argv) {
  if (argc != 7) return 2;
  const int rows = atoi(argv[1]), row_vecs = atoi(argv[2]), ws = atoi(argv[3]), splits = atoi(argv[4]),
            copy_wgs = atoi(argv[5]), helper_wgs = atoi(argv[6]);
  const int chunks = ws * splits;
  const int64_t chunk_vecs = (int64_t)rows * row_vecs;
  std::vector<u32x4> src(chunk_vecs * chunks), dst(chunk_vecs * chunks);
  for (size_t i = 0; i < src.size(); ++i) src[i] = u32x4{(uint32_t)i, (uint32_t)(i >> 32), 7u, (uint32_t)(i * 2654435761u)};
  memset(dst.data(), 0xEE, dst.size() * 16);
  g_src_lo = src.data(); g_src_hi = src.data() + src.size(); g_dst_lo = dst.data(); g_dst_hi = dst.data() + dst.size();
  std::vector<uint64_t> ptrs(ws);
  for (int r = 0; r < ws; ++r) ptrs[r] = (uint64_t)(uintptr_t)(src.data() + (int64_t)r * splits * chunk_vecs);
  std::vector<uint32_t> state(3 * chunks + 1, 0);
  CopyJob job = {};
  job.buffer_ptrs = ptrs.data(); job.a_out = (uint8_t*)dst.data();
  job.flags = state.data(); job.tickets = state.data() + chunks; job.finished = state.data() + 2 * chunks;
  job.exits = state.data() + 3 * chunks;
  job.chunk_vecs = chunk_vecs; job.pieces = (int)((chunk_vecs + kPullPieceVecs - 1) / kPullPieceVecs);
  job.chunks = chunks; job.splits = splits; job.rank = 0; job.world_size = ws; job.gemm_grid = helper_wgs;
  const int wgs = copy_wgs + helper_wgs;
  gridDim.x = wgs;
  std::vector<pthread_barrier_t> bars(wgs);
  std::vector<std::vector<uint32_t>> lds(wgs, std::vector<uint32_t>(64));
  for (auto& b : bars) pthread_barrier_init(&b, nullptr, kGemmThreads);
  std::vector<std::thread> th;
  std::vector<uint64_t> trace(kTraceProducerWords, 0);
  for (int w = 0; w < wgs; ++w)
    for (int t = 0; t < kGemmThreads; ++t)
      th.emplace_back([&, w, t]() {
        threadIdx.x = t; blockIdx.x = w; wg_barrier = &bars[w]; wg_lds = lds[w].data();
        if (w >= helper_wgs) {
          for (int step = 0; step < job.world_size; ++step) {
            const int src_rank = (job.rank + step + 1) % job.world_size;
            for (int split = 0; split < job.splits; ++split) copy_pieces<2>(job, src_rank * job.splits + split, 0, trace.data());
          }
        } else {
          for (int c = chunks - 1; c >= 0; --c) copy_pieces<1>(job, (c + w) % chunks, 0, trace.data());
        }
        leave(job);
      });
  for (auto& t : th) t.join();
  int bad = 0;
  if (memcmp(src.data(), dst.data(), src.size() * 16) != 0) { bad = 1; fprintf(stderr, "data mismatch\n"); }
  for (auto v : state) if (v) { bad = 1; fprintf(stderr, "state not zero\n"); break; }
  for (int c = 0; c < chunks && c < kTraceProducerWords - 1; ++c) if (!trace[c]) { bad = 1; fprintf(stderr, "flag of chunk %d never raised\n", c); }
  printf("rows %d row_vecs %d ws %d splits %d copy %d helpers %d: %s\n", rows, row_vecs, ws, splits, copy_wgs, helper_wgs, bad ? "FAIL" : "ok");
  return bad;
}
