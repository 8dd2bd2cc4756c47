/*
 * CPU model of the blockwise barrier's flag protocol.  TEST INFRASTRUCTURE ONLY:
 * built and run by the test suite, never linked into the library.
 *
 * Restates symm_mem_recipes/triton_barrier.py:100-139 with C11 atomics and one
 * host thread per rank: for block b, rank k sends by CAS(pad[r][b*ws + k], 0 -> 1)
 * with release order and waits by CAS(pad[k][b*ws + r], 1 -> 0); an acquire fence
 * follows, as the reference's acquire loads do (:145-153).  No slot is ever reset
 * from outside.
 *
 * What it checks, for `rounds` back-to-back rounds on `blocks` blocks:
 *   - termination (a watchdog aborts after 20 s),
 *   - causality: the word a rank stores before round n is what every peer reads
 *     after round n (a data race or a late flag shows up as a stale word),
 *   - all pads are zero at the end.
 * usage: barrier_model [world_size] [blocks] [rounds]   (exit code 0 = all good)
 */
#include <pthread.h>
#include <stdatomic.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <time.h>

#define MAX_WS 8
#define MAX_BLOCKS 64

static int g_ws = 8, g_blocks = 4, g_rounds = 2000;
static _Atomic uint32_t g_pad[MAX_WS][MAX_BLOCKS * MAX_WS];
static uint32_t g_payload[MAX_WS][MAX_BLOCKS];   /* plain memory handed over by the barrier */
static atomic_int g_errors;
static atomic_int g_done;

static void barrier_block(int rank, int block) {
  const int ws = g_ws;
  for (int r = 0; r < ws; ++r) { /* send half, triton_barrier.py:119-122 */
    uint32_t expected = 0;
    while (!atomic_compare_exchange_weak_explicit(&g_pad[r][block * ws + rank], &expected, 1u,
                                                  memory_order_release, memory_order_relaxed))
      expected = 0;
  }
  for (int r = 0; r < ws; ++r) { /* wait half, :124-129 (relaxed: acquire follows) */
    uint32_t expected = 1;
    while (!atomic_compare_exchange_weak_explicit(&g_pad[rank][block * ws + r], &expected, 0u,
                                                  memory_order_relaxed, memory_order_relaxed))
      expected = 1;
  }
  atomic_thread_fence(memory_order_acquire); /* :145-153 */
}

static void* rank_main(void* arg) {
  const int rank = (int)(intptr_t)arg;
  for (int n = 0; n < g_rounds; ++n) {
    for (int b = 0; b < g_blocks; ++b) {
      g_payload[rank][b] = (uint32_t)(n * 131 + rank * 17 + b);
      barrier_block(rank, b);
      for (int r = 0; r < g_ws; ++r)
        if (g_payload[r][b] != (uint32_t)(n * 131 + r * 17 + b)) atomic_fetch_add(&g_errors, 1);
      /* second barrier: nobody overwrites its word while a peer still reads it */
      barrier_block(rank, b);
    }
  }
  atomic_fetch_add(&g_done, 1);
  return NULL;
}

int main(int argc, char** argv) {
  if (argc > 1) g_ws = atoi(argv[1]);
  if (argc > 2) g_blocks = atoi(argv[2]);
  if (argc > 3) g_rounds = atoi(argv[3]);
  if (g_ws < 1 || g_ws > MAX_WS || g_blocks < 1 || g_blocks > MAX_BLOCKS || g_rounds < 1) {
    fprintf(stderr, "bad arguments\n");
    return 2;
  }
  pthread_t th[MAX_WS];
  for (int k = 0; k < g_ws; ++k) pthread_create(&th[k], NULL, rank_main, (void*)(intptr_t)k);
  const time_t t0 = time(NULL);
  while (atomic_load(&g_done) < g_ws) {
    if (time(NULL) - t0 > 20) {
      fprintf(stderr, "barrier_model: no termination within 20 s\n");
      return 3;
    }
    struct timespec ts = {0, 2000000};
    nanosleep(&ts, NULL);
  }
  for (int k = 0; k < g_ws; ++k) pthread_join(th[k], NULL);
  int nonzero = 0;
  for (int k = 0; k < g_ws; ++k)
    for (int i = 0; i < g_blocks * g_ws; ++i) nonzero += atomic_load(&g_pad[k][i]) != 0;
  printf("world_size=%d blocks=%d rounds=%d stale_reads=%d nonzero_slots=%d\n", g_ws, g_blocks, g_rounds,
         atomic_load(&g_errors), nonzero);
  return (atomic_load(&g_errors) == 0 && nonzero == 0) ? 0 : 1;
}
