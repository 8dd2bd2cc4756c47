/*
 * smr.h - C ABI of libsmr_gfx950.so: the symmetric-memory hot path
 * (one-shot all-reduce, blockwise barrier / signal-pad flags, all-gather matmul,
 * split-K GEMV + reduce) as hand-written HIP kernels for MI355X (gfx950).
 *
 * Conventions for every entry point
 *   - returns int: 0 on success, otherwise a hipError_t value or a negative
 *     SMR_E_* code; smr_last_error_string() describes the last failure of the
 *     calling thread.  Nothing throws.
 *   - all pointers are borrowed; "dev" pointers are device addresses.
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); the
 *     work is enqueued asynchronously on it.
 *   - `status` (nullable) is a device array of SMR_STATUS_WORDS uint32.  Every
 *     in-kernel spin is bounded by the spin timeout; a spin that expires writes
 *     a SMR_ST_* code into status[0] (first error wins), the identity of the
 *     waiter into status[1..3], and the kernel carries on to its end so that the
 *     grid always drains.  status[0] == 0 after a synchronize means the result
 *     is valid.
 *   - "emulated ranks": the multi-GPU symmetric-memory layout is emulated on one
 *     GPU.  `buffer_ptrs_dev` / `signal_pad_ptrs_dev` are device arrays of
 *     world_size uint64 addresses (one buffer / one zero-initialised uint32 pad
 *     per rank), exactly what the reference hands to its kernels
 *     (symm_mem_recipes/triton_one_shot_all_reduce.py:115-116,
 *     symm_mem_recipes/triton_barrier.py:167).
 *
 * The device functions of the flag protocol (blockwise_barrier, send_signal, wait_signal,
 * wait_signal_reset), which the reference's kernels import from one another, are in
 * smr_device.h for HIP kernels of other libraries; this header is the host side.
 */
#ifndef SMR_H_
#define SMR_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SMR_VERSION 111

#define SMR_DTYPE_BF16 0
#define SMR_DTYPE_FP32 1
#define SMR_DTYPE_BF16_STEPWISE 2 /* bf16 buffers, accumulator rounded to bf16 after every add:
                                   the reference's add.bf16x2 chain, triton_one_shot_all_reduce.py:36-49,84-89 */

#define SMR_MAX_WORLD_SIZE 8
#define SMR_STATUS_WORDS 4

/* negative return codes (argument validation on the host) */
#define SMR_E_INVALID   (-1)  /* bad argument (null pointer, size, alignment, dtype) */
#define SMR_E_UNSUPPORTED (-2) /* shape the kernels do not cover */

/* status[0] codes written by kernels */
#define SMR_ST_OK            0u
#define SMR_ST_SEND_TIMEOUT  1u  /* CAS 0->1 on a peer's slot never succeeded (stale non-zero pad) */
#define SMR_ST_WAIT_TIMEOUT  2u  /* a flag that was waited on never arrived */
#define SMR_ST_MISMATCH      3u  /* signal-round checksum differed from the expected value */

/* barrier_mode of smr_one_shot_all_reduce */
#define SMR_BARRIER_NONE   0  /* no handshake: peers' data are already stream-ordered */
#define SMR_BARRIER_PROXY  1  /* the rank's blocks run the real handshake; spare lanes of the
                                 wave that does it play the absent ranks' halves */
#define SMR_BARRIER_BOTH   2  /* as PROXY, and a second handshake after the last store: the
                                 reference has none behind triton_one_shot_all_reduce.py:93, so
                                 a peer may overwrite its buffer while others still read it */

int smr_version(void);
const char* smr_last_error_string(void);

/* Bound for every in-kernel spin, in microseconds of the GPU's constant-rate
 * clock.  0 = unbounded, which is what the reference does
 * (triton_barrier.py:119-129, triton_all_gather_matmul.py:80-83).  Default 2 s. */
int smr_set_spin_timeout_us(int64_t us);

/* Diagnostics: register (or, with NULL/0, remove) a device buffer of uint64 words
 * into which the all-gather producer and the GEMM write time stamps of the
 * GPU's 100 MHz constant clock.  Words 0..62: time progress flag i was raised,
 * word 63: producer start.  Words 64 + (workgroup*16 + step)*4 + k: GEMM
 * workgroup's step-th tile, k = 0 tile picked (step 0: kernel entry), 1 flag wait
 * over (in a fused launch: the workgroup's copying at the chunk included), 2 K loop
 * done, 3 tile stored.  Needs 64 + 256*16*4 words for the GEMM part.  The reference's
 * counterpart is its profiler hook (symm_mem_recipes/utils.py:41-52). */
int smr_set_trace_buffer(uint64_t* trace_dev, int64_t words);
int64_t smr_get_spin_timeout_us(void);

/* One-shot all-reduce.  Replaces one_shot_all_reduce_kernel + its launch
 * (symm_mem_recipes/triton_one_shot_all_reduce.py:59-93, :114-124).
 *   out[j] = cast(((0 + buf_0[j]) + buf_1[j]) + ... + buf_{ws-1}[j]), fp32 accumulator.
 *   numel      elements per buffer; 16-byte multiple (bf16: %8, fp32: %4), as :103-105
 *   rank       0..ws-1: that rank's share.  -1: all emulated ranks in one launch
 *              (out is then [ws, numel], and the ranks run the real barrier
 *              against each other when barrier_mode != NONE)
 *   dtype      SMR_DTYPE_BF16 / _FP32: fp32 accumulator as above; _BF16_STEPWISE: the
 *              accumulator is rounded to bf16 after every add, as :36-49 does
 *   write_all  0: result goes to `out`.  1: result is written back into all ws
 *              peer buffers in place (`out` may be NULL).  With rank = -1 this is the
 *              two-shot form: rank r reduces slots [numel/16*r/ws, numel/16*(r+1)/ws)
 *              only and writes them to every peer, between two handshakes
 *              (barrier_mode must be SMR_BARRIER_BOTH); no reference counterpart
 *   signal_pad_ptrs_dev may be NULL when barrier_mode == SMR_BARRIER_NONE;
 *              each pad must hold smr_reduce_num_blocks(...) * ws uint32 slots. */
int smr_one_shot_all_reduce(const uint64_t* buffer_ptrs_dev, const uint64_t* signal_pad_ptrs_dev,
                            void* out, int64_t numel, int dtype, int rank, int world_size,
                            int write_all, int barrier_mode, uint32_t* status, void* stream);

/* The same call for a host that knows the peers' addresses: `buffer_ptrs_host` and
 * `signal_pad_ptrs_host` (NULL allowed when barrier_mode == SMR_BARRIER_NONE) are HOST arrays
 * of world_size device addresses, read during the call and passed to the kernel as
 * arguments, so no thread starts with a dependent load from the device tables that the
 * reference's kernels read (triton_one_shot_all_reduce.py:86-87, triton_barrier.py:100-110):
 * one memory round trip less in front of the data, one in front of the handshake.
 * Everything else, results included, as smr_one_shot_all_reduce. */
int smr_one_shot_all_reduce_addrs(const uint64_t* buffer_ptrs_host, const uint64_t* signal_pad_ptrs_host,
                                  void* out, int64_t numel, int dtype, int rank, int world_size,
                                  int write_all, int barrier_mode, uint32_t* status, void* stream);

/* Number of workgroups (= barrier blocks per rank) the reduce launches for a
 * message; host-only.  Counterpart of the grid formula at
 * triton_one_shot_all_reduce.py:97-109, resized for 256 CUs. */
int smr_reduce_num_blocks(int64_t numel, int dtype);

/* Tuning knob: threads per workgroup (multiple of 64, <= 1024) and the cap on
 * workgroups of the reduce; 0 restores a default.  Process-wide.  The reference
 * hard-codes its counterparts (MAX_NUM_BLOCKS, NUM_WARPS,
 * triton_one_shot_all_reduce.py:97-100). */
int smr_set_reduce_launch(int threads, int max_blocks);

/* Blockwise barrier, `rounds` back-to-back rounds on `num_blocks` blocks.
 * Replaces barrier_test_kernel / barrier_test (symm_mem_recipes/triton_barrier.py:156-170)
 * around the device function blockwise_barrier (:50-153).
 *   rank -1: all ws emulated ranks in one launch (ws*num_blocks workgroups)
 *   rank >= 0: only that rank's num_blocks workgroups; its peers must be running
 *              concurrently on other streams or the spins time out.
 *   order_memory 1: every round releases the workgroup's earlier writes before the
 *              sends and acquires after the waits, as the reference's barrier does
 *              (release CAS :119-122, acquire loads :145-153).  0: flags only,
 *              for data handed over with coherent accesses. */
int smr_barrier(const uint64_t* signal_pad_ptrs_dev, int rank, int world_size, int num_blocks,
                int rounds, int order_memory, uint32_t* status, void* stream);

/* Host-callable halves of the flag protocol, one workgroup each.
 * smr_send_signal: release-CAS 0->1 (triton_barrier.py:119-122).
 * smr_wait_signal: spin until *addr == 1, acquire; never resets the flag
 *                  (symm_mem_recipes/triton_all_gather_matmul.py:72-95).
 * smr_wait_signal_reset: CAS 1->0 (triton_barrier.py:124-129).
 * smr_stream_write_value32: stream-ordered release store of `value`, the
 *                  stand-in for symm_mem.stream_write_value32
 *                  (triton_all_gather_matmul.py:50-55). */
int smr_send_signal(uint32_t* addr_dev, uint32_t* status, void* stream);
int smr_wait_signal(const uint32_t* addr_dev, uint32_t* status, void* stream);
int smr_wait_signal_reset(uint32_t* addr_dev, uint32_t* status, void* stream);
int smr_stream_write_value32(uint32_t* addr_dev, uint32_t value, void* stream);

/* Producer/consumer signal-pad round benchmark: ws*num_blocks workgroups; in each
 * round workgroup (rank r, block b) publishes its chunk (src words + round) into
 * rank r's symmetric buffer, runs the blockwise handshake for block b, then sums
 * the ws chunks of block b and compares with expected_base[b] + ws*words*round.
 * No counterpart kernel in the reference; it drives blockwise_barrier
 * (triton_barrier.py:50-153) with a payload.
 *   src_dev          uint32 [ws, num_blocks, chunk_bytes/4] payload source
 *   buffer_ptrs_dev  ws symmetric buffers, each >= 2*num_blocks*chunk_bytes
 *                    (two halves alternate by round parity)
 *   expected_base_dev uint32 [num_blocks]: wrapping sum of the ws source chunks of a block
 *   checksums_dev    uint32 [ws, num_blocks]: the last round's sums
 *   mismatches_dev   uint32 [1]: number of (rank, block, round) sums that differed
 *   chunk_bytes      0 = flags only (no payload), else a multiple of 16 */
int smr_signal_round(const uint32_t* src_dev, const uint64_t* buffer_ptrs_dev,
                     const uint64_t* signal_pad_ptrs_dev, const uint32_t* expected_base_dev,
                     uint32_t* checksums_dev, uint32_t* mismatches_dev, int world_size,
                     int num_blocks, int64_t chunk_bytes, int rounds, uint32_t* status,
                     void* stream);

/* All-gather producer.  Replaces all_gather_with_progress
 * (symm_mem_recipes/triton_all_gather_matmul.py:20-56): copies every peer's
 * shard into a_out in the order rank+1, ..., rank+ws-1, rank and, after each
 * chunk, release-stores 1 into progress[src*splits_per_rank + split].
 *   buffer_ptrs_dev  ws shard addresses (each shard_bytes long)
 *   counters_dev     uint32 [ws*splits_per_rank] scratch, zero on entry
 *   num_workgroups   copy workgroups (0 = default); kept small on purpose so the
 *                    producer shares the GPU with the consumer GEMM */
int smr_all_gather_with_progress(const uint64_t* buffer_ptrs_dev, void* a_out_dev,
                                 uint32_t* progress_dev, uint32_t* counters_dev, int rank,
                                 int world_size, int64_t shard_bytes, int splits_per_rank,
                                 int num_workgroups, void* stream);

/* The same gather for a caller that does not watch the flags on the way (a GEMM queued
 * behind it in stream order): all chunks are copied together and every flag is raised at
 * the end.  Same arguments and the same final state of a_out, progress and counters as
 * smr_all_gather_with_progress (triton_all_gather_matmul.py:20-56 run to completion). */
int smr_all_gather_at_once(const uint64_t* buffer_ptrs_dev, void* a_out_dev,
                           uint32_t* progress_dev, uint32_t* counters_dev, int rank,
                           int world_size, int64_t shard_bytes, int splits_per_rank,
                           int num_workgroups, void* stream);

/* Flag-gated bf16 GEMM.  Replaces matmul_kernel_tma_persistent and its launch
 * (symm_mem_recipes/triton_all_gather_matmul.py:98-193, :287-315).
 *   C[M,N] = A[M,K] * B[N,K]^T, fp32 accumulate, bf16 output, all row-major.
 *   Rows of the local comm blocks (those owned by `rank`) are read from a_shard,
 *   all others from a_out after waiting for progress[comm_block] == 1; tiles are
 *   visited starting at the local shard and proceeding in ring order.
 *   progress_dev NULL = ungated (the reference's mm_only comparator, :246-247).
 *   comm_block_m  rows per progress flag = M / ws / splits_per_rank.
 *   whole_gpu     only looked at for a gated launch.  0: the launch leaves compute units free
 *                 for a producer kernel that needs them (smr_all_gather_with_progress; see
 *                 smr_ag_matmul_grid).  1: whoever raises the flags needs no compute units of
 *                 his own - copy engines as in the reference (:46-55), or smr_all_gather_beside,
 *                 whose workgroups fit beside this kernel's on the same compute units - and the
 *                 launch takes every compute unit, like an ungated one. */
int smr_ag_matmul(const void* a_shard_dev, const void* a_out_dev, const void* b_nk_dev,
                  void* c_dev, const uint32_t* progress_dev, int M, int N, int K, int rank,
                  int world_size, int comm_block_m, int whole_gpu, uint32_t* status, void* stream);

/* The same producer (same arguments, same order of chunks and flags, same final state) in a
 * form that needs no compute units of its own, like the copy engines it stands in for
 * (triton_all_gather_matmul.py:46-55): workgroups of 256 threads with a few dozen registers and
 * no LDS, which the hardware places beside the GEMM's workgroups on the same compute units (a
 * bf16 GEMM workgroup leaves at least 88 of a SIMD's 512 registers per lane).  The GEMM it
 * feeds is launched with whole_gpu = 1.  The first rank's chunks - the ones half of the GEMM's
 * workgroups wait for at the start - are copied at full speed, the others on a timetable when
 * the caller gives one (step_us, lead_ranks): the GEMM needs a rank's chunks per world_size-th
 * of its run, and a copy that runs flat out beside it slows it down.
 * Exception: the 256x256 tile of smr_ag_matmul_fp8 takes every register of its compute unit,
 * so nothing fits beside it - with that GEMM use smr_all_gather_with_progress and whole_gpu = 0.
 *   num_workgroups  0 = one per compute unit of a 256-CU part
 *   step_us, lead_ranks  the timetable (smr_ag_matmul_pace gives both for a GEMM).  The ranks at
 *                   ring positions 1 .. lead_ranks-1 (1 = the next rank) are copied flat out: the
 *                   GEMM's first pass waits for them.  The rank at position r >= lead_ranks is
 *                   spread over [r - lead_ranks, r - lead_ranks + 1) * step_us from the kernel's
 *                   start, less a margin of an eighth; a producer that is behind its timetable
 *                   copies flat out.  step_us = 0: no timetable, everything flat out - right for a
 *                   GEMM that is shorter than the copy, 2 % slower for the M=16384 N=3584 K=8192 one. */
int smr_all_gather_beside(const uint64_t* buffer_ptrs_dev, void* a_out_dev, uint32_t* progress_dev,
                          uint32_t* counters_dev, int rank, int world_size, int64_t shard_bytes,
                          int splits_per_rank, int num_workgroups, int64_t step_us, int lead_ranks,
                          void* stream);

/* Host-only: the timetable on which a gated smr_ag_matmul (elem_bytes 2) or smr_ag_matmul_fp8 (1)
 * with whole_gpu = 1 needs its chunks on the current device.  out2 = {step_us, lead_ranks} for
 * smr_all_gather_beside: a world_size-th of the planner's estimate of the GEMM's time, and the
 * number of ranks whose tiles the first pass of the persistent grid touches (the local one
 * included).  {0, world_size} for a GEMM of a single pass, which needs everything at once.
 * Negative SMR_E_* for shapes the GEMM refuses.  No reference counterpart (its copy engines
 * run flat out and disturb nobody, triton_all_gather_matmul.py:46-55). */
int smr_ag_matmul_pace(int M, int N, int K, int world_size, int comm_block_m, int elem_bytes, int32_t* out2);

/* Host-only: the tile order smr_ag_matmul uses on a 256-CU part.  Writes up to
 * max_tiles records of 8 int32 (workgroup, step, row0, col0, tile rows, tile
 * columns, comm_block, local; grouped by workgroup, in visiting order) and
 * returns the number of tiles, or a negative SMR_E_* code.
 * Counterpart of the index arithmetic at triton_all_gather_matmul.py:125-174.
 *   gated  0: ungated launch, 1: gated with compute units left to a producer kernel,
 *          2: gated with whole_gpu = 1 */
int smr_ag_matmul_schedule(int M, int N, int K, int rank, int world_size, int comm_block_m,
                           int gated, int32_t* out_records, int max_tiles);

/* The whole all-gather matmul in one launch on one stream.  Replaces the body of
 * all_gather_matmul_tma_persistent (symm_mem_recipes/triton_all_gather_matmul.py:246-318:
 * fresh flags, producer on a second stream, persistent GEMM, stream join).  The reference's
 * producer is a copy engine and costs no SMs; on one GPU the copy runs on compute units, and
 * here it runs inside the GEMM's own grid:
 *   - `producer_workgroups` extra workgroups (0 = the plan's, see smr_ag_matmul_plan; never
 *     fewer than one: the local shard reaches a_out through them) only copy: the peers'
 *     shards from buffer_ptrs_dev into a_out in the reference's order (sources rank+1, ...,
 *     rank+ws-1, rank; :43-44), in 64 KiB pieces taken by ticket;
 *   - a GEMM workgroup whose next tile's chunk is not in place takes pieces of that chunk
 *     too instead of spinning, so the launch finishes whichever of its workgroups are
 *     resident, and needs no second stream and no kernel running beside it;
 *   elem_bytes 2 = smr_ag_matmul's arithmetic (bf16), 1 = smr_ag_matmul_fp8's (e4m3fn).
 *   state_dev  uint32 [smr_ag_matmul_fused_state_words(ws, splits)]: flags, tickets and
 *              counters.  Zero before the first launch; the last workgroup to finish zeroes
 *              it again, so the next launch (or the next replay of a captured graph) needs no
 *              fill.  One launch at a time per state array; after a launch that reported a
 *              timeout in `status` the caller must zero it.
 * On return a_out holds all ws shards and c the product; c is identical, bit for bit, to
 * smr_ag_matmul on the gathered operand. */
int smr_ag_matmul_fused(const void* a_shard_dev, void* a_out_dev, const void* b_nk_dev, void* c_dev,
                        uint32_t* state_dev, const uint64_t* buffer_ptrs_dev, int elem_bytes, int M,
                        int N, int K, int rank, int world_size, int comm_block_m,
                        int producer_workgroups, uint32_t* status, void* stream);
int smr_ag_matmul_fused_state_words(int world_size, int splits_per_rank);

/* The same GEMM with e4m3fn (OCP FP8) operands and result, fp32 accumulation: the
 * reference's FP8_OUTPUT switch (triton_all_gather_matmul.py:115,123,188,311).  The cast of
 * the accumulator rounds to nearest even and saturates to +-448, NaN stays NaN (what
 * Triton's cast compiles to on the reference's hardware, cvt.rn.satfinite).
 * K % 128 == 0, N % 16 == 0; otherwise as smr_ag_matmul (same tile shapes, same schedule). */
int smr_ag_matmul_fp8(const void* a_shard_dev, const void* a_out_dev, const void* b_nk_dev, void* c_dev,
                      const uint32_t* progress_dev, int M, int N, int K, int rank, int world_size,
                      int comm_block_m, int whole_gpu, uint32_t* status, void* stream);
/* smr_ag_matmul_plan for the e4m3fn GEMM. */
int smr_ag_matmul_plan_fp8(int M, int N, int K, int world_size, int comm_block_m, int32_t* out5);

/* Host-only: how a fused launch of this shape splits the GPU.  out5 = {GEMM grid,
 * producer workgroups, fused_us, sequential_us, sequential}.  The first two are the split
 * of a fused launch: smr_ag_matmul gated uses that grid, the producer
 * (smr_all_gather_with_progress) gets that many workgroups beside it.  fused_us and
 * sequential_us are the planner's estimates, in microseconds, of that launch and of the
 * alternative: gather with the whole GPU (smr_all_gather_at_once, one workgroup per
 * compute unit), then smr_ag_matmul with progress = NULL behind it in stream order.
 * sequential = 1 recommends the alternative (its estimate is the lower one by a margin fitted to
 * timed launches, 2 % for bf16, -5 % for e4m3fn): the GEMM is too short to hide the copy behind.
 * Replaces the fixed NUM_SMS grid of triton_all_gather_matmul.py:287-294: there the copy
 * engines cost no SMs. */
int smr_ag_matmul_plan(int M, int N, int K, int world_size, int comm_block_m, int32_t* out5);

/* 1: the gated GEMM issues an acquire fence (cache invalidate) behind every flag wait, as a
 * literal reading of wait_signal + the loads that follow (triton_all_gather_matmul.py:72-95,
 * 170-174) asks for.  0 (default): flag poll past the caches and a workgroup barrier only;
 * the rows of a comm block cannot be in a cache before its flag is up, because nobody reads
 * them earlier inside the launch and a launch starts from invalidated caches.
 * Preconditions of the default, which the caller owns: (1) nothing else on the GPU reads
 * a_out while the launch runs (a concurrent reader on another stream could leave lines of
 * a chunk in an L2 before its flag); (2) whoever writes a chunk writes it through to memory
 * (agent-scope or system-scope stores, DMA) and raises the flag only after the writes are
 * acknowledged - this library's producers do.  A caller that cannot promise both turns the
 * fence on.  Process-wide. */
int smr_set_ag_matmul_acquire(int on);

/* Tuning knob: cap on the workgroups of the GEMM's persistent grid (rounded down to a multiple
 * of 8; 0 = none), for measuring how the kernel scales with the compute units it is given.
 * Process-wide.  No reference counterpart (its grid is NUM_SMS, triton_all_gather_matmul.py:287-294). */
int smr_set_ag_matmul_grid_limit(int workgroups);

/* Workgroups smr_ag_matmul launches on the current device for this shape (gated: 0, 1 or 2
 * as for smr_ag_matmul_schedule); a gated launch without whole_gpu keeps at least 8 compute
 * units free for the producer, whose workgroup count should not exceed the number left free.
 * Host-only, no reference counterpart (the reference's producer is a copy
 * engine and needs no compute units, triton_all_gather_matmul.py:46-49). */
int smr_ag_matmul_grid(int M, int N, int K, int world_size, int comm_block_m, int gated);

/* Split-K GEMV + rank-ordered combine through signal-pad flags.  No reference
 * code exists for it in symm_mem_recipes; it reuses the send/wait protocol of
 * triton_barrier.py:119-129 and triton_all_gather_matmul.py:72-95.
 *   x [batch,K] bf16, w [K,N] bf16 row-major, K split into ws rank shards, each
 *   cut further into sub-shards (one workgroup per column block and sub-shard);
 *   S = smr_gemv_senders(N, K, ws) partial producers per column block.
 *   partials fp32 [S, batch, N] scratch; flags uint32 [smr_gemv_flag_words(N, K, ws)]
 *   (= smr_gemv_flag_blocks(N) * (S + 1): per column block one flag per producer and one
 *   arrival word), zero on entry and zero again on exit.  Every producer raises its flag and
 *   counts itself in; the one that arrives last consumes the flags and adds the partials:
 *   out [batch,N] bf16 = the fp32 sum of the S partials in sender order (rank-major), i.e.
 *   bf16(((0 + p_0) + p_1) + ... + p_{ws-1}) when S == ws.  batch <= 8.
 *   partials_bytes, flag_words: what the caller allocated for the two scratch arrays.  The
 *   layout of both follows the process-wide launch knobs (smr_set_gemv_launch), so a caller
 *   that sized them under another setting is told (SMR_E_INVALID) instead of having the
 *   kernel write past the end. */
int smr_gemv_allreduce(const void* x_dev, const void* w_dev, float* partials_dev, int64_t partials_bytes,
                       uint32_t* flags_dev, int64_t flag_words, void* out_dev, int batch, int K, int N,
                       int world_size, uint32_t* status, void* stream);
int smr_gemv_flag_blocks(int N);
int smr_gemv_senders(int N, int K, int world_size);
int smr_gemv_flag_words(int N, int K, int world_size);

/* smr_gemv_allreduce for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Same kernels, same result bit for bit; the fp32 partials and the flags live in
 * a fixed array inside the library (one copy per GPU, 4 MiB + 16 KiB, held until the process
 * ends) instead of caller-provided scratch, and the call allocates nothing.
 *   Limits: smr_gemv_senders(N, K, ws) * batch * N * 4 <= smr_gemv_static_scratch_bytes()
 *   (4 MiB; K = N = 8192, batch 8, ws 8 needs 2 MiB) and smr_gemv_flag_words(N, K, ws) <= 4096
 *   (one word per workgroup and one per column block); beyond them SMR_E_UNSUPPORTED.
 *   Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two
 *   streams, two threads) race and must be serialised by the caller.  The flags are cleared
 *   by a small kernel ahead of the launch, so a call that timed out leaves nothing behind. */
int smr_gemv_allreduce_static(const void* x_dev, const void* w_dev, void* out_dev, int batch, int K,
                              int N, int world_size, uint32_t* status, void* stream);
int64_t smr_gemv_static_scratch_bytes(void);
/* Tuning knob: threads per contiguous row segment (16 or 64; 0 = default 16) and
 * sub-shards per rank (1..8; 0 = chosen so that at least 256 workgroups run). */
int smr_set_gemv_launch(int threads_per_row, int sub_shards);
/* Tuning knob: 1 (default) runs batches of 3..8 rows on the matrix cores (W tiles turned
 * through LDS with transposing reads, v_mfma_f32_16x16x32_bf16 with x padded to 16 rows);
 * 0 keeps every batch on the vector ALUs (v_dot2c_f32_bf16), as batches of 1 and 2 always
 * are.  The two kernels add a rank's K rows in different orders: their fp32 partials agree
 * to rounding, not bit for bit.  Process-wide. */
int smr_set_gemv_matrix_cores(int on);

#ifdef __cplusplus
}
#endif
#endif /* SMR_H_ */
