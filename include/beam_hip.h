/*
 * beam_hip.h -- C ABI of the MI355X (gfx950) gemmrc library, libbeam_hip.so.
 *
 * gemmrc:  C[M][N] = A[M][K] . B[N][K]^T   (A, B, C row-major 16-bit; fp32 accumulation on the
 * matrix cores; round-to-nearest-even output).  All pointers are DEVICE pointers unless the
 * name says host.  Every entry point returns a beam_status; nothing aborts, nothing returns
 * silently leaving C untouched.  Launches are asynchronous on the stream passed in
 * (a hipStream_t cast to void*, NULL = the default stream).
 *
 * Each declaration cites the reference interface it stands in for
 * (paths relative to the reference repository).
 */
#ifndef BEAM_HIP_H
#define BEAM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum beam_status {
  BEAM_OK = 0,
  BEAM_ERR_INVALID = 1,     /* bad pointer / shape / argument                                 */
  BEAM_ERR_UNSUPPORTED = 2, /* tile / dtype / alignment combination that has no kernel        */
  BEAM_ERR_WORKSPACE = 3,   /* workspace missing or too small                                 */
  BEAM_ERR_HIP = 4,         /* HIP runtime error, text in beam_last_error()                   */
  BEAM_ERR_DEVICE = 5       /* not a gfx950 device                                            */
} beam_status;

typedef enum beam_dtype { BEAM_F16 = 0, BEAM_BF16 = 1 } beam_dtype;

/* One point of the tunable space.
 * Replaces the (shape_threadblock, shape_warp) pair of
 * cuda/cutlass_kernels/main.cc:125-142 and cuda/cutlass_kernels/cutlass_gemmrc.cu:85-110. */
typedef struct beam_tile_cfg {
  int block_m, block_n; /* workgroup tile of C ("shape_threadblock")                          */
  int wave_m, wave_n;   /* wavefront tile ("shape_warp"); block/wave = wavefront grid         */
  int pipeline;         /* LDS slots per operand: 0 = 3 for A + 2 for B, 1 = 2 + 2,             */
                        /* 2 = as many as fit 160 KiB, up to 8 + 7 (small tiles, split-K)       */
  int group_m;          /* rasterisation group height in tiles; 0 = library default           */
} beam_tile_cfg;

/* ---- library ------------------------------------------------------------------------- */

/* Checks that device 0 is gfx950 and raises the kernels' LDS limits.  Called implicitly.
 * Stands in for the module initialiser cuda/main.cc:51-60. */
int beam_init(void);
/* Text of the last error on the calling thread ("" if none). */
const char* beam_last_error(void);
/* name[<=len], compute units, peak engine clock (kHz), total device memory (bytes). */
int beam_device_info(char* name, int len, int* compute_units, int* clock_khz, size_t* mem_bytes);

/* ---- tunable space -------------------------------------------------------------------- */

/* Number of compiled tile configurations and the i-th of them (both dtypes share the table).
 * Replaces the hard-coded search spaces of python/beam/tuner.py:52-95. */
int beam_num_configs(void);
int beam_get_config(int index, beam_tile_cfg* out);
/* Library default for a problem: writes the configuration and, if split_k is not NULL, the
 * number of K slices that goes with it (1 = no split; the tile is then the one that is best
 * *with* that many slices and a workspace).  split_k == NULL: the best tile without a split.
 * Replaces CUTLASS's default shapes, cuda/cutlass_kernels/cutlass_gemmrc.cu:22-24. */
int beam_default_config(int M, int N, int K, beam_tile_cfg* cfg, int* split_k);

/* ---- tiled GEMM ------------------------------------------------------------------------ */

/* cfg == NULL: beam_default_config() picks the tile (never a split).
 * Replaces entry_cutlass_gemmrc / entry_cutlass_gemmrc_spec
 * (cuda/cutlass_kernels/main.cc:11-15, cutlass_gemmrc.cu:21-40,55-111). */
int beam_gemmrc(const void* A, const void* B, void* C, int M, int N, int K, int dtype,
                const beam_tile_cfg* cfg, void* stream);

/* fp16 only, fixed tiles, same argument order as the reference launchers.
 * Replace entry_custom_gemmrc_128x128 / entry_custom_gemmrc_128x256
 * (cuda/cute_kernels/main.cc:13-18, cute_gemm_128x128.cu:193-205, cute_gemm_128x256.cu:196-208);
 * 256x128 is the third tile the configuration list names. */
int beam_custom_gemmrc_128x128(const void* A, const void* B, void* C, int M, int N, int K, void* stream);
int beam_custom_gemmrc_128x256(const void* A, const void* B, void* C, int M, int N, int K, void* stream);
int beam_custom_gemmrc_256x128(const void* A, const void* B, void* C, int M, int N, int K, void* stream);

/* ---- split-K ---------------------------------------------------------------------------- */

/* The reference's slice count for `tiles` output tiles on `compute_units` CUs: the rule of
 * get_slice_heuristic (cuda/cutlass_kernels/cutlass_gemmrc_splitk.cu:44-57) with the device's
 * CU count in place of the hard-coded 108.  Kept for callers that want that rule; it aims at a
 * last round of workgroups that is at least half full, which on this machine (one workgroup
 * of a split-K tile per CU, launch-latency bound) is slower than exactly one full round, so
 * beam_gemmrc_splitk with split_k <= 0 uses floor(CUs / tiles) instead (at most 64, at least
 * 4 K tiles of 64 per slice, and no more slices than give 16 K tiles each once half the CUs are busy;
 * 1 when the tiles already fill half the CUs). */
int beam_slice_heuristic(int tiles, int compute_units);
/* Bytes of workspace for `split_k` slices: the fp32 partial results [split_k][M][N] and, behind them, the
 * synchronisation words of the one-launch form (a few KiB).  Replaces the hidden grow-only buffer
 * get_the_buffer, cutlass_gemmrc_splitk.cu:31-42: the caller owns the workspace.  The workspace never has
 * to be cleared or prepared, and may be shared by calls of any shapes that do not overlap in time. */
size_t beam_splitk_workspace_bytes(int M, int N, int split_k);
/* split_k <= 0: the library chooses (see above; with cfg == NULL the tile is chosen together
 * with its slice count).  The effective factor is clamped to [1, ceil(K/64)].
 * Slice s covers K elements [s*len, (s+1)*len), len = ceil(ceil(K/64)/split_k)*64; partial
 * sums are fp32 in ws[split][M][N]; they are added in slice order 0,1,2,... and rounded once, so results
 * are bit-identical from run to run.  One launch: the workgroups that add ride in the same grid behind
 * the ones that multiply and start on a tile as soon as its slices have signalled (they are placed after
 * every multiplying workgroup, so what they wait for always arrives; the wait is bounded all the same, by
 * beam_set_ln_spin_limit: a workgroup that gives up writes NaN, see beam_gemmrc_splitk_timed_out).  Two
 * launches (partial kernel, reduce kernel; the same bits) for tiles above 128 x 128, N not a multiple of
 * 4, more than 64 slices, M * N above 2^28, outputs so large that the adding workgroups would need more than
 * two rounds of the CUs, or a workspace that only holds the partial sums
 * (split_k * M * N * 4 bytes; anything smaller is BEAM_ERR_WORKSPACE).
 * Replaces entry_cutlass_gemmrc_splitk / _spec
 * (cuda/cutlass_kernels/main.cc:17-21, cutlass_gemmrc_splitk.cu:59-105,107-195). */
int beam_gemmrc_splitk(const void* A, const void* B, void* C, int M, int N, int K, int dtype,
                       const beam_tile_cfg* cfg, int split_k, void* ws, size_t ws_bytes,
                       void* stream);
/* Waits for `stream`; *timed_out = 1 if the latest split-K call on this workspace ran as one launch and one of its
 * reducing workgroups gave up waiting (its outputs are NaN).  ws_bytes, M, N: as given to that call;
 * split_k_effective: beam_splitk_effective of that call.  0 for a call that had no waiting workgroups (one slice,
 * two launches, a workspace that ends with the partial sums).  Does not happen on a working device; the bound
 * exists so that no kernel of the library can wait for ever. */
int beam_gemmrc_splitk_timed_out(const void* ws, size_t ws_bytes, int M, int N, int split_k_effective, void* stream,
                                 int* timed_out);
/* on != 0: beam_gemmrc_splitk always runs as two launches.  Off by default (environment:
 * BEAM_SPLITK_TWO_LAUNCHES=1).  Results are the same bits either way. */
int beam_set_splitk_two_launches(int on);
/* The effective split factor beam_gemmrc_splitk would use for these arguments. */
int beam_splitk_effective(int M, int N, int K, const beam_tile_cfg* cfg, int split_k);
/* verbose != 0: when the library chooses the slice count itself, beam_gemmrc_splitk writes one line to
 * stderr the first time it sees a (shape, dtype, tile): the tile, the slice count, the workgroups that
 * makes and how many rounds of the device's CUs they are.  Off by default; the environment variable
 * BEAM_VERBOSE=1 turns it on at load.  Stands in for the once-per-shape "[INFO] ... split_k(..), CTAs(..),
 * waves(..)" line of cuda/cutlass_kernels/cutlass_gemmrc_splitk.cu:12-24,87-93. */
int beam_set_verbose(int verbose);
/* beam_gemmrc_splitk without a workspace argument and without any allocation: the fp32 partial sums go
 * into device memory built into the library (a fixed array of beam_splitk_noalloc_max_bytes() = 16 MiB
 * for them, plus 256 KiB for the synchronisation words of the one-launch form, per GPU, present from the
 * first call into the library until the process ends).  No counterpart in
 * the reference; it is for callers that cannot allocate: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  Same results as beam_gemmrc_splitk, bit for bit.
 * split_k * M * N * 4 bytes beyond the array's size -> BEAM_ERR_WORKSPACE.  All calls on one GPU share
 * the array: calls that overlap in time on one GPU (different streams) race; order them. */
size_t beam_splitk_noalloc_max_bytes(void);
int beam_gemmrc_splitk_noalloc(const void* A, const void* B, void* C, int M, int N, int K, int dtype,
                               const beam_tile_cfg* cfg, int split_k, void* stream);

/* ---- fused GEMM + LayerNorm --------------------------------------------------------------- */

/* Y[m][:] = LayerNorm_N(A.B^T)[m][:] * gamma + beta, statistics (biased variance over N) and
 * normalisation computed from the fp32 accumulators, Y rounded once to the 16-bit dtype.
 * gamma, beta: 16-bit [N].  The reference has no LayerNorm (its
 * entry_cute_parallel_gemmrc_lnr, cuda/cute_kernels/main.cc:19-22 and cute_gemm_ln.cu:230-245,
 * is a GEMM plus an unrelated SiLU); this entry takes that slot in the interface. */
size_t beam_gemmrc_ln_workspace_bytes(int M, int N, const beam_tile_cfg* cfg);
int beam_gemmrc_ln(const void* A, const void* B, const void* gamma, const void* beta, float eps,
                   void* Y, int M, int N, int K, int dtype, const beam_tile_cfg* cfg, void* ws,
                   size_t ws_bytes, void* stream);

/* The two ways the library computes it, selectable for testing and tuning:
 *   BEAM_LN_FUSED   one kernel: each workgroup keeps its fp32 accumulators in registers, the column
 *                   tiles of a row band exchange per-row (mean, M2) pairs through the workspace (every
 *                   workgroup publishes its own and polls, boundedly, for the others'), then every
 *                   workgroup normalises and stores its own tile.  Needs all column tiles of a band
 *                   resident at once: N / block_n <= 64, a device of 256 CUs in 8 XCDs, and the device
 *                   not shared with other work while it runs (otherwise the wait runs into its bound, the
 *                   rows concerned come out as NaN and beam_gemmrc_ln_timed_out says so;
 *                   beam_gemmrc_ln_checked then repeats the call as two passes by itself).
 *   BEAM_LN_TWOPASS the GEMM kernel stores fp32 X and per-tile statistics, a second kernel normalises.
 *   BEAM_LN_AUTO    fused when it applies, else two-pass (what beam_gemmrc_ln does); two-pass under
 *                   stream capture. */
typedef enum beam_ln_mode { BEAM_LN_AUTO = 0, BEAM_LN_TWOPASS = 1, BEAM_LN_FUSED = 2 } beam_ln_mode;
/* Workspace bytes.  _for is enough for the call beam_gemmrc_ln_ex(M, N, K, cfg, mode) on operands aligned as the
 * tiled kernels need them (A, B, Y 16 bytes, gamma and beta 8): exact for BEAM_LN_TWOPASS and BEAM_LN_FUSED; for
 * BEAM_LN_AUTO the larger of the two forms it can resolve to (one kernel eagerly; two passes under stream capture
 * and as the retry of beam_gemmrc_ln_checked).  The forms without K are enough for any call with these M, N, cfg and
 * mode: every K (cfg == NULL: every tile the library could pick), operands aligned to an element only, captured or
 * not. */
size_t beam_gemmrc_ln_workspace_bytes_for(int M, int N, int K, const beam_tile_cfg* cfg, int mode);
size_t beam_gemmrc_ln_workspace_bytes_ex(int M, int N, const beam_tile_cfg* cfg, int mode);
int beam_gemmrc_ln_ex(const void* A, const void* B, const void* gamma, const void* beta, float eps,
                      void* Y, int M, int N, int K, int dtype, const beam_tile_cfg* cfg, int mode,
                      void* ws, size_t ws_bytes, void* stream);
/* beam_gemmrc_ln (BEAM_LN_AUTO) for callers that want the result whatever else runs on the device.  Synchronous:
 * after the call it waits for `stream`; if the one-kernel form gave up waiting for a band of workgroups (a device that
 * other work keeps occupied: beam_gemmrc_ln_timed_out), it runs the call again as two passes, which wait for
 * nothing, and waits for that.  *fell_back (may be NULL) = 1 then.  ws_bytes as for BEAM_LN_AUTO.  Under stream
 * capture it is beam_gemmrc_ln (two passes, nothing to check).  What the Python layer's gemmrc_ln calls by default. */
int beam_gemmrc_ln_checked(const void* A, const void* B, const void* gamma, const void* beta, float eps, void* Y,
                           int M, int N, int K, int dtype, const beam_tile_cfg* cfg, void* ws, size_t ws_bytes,
                           void* stream, int* fell_back);
/* The fused path's workspace needs no preparation and carries no state from call to call: every
 * fused launch has a tag that no earlier launch had, and a statistics word counts only if it carries
 * that tag (a stray word passes with probability 2^-32, and both words of a row have to).  So a fresh
 * buffer, one the allocator hands out again, one used for another shape or written over by somebody
 * else all work as they are, and the library keeps no host-side record of workspaces.  Launches that
 * share one workspace must be ordered on one stream.  This call only zeroes the header's record of the latest
 * launch and its time-out (synchronously; the replay counter of captured launches stays); nothing requires it. */
int beam_gemmrc_ln_workspace_reset(const void* ws);
/* Waits for `stream`, then *timed_out = 1 if the latest fused call on this workspace gave up
 * waiting for a band: the rows concerned are then NaN in Y.  Only possible if the device could not
 * hold a whole band of workgroups at once, e.g. because another process occupied most of it.  The
 * record names the launch it is about, so every fused call starts with a clean slate. */
int beam_gemmrc_ln_timed_out(const void* ws, void* stream, int* timed_out);
/* Bound of that wait: polls of statistics slots per thread (3-4 microseconds each once the pauses between
 * tries have grown; default 16384, about 60 ms: what a workgroup legitimately waits for is at most one tile's K loop
 * behind it).  0 makes every thread that finds a slot unpublished give up at once; -1 makes every wait give
 * up whatever it finds: the kernel still ends normally and the flag is set, which is how the failure
 * path is exercised without hanging anything.  The same number bounds the wait of the reducing workgroups
 * of the one-launch split-K (polls of a tile's flags). */
int beam_set_ln_spin_limit(int polls);
/* How the fused kernel of the 256 x 256 tile of four wavefronts covers a problem of more tiles than CUs.
 * on != 0 (the default; environment: BEAM_LN_WALK=0 turns it off): one workgroup per CU walks its tiles, the next
 * tile's first operands arriving while the band's statistics are exchanged.  Every workgroup of the launch must then
 * be resident at once: on a device that other work occupies in part, bands whose workgroups were not placed time
 * out (NaN rows, beam_gemmrc_ln_timed_out; beam_gemmrc_ln_checked repeats the call as two passes).  on = 0: one
 * workgroup per tile in band order, which finishes band by band on whatever part of the device it gets.  The two
 * forms give the same bits and measure within 2% of each other. */
int beam_set_ln_walk(int on);

/* ---- GEMM with an independent elementwise job hidden in its K loop ------------------------ */

/* C = A . B^T as beam_gemmrc and, in the same launch, Y[i] = silu(X[i]) = X[i] / (1 + exp(-X[i]))
 * for i in [0, count): 16-bit in, fp32 arithmetic, round-to-nearest 16-bit out.  The array is cut into
 * units of 4, 8 or 16 bytes (the narrowest with which the job still ends inside the K loop), dealt out in
 * contiguous runs over the GEMM's workgroups and carried, a few units per K tile, by the wavefronts that
 * issue the operand loads, so the elementwise traffic rides in the memory-side slack of the
 * matrix-core-bound loop.  Replaces
 * entry_cute_parallel_gemmrc_lnr (cuda/cute_kernels/cute_gemm_ln.cu:230-245, kernel :24-228, bound
 * as cutlass_parallel_gemmrc_lnr in cuda/cute_kernels/main.cc), whose lnA/lnB are X/Y here and whose
 * lnM*lnN is `count`.  Unlike the reference, which gives the job to a quarter of the workgroups and
 * drops whatever does not fit their K loops, every element is processed exactly once for any
 * count and any GEMM shape.  X, Y: device pointers, 16-byte aligned, count <= 1 073 741 696;
 * Y may be X (in place) but must not overlap it otherwise; neither may overlap C.
 * cfg->pipeline must be 0 or 1. */
int beam_parallel_gemmrc_silu(const void* A, const void* B, void* C, int M, int N, int K, const void* X,
                              void* Y, long long count, int dtype, const beam_tile_cfg* cfg, void* stream);

/* The elementwise job alone (one streaming kernel): the baseline beam_parallel_gemmrc_silu is
 * measured against, and what it falls back on when the GEMM is empty (M, N or K = 0).  The
 * reference has no separate entry for it (the formula is cuda/cute_kernels/cute_gemm_ln.cu:191-192). */
int beam_silu(const void* X, void* Y, long long count, int dtype, void* stream);

/* ---- B stored [K][N] ----------------------------------------------------------------------- */

/* C[M][N] = A[M][K] . B[K][N], all row-major: the layout of the reference's Triton matmul(a, b)
 * (python/beam/triton_kernels/gemm.py:78-99, kernel :10-76), which torch.matmul callers use.  Same
 * arithmetic as beam_gemmrc (fp32 accumulation, one rounding to 16 bits); same tile space.  B tiles
 * are staged in LDS as they lie in memory and transposed on their way into registers
 * (ds_read_b64_tr_b16), so no transposed copy of B is made.  N % 8 != 0 (rows of B that are not multiples of
 * 16 bytes) runs on the plain kernel, like K % 8 != 0.  With cfg NULL the library starts from the tile it would
 * take for beam_gemmrc and prefers wavefront tiles of 32 columns to those of 64 (a B fragment is two LDS reads
 * in this layout). */
int beam_matmul_nn(const void* A, const void* B, void* C, int M, int N, int K, int dtype, const beam_tile_cfg* cfg,
                   void* stream);

/* ---- timing ------------------------------------------------------------------------------- */

/* Which operation beam_bench times. */
typedef enum beam_op {
  BEAM_OP_GEMM = 0,
  BEAM_OP_SPLITK = 1,
  BEAM_OP_GEMM_LN = 2,
  BEAM_OP_GEMM_SILU = 3, /* beam_parallel_gemmrc_silu */
  BEAM_OP_SILU = 4,      /* beam_silu alone            */
  BEAM_OP_MATMUL_NN = 5  /* beam_matmul_nn             */
} beam_op;

typedef struct beam_problem {
  const void* A;
  const void* B;
  void* C;            /* C or Y                                                     */
  const void* gamma;  /* BEAM_OP_GEMM_LN only                                       */
  const void* beta;
  float eps;
  int M, N, K, dtype;
  int split_k;        /* BEAM_OP_SPLITK                                             */
  void* ws;
  size_t ws_bytes;
  const void* side_x;   /* BEAM_OP_GEMM_SILU, BEAM_OP_SILU                            */
  void* side_y;
  long long side_count;
  int ln_mode;          /* BEAM_OP_GEMM_LN: a beam_ln_mode (0 = BEAM_LN_AUTO)          */
} beam_problem;

/* `warmup` untimed calls, then `iters` back-to-back calls bracketed by HIP events on `stream`;
 * *avg_ms = elapsed / iters.  Replaces test_pipeline (cuda/cublas.cc:12-40) and
 * triton.testing.do_bench as used by python/beam/tuner.py:33-44. */
int beam_bench(int op, const beam_problem* prob, const beam_tile_cfg* cfg, int warmup, int iters,
               void* stream, float* avg_ms);

/* Events for hosts that time their own call sequences (what triton.testing.do_bench gives the
 * reference's tuner, python/beam/tuner.py:38-39).  elapsed waits for `stop` to complete. */
int beam_event_create(void** event);
int beam_event_record(void* event, void* stream);
int beam_event_elapsed_ms(void* start, void* stop, float* ms);
int beam_event_destroy(void* event);

/* ---- streams and graphs (so that hosts need no other GPU runtime) -------------------------- */

/* Every operator above is one to three kernel launches on the caller's stream and neither allocates nor
 * synchronises, so a sequence of them can be captured once and replayed as a HIP graph: the usual cure
 * for launch-bound loops of small GEMMs (a split-K call is one launch of 13 us).  The reference
 * has no counterpart (it launches on the legacy default stream, cuda/cute_kernels/cute_gemm_128x128.cu:
 * 203).  Rules: call every operator once eagerly before capturing it (the first launch of a kernel
 * configures its LDS size); BEAM_LN_AUTO takes the two-pass path under capture (BEAM_LN_FUSED is honoured:
 * a one-thread kernel recorded in front of it makes every replay's tag new); K = 0 clears C with a kernel, not a
 * memset node.  Streams are created at the default priority. */
int beam_stream_create(void** stream);
int beam_stream_destroy(void* stream);
int beam_graph_begin_capture(void* stream);               /* not the default stream */
int beam_graph_end_capture(void* stream, void** graph_exec);
int beam_graph_launch(void* graph_exec, void* stream);
int beam_graph_destroy(void* graph_exec);

/* ---- device memory (so that hosts need no other GPU runtime) ------------------------------ */

int beam_malloc(void** dptr, size_t bytes);
int beam_free(void* dptr);
int beam_memcpy_h2d(void* dst, const void* src_host, size_t bytes);
int beam_memcpy_d2h(void* dst_host, const void* src, size_t bytes);
int beam_memcpy_d2d(void* dst, const void* src, size_t bytes);
int beam_memset(void* dptr, int byte, size_t bytes);
int beam_sync(void* stream);

/* ---- synthetic data (host) ----------------------------------------------------------------- */

/* Counter-based generator: element i of tensor `tensor_id` under `seed` depends on nothing
 * else, so any number of threads produce the same bits.  dst_host: 16-bit [n].
 *   uniform: value in [-1, 1) with 24 random bits, rounded RN to the dtype
 *   normal : mean + scale * N(0,1) (Box-Muller in double), rounded RN to the dtype
 * The reference draws unseeded torch.randn on the GPU (python/gemm_test.py:81). */
int beam_host_fill_uniform(void* dst_host, size_t n, int dtype, uint64_t seed, uint64_t tensor_id);
int beam_host_fill_normal(void* dst_host, size_t n, int dtype, uint64_t seed, uint64_t tensor_id,
                          float mean, float scale);

#ifdef __cplusplus
}
#endif
#endif /* BEAM_HIP_H */
