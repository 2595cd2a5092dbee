/*
 * beam_hip_debug.h -- test and measurement surface of libbeam_hip.so.
 *
 * Nothing here stands in for an interface of the reference, and nothing a caller of the operators needs:
 * the index maps the kernels use, exported so that host tests can check them by brute force, and launches
 * that are not operators but measure what the machine allows (the floors and ceilings the operators'
 * timings are read against).  The operators themselves are in beam_hip.h.
 */
#ifndef BEAM_HIP_DEBUG_H
#define BEAM_HIP_DEBUG_H

#include "beam_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- measurement launches ------------------------------------------------------------------- */

/* Further values of the `op` argument of beam_bench: launches that are not operators. */
typedef enum beam_probe_op {
  BEAM_OP_PROBE_EMPTY = 6,        /* one empty kernel of 256 workgroups x 256 threads                */
  BEAM_OP_PROBE_EMPTY_PAIR = 7,   /* two empty kernels in a row (256 x 256, then 1024 x 64 threads)   */
  BEAM_OP_PROBE_SPLITK_LOADS = 8, /* the partial kernel of BEAM_OP_SPLITK for the same arguments with its
                                     loads and LDS reads but no MFMAs and no stores, and no reduction;
                                     fp16, tiles 64x128 (wave 32x64) and 64x64 (wave 32x32), pipeline 2 */
  BEAM_OP_PROBE_LN_APPLY = 9      /* the normalisation pass of a two-pass BEAM_OP_GEMM_LN alone, on the fp32
                                     X and statistics that such a call (same arguments) left in the workspace:
                                     reads 4 M N bytes, writes 2 M N                                          */
} beam_probe_op;

/* What the matrix cores sustain with no memory instruction at all: one workgroup of four wavefronts per
 * CU (one wavefront per SIMD, the occupancy of the large-problem kernel), every wavefront issuing `passes`
 * times 1024 matrix-core cycles of independent MFMAs on operands that sit in registers (accumulators in
 * the accumulation registers), consecutive MFMAs sharing one operand as in the kernels.
 *   mfma_shape  BEAM_MFMA_16X16X32 (64 MFMAs of 16 cycles per pass, what the kernels use) or
 *               BEAM_MFMA_32X32X16 (32 MFMAs of 32 cycles per pass)
 *   data        BEAM_PROBE_DATA_NORMAL: operands N(0,1)/sqrt(8192) drawn into registers once (the
 *               distribution of the headline workload); BEAM_PROBE_DATA_ZEROS: all-zero operands.
 * On a power-limited part the two differ by the clock the power cap allows.  `warmup` untimed launches,
 * then `iters` timed ones bracketed by HIP events on `stream`; *avg_ms per launch, *flop_per_launch =
 * CUs x 4 x passes x 1024 cycles x 1024 flop per cycle.  The peak constants of the reference's roofline
 * script (python/scripts/gemm_flops.py:26-32) are vendor figures; this measures the counterpart. */
enum { BEAM_MFMA_16X16X32 = 0, BEAM_MFMA_32X32X16 = 1 };
enum { BEAM_PROBE_DATA_NORMAL = 0, BEAM_PROBE_DATA_ZEROS = 1 };
int beam_probe_mfma(int dtype, int mfma_shape, int data, int passes, int warmup, int iters, void* stream,
                    float* avg_ms, double* flop_per_launch);

/* ---- index maps, exported for host-side verification ---------------------------------------- */

/* Workgroup id -> (tile_m, tile_n) as the kernels compute it (divisions done as multiplications by constants the
 * host prepares), and the same map written with plain divisions, which defines it. */
int beam_dbg_tile_of_workgroup(int wg, int tiles_m, int tiles_n, int group_m, int* tm, int* tn);
int beam_dbg_tile_of_workgroup_by_division(int wg, int tiles_m, int tiles_n, int group_m, int* tm, int* tn);
/* n / d (n < 2^31, d >= 1) through the multiplier the host would prepare for d. */
unsigned beam_dbg_fast_div(unsigned n, unsigned d);
/* Byte offset of (row, 16-byte chunk) inside an LDS stage. */
int beam_dbg_lds_offset(int row, int chunk);
/* Byte offset of element (k, n), n a multiple of 4, inside a K-major LDS stage of block_n columns
 * (B stored [K][N], beam_matmul_nn). */
int beam_dbg_kmajor_lds_offset(int k, int n, int block_n);
/* Workspace bytes beam_gemmrc_ln_ex(M, N, K, cfg, mode) insists on, by the path the call takes: `plain` (operands
 * aligned to an element only; K % 8 != 0 implies it), `capturing` (the stream is being captured), `wide_io` (Y, gamma
 * and beta 16-byte aligned).  The entry point computes its requirement with the same function; the workspace queries
 * are tested against it.  0 on error. */
size_t beam_dbg_ln_plan_bytes(int M, int N, int K, const beam_tile_cfg* cfg, int mode, int plain, int capturing, int wide_io);
/* A measurement, off by default: on != 0 makes the one-launch split-K run without reducing workgroups wherever its
 * multiplying workgroups fit one round of the CUs; the workgroup of (tile, slice s) then adds parts s, s + slices, ...
 * of its tile itself.  Same bits.  Unlike the shipped form this needs every workgroup of the launch resident at once
 * (the wait is bounded all the same). */
int beam_dbg_set_splitk_self_reduce(int on);
/* For tests on a host without a GPU: the CU count the library's choices assume when no device could be probed
 * (refused once a device has been). */
int beam_dbg_assume_compute_units(int compute_units);
/* The tile a beam_gemmrc_ln call without a tile takes for its one-kernel form on a device of `compute_units` CUs
 * (the library's LayerNorm cost model; BEAM_ERR_UNSUPPORTED where that form applies with no tile). */
int beam_dbg_ln_default_config(int M, int N, int K, int compute_units, beam_tile_cfg* cfg);
/* The 4-wavefront kernel with B stored [K][N] (256 columns, 512 bytes per row of k in an LDS slot): the XOR code of
 * the 16-byte chunks of row k, and the byte offset of the 8 bytes that lane 16 g + 4 e + q supplies to the first
 * transposing read of 16-column block b (0..7) of the wavefront's column half wn (0, 1). */
int beam_dbg_w4_kmajor_swizzle(int k);
int beam_dbg_w4_kmajor_read_offset(int wn, int b, int g, int e, int q);
/* Workgroup id -> tile of the padded band-block grid used by the fused GEMM+LayerNorm (tm = -1:
 * the id is padding), and the size of that grid. */
int beam_dbg_band_block_tile(int wg, int tiles_m, int tiles_n, int gb, int gc, int* tm, int* tn);
int beam_dbg_band_block_grid(int tiles_m, int gb, int gc);
/* The three orders as the kernels compute them, divisions done by multiplication: group_n > 0 is the band-block
 * order with gb = group_m and gc = group_n, group_n == 0 the whole-bands order with bx = group_m, group_n < 0 plain
 * band after band (id = band * tiles_n + column). */
int beam_dbg_band_order_tile(int id, int tiles_m, int tiles_n, int group_m, int group_n, int* tm, int* tn);
/* The same for the order that keeps whole bands (bx at a time) on one XCD, used when a band is
 * short enough for it. */
int beam_dbg_band_xcd_tile(int wg, int tiles_m, int tiles_n, int bx, int* tm, int* tn);
int beam_dbg_band_xcd_grid(int tiles_m, int tiles_n, int bx);

#ifdef __cplusplus
}
#endif
#endif /* BEAM_HIP_DEBUG_H */
