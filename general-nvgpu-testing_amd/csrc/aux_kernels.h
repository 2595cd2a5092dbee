// Launchers of the split-K reduction, the LayerNorm normalisation pass and the streaming SiLU.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>

#include "../../include/beam_hip.h"

namespace beam {

// C[mn] (16-bit) = sum over `splits` fp32 slices of ws[splits][mn], added in slice order.
// sync_header, if not null: the synchronisation words of a split-K workspace; their "latest launch" word is cleared.
hipError_t launch_splitk_reduce(const float* ws, void* C, size_t mn, int splits, int dtype, int* sync_header,
                                hipStream_t stream);

// Y[M][N] (16-bit) = normalise fp32 X[M][N] with per-(row, column tile) (mean, M2) pairs.
hipError_t launch_ln_apply(const float* X, const float* stats, const void* gamma, const void* beta,
                           void* Y, int M, int N, int tiles_n, int block_n, float eps, int dtype,
                           hipStream_t stream);

// One thread moves on the replay counter in the header of a fused GEMM+LayerNorm workspace: recorded in front
// of a fused launch when the stream is being captured (see ln_launch_tag in gemm_kernel.h).
hipError_t launch_ln_replay_bump(int* header, hipStream_t stream);

// gemmrc without any condition on K, N or alignment (slow; what the tiled kernels refuse runs here):
// C[M][N] = A[M][K] . B^T with B as [N][K], or as [K][N] when b_kmajor; C 16-bit, or fp32 when out_fp32.
// Grid dimension y = ceil(M / 64) must stay below 65536.
hipError_t launch_generic_gemm(const void* A, const void* B, void* C, int M, int N, int K, int dtype, bool b_kmajor,
                               bool out_fp32, hipStream_t stream);
// Y[m][:] (16-bit) = LayerNorm of the fp32 row X[m][:], statistics computed here (generic path).
hipError_t launch_ln_rows(const float* X, const void* gamma, const void* beta, void* Y, int M, int N, float eps, int dtype,
                          hipStream_t stream);

// y[i] (16-bit) = silu(x[i]) for i in [0, count); x and y 16-byte aligned.
hipError_t launch_silu(const void* x, void* y, size_t count, int dtype, hipStream_t stream);

// 16-bit p[0 .. n) = 0: what an operator with K = 0 writes (a kernel, so that the call can be captured in a graph)
hipError_t launch_zero_u16(void* p, size_t n, hipStream_t stream);
// ints[0 .. n) = 0 (a fill kernel rather than hipMemsetAsync, so that callers may capture it in a graph).
hipError_t launch_zero_ints(int* ints, int n, hipStream_t stream);
// A kernel that does nothing, `workgroups` x `threads`: what a launch costs from submission to completion.
hipError_t launch_empty(int workgroups, int threads, hipStream_t stream);
// floats[0 .. n) = value
hipError_t launch_fill_floats(float* floats, size_t n, float value, hipStream_t stream);

}  // namespace beam
