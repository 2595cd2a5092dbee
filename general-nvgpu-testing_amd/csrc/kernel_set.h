// Table of compiled gemmrc kernels: one KernelSet per (workgroup tile, wavefront tile),
// holding a launcher for every (dtype, epilogue, pipeline depth) combination.
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>

#include "../../include/beam_hip.h"
#include "gemm_kernel.h"

namespace beam {

typedef hipError_t (*GemmLauncher)(const GemmParams& p, dim3 grid, hipStream_t stream);

struct KernelSet {
  int block_m, block_n, wave_m, wave_n;
  int threads;
  int lds_bytes;
  int lds_bytes_shallow;
  int lds_bytes_deep;
  // [dtype][epilogue][pipeline: 0 = 3 A + 2 B slots, 1 = 2 + 2, 2 = deep (store / partial only)]
  GemmLauncher launch[2][kNumEpilogues][3];
  // B stored [K][N] instead of [N][K], kEpiStore only: [dtype][pipeline]
  GemmLauncher launch_kmajor[2][3];
  // Split-K in one launch (kEpiPartialFused), tiles up to 128 x 128 only (what split-K problems run on):
  // [dtype][pipeline]; nullptr otherwise.
  GemmLauncher launch_partial_fused[2][3];
};

// Raises a kernel's dynamic LDS limit on the current device the first time the kernel is launched there: the
// attribute is a property of (kernel, device), so `done` keeps one bit per device index.  (A race between two
// first launches is benign: the call is idempotent.)
inline hipError_t allow_lds_once(std::atomic<unsigned long long>& done, const void* kern, int lds_bytes) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const unsigned long long bit = 1ull << (dev & 63);
  if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
  e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
  if (e != hipSuccess) return e;
  done.fetch_or(bit, std::memory_order_release);
  return hipSuccess;
}

template <typename T, int BM, int BN, int WVM, int WVN, int EPI, int AST, int BST, bool B_KMAJOR = false>
hipError_t launch_gemm(const GemmParams& p, dim3 grid, hipStream_t stream) {
  using Tile = GemmTile<T, BM, BN, WVM, WVN, EPI, AST, BST, B_KMAJOR>;
  auto kern = gemmrc_kernel<T, BM, BN, WVM, WVN, EPI, AST, BST, B_KMAJOR>;
  static std::atomic<unsigned long long> configured{0};
  if (hipError_t e = allow_lds_once(configured, reinterpret_cast<const void*>(kern), Tile::LDS_BYTES); e != hipSuccess) return e;
  hipLaunchKernelGGL(kern, grid, dim3(Tile::NT), Tile::LDS_BYTES, stream, p);
  return hipGetLastError();
}

// The looping store kernel exists for the large 8-wavefront tiles, the ones problems of several
// rounds of workgroups run with (3 A + 2 B slots only).
template <typename T, int BM, int BN, int WVM, int WVN>
GemmLauncher loop_launcher() {
  if constexpr (WVM * WVN == 8 && BM >= 192 && BN == 256 && BN / WVN == 64)
    return launch_gemm<T, BM, BN, WVM, WVN, kEpiStoreLoop, 3, 2>;
  else
    return nullptr;
}

template <typename T, int BM, int BN, int WVM, int WVN, int AST, int BST>
GemmLauncher partial_fused_launcher() {
  if constexpr (BM * BN <= 128 * 128) return launch_gemm<T, BM, BN, WVM, WVN, kEpiPartialFused, AST, BST>;
  else return nullptr;
}

template <int BM, int BN, int TM, int TN>
KernelSet make_kernel_set() {
  constexpr int WVM = BM / TM, WVN = BN / TN;
  KernelSet k;
  k.block_m = BM;
  k.block_n = BN;
  k.wave_m = TM;
  k.wave_n = TN;
  k.threads = WVM * WVN * 64;
  k.lds_bytes = GemmTile<_Float16, BM, BN, WVM, WVN, kEpiStore, 3, 2>::LDS_BYTES;
  k.lds_bytes_shallow = GemmTile<_Float16, BM, BN, WVM, WVN, kEpiStore, 2, 2>::LDS_BYTES;
  constexpr int DA = deep_a_slots(BM, BN);
  k.lds_bytes_deep = GemmTile<_Float16, BM, BN, WVM, WVN, kEpiStore, DA, DA - 1>::LDS_BYTES;
#define BEAM_FILL(D, T)                                                             \
  k.launch[D][kEpiStore][0] = launch_gemm<T, BM, BN, WVM, WVN, kEpiStore, 3, 2>;     \
  k.launch[D][kEpiStore][1] = launch_gemm<T, BM, BN, WVM, WVN, kEpiStore, 2, 2>;     \
  k.launch[D][kEpiStore][2] = launch_gemm<T, BM, BN, WVM, WVN, kEpiStore, DA, DA - 1>; \
  k.launch[D][kEpiPartial][0] = launch_gemm<T, BM, BN, WVM, WVN, kEpiPartial, 3, 2>; \
  k.launch[D][kEpiPartial][1] = launch_gemm<T, BM, BN, WVM, WVN, kEpiPartial, 2, 2>; \
  k.launch[D][kEpiPartial][2] = launch_gemm<T, BM, BN, WVM, WVN, kEpiPartial, DA, DA - 1>; \
  k.launch[D][kEpiLnStats][2] = nullptr;                                               \
  k.launch[D][kEpiLnFused][2] = nullptr;                                               \
  k.launch[D][kEpiLnStats][0] = launch_gemm<T, BM, BN, WVM, WVN, kEpiLnStats, 3, 2>; \
  k.launch[D][kEpiLnStats][1] = launch_gemm<T, BM, BN, WVM, WVN, kEpiLnStats, 2, 2>; \
  k.launch[D][kEpiLnFused][0] = launch_gemm<T, BM, BN, WVM, WVN, kEpiLnFused, 3, 2>; \
  k.launch[D][kEpiLnFused][1] = launch_gemm<T, BM, BN, WVM, WVN, kEpiLnFused, 2, 2>; \
  k.launch[D][kEpiStoreSide][0] = launch_gemm<T, BM, BN, WVM, WVN, kEpiStoreSide, 3, 2>; \
  k.launch[D][kEpiStoreSide][1] = launch_gemm<T, BM, BN, WVM, WVN, kEpiStoreSide, 2, 2>; \
  k.launch[D][kEpiStoreSide][2] = nullptr; \
  k.launch_kmajor[D][0] = launch_gemm<T, BM, BN, WVM, WVN, kEpiStore, 3, 2, true>; \
  k.launch_kmajor[D][1] = launch_gemm<T, BM, BN, WVM, WVN, kEpiStore, 2, 2, true>; \
  k.launch_kmajor[D][2] = launch_gemm<T, BM, BN, WVM, WVN, kEpiStore, DA, DA - 1, true>; \
  k.launch[D][kEpiStoreLoop][0] = loop_launcher<T, BM, BN, WVM, WVN>();              \
  k.launch[D][kEpiStoreLoop][1] = nullptr;                                            \
  k.launch[D][kEpiStoreLoop][2] = nullptr;                                            \
  k.launch_partial_fused[D][0] = partial_fused_launcher<T, BM, BN, WVM, WVN, 3, 2>();  \
  k.launch_partial_fused[D][1] = partial_fused_launcher<T, BM, BN, WVM, WVN, 2, 2>();  \
  k.launch_partial_fused[D][2] = partial_fused_launcher<T, BM, BN, WVM, WVN, DA, DA - 1>();
  BEAM_FILL(0, _Float16)
  BEAM_FILL(1, __bf16)
#undef BEAM_FILL
  return k;
}

// One definition per instantiation file (gemm_inst_*.hip).
#define BEAM_DECLARE_SET(BM, BN, TM, TN) KernelSet kernel_set_##BM##x##BN##_##TM##x##TN();
#define BEAM_DEFINE_SET(BM, BN, TM, TN) \
  KernelSet kernel_set_##BM##x##BN##_##TM##x##TN() { return make_kernel_set<BM, BN, TM, TN>(); }

// (workgroup tile M, N, wavefront tile M, N)
#define BEAM_FOR_EACH_SET(X) \
  X(256, 256, 128, 64)       \
  X(256, 256, 64, 128)       \
  X(256, 256, 128, 128)      \
  X(224, 256, 112, 64)       \
  X(192, 256, 96, 64)        \
  X(256, 128, 64, 64)        \
  X(256, 128, 128, 32)       \
  X(256, 128, 32, 128)       \
  X(256, 128, 128, 64)       \
  X(128, 256, 64, 64)        \
  X(128, 256, 64, 128)       \
  X(128, 128, 64, 64)        \
  X(128, 128, 64, 32)        \
  X(128, 64, 64, 32)         \
  X(64, 128, 32, 64)         \
  X(64, 64, 32, 32)

BEAM_FOR_EACH_SET(BEAM_DECLARE_SET)

// The large-problem kernel of gemm_w4.h (256 x 256 tile, four wavefronts of 128 x 128, one workgroup per
// CU walking its tiles).  Needs K % 64 == 0, K >= 192, N % 8 == 0, C 16-byte aligned and
// grid <= tiles_m * tiles_n; kW4MinK names the K bound.
constexpr int kW4MinK = 192;
hipError_t launch_gemm_w4(const GemmParams& p, int dtype, dim3 grid, hipStream_t stream);
// The same with B stored [K][N]; additionally K * N * 2 < 2^31.
hipError_t launch_gemm_w4_kmajor(const GemmParams& p, int dtype, dim3 grid, hipStream_t stream);
// Its fused GEMM+LayerNorm form: parameters as for the kEpiLnFused kernels plus ln_ids, the number of ids of the band
// order (padding included); a grid of ln_ids workgroups gives every workgroup one tile, a smaller grid (one
// workgroup per CU) makes them walk, which needs tiles_n <= kW4LnCompactTiles.  gamma and beta 16-byte aligned as well.
constexpr int kW4LnCompactTiles = 32;
hipError_t launch_gemm_w4_ln(const GemmParams& p, int dtype, dim3 grid, hipStream_t stream);
// Measurement only: the split-K partial kernel of the 64 x 128 (wave 32 x 64) or 64 x 64 (wave 32 x 32) tile, deep
// pipeline, fp16, with its loads and fragment reads but no MFMAs and no stores (kEpiProbeLoads); hipErrorInvalidValue
// for any other tile.
hipError_t launch_probe_splitk_loads(const GemmParams& p, int block_m, int block_n, dim3 grid, hipStream_t stream);
// Measurement only: `workgroups` (<= 1024) x 4 wavefronts, each issuing passes x 1024 matrix-core cycles of MFMAs on
// operands in registers (mfma_shape 0: 16x16x32, 1: 32x32x16; zeros: all-zero operands instead of N(0,1)/sqrt(8192)).
hipError_t launch_probe_mfma(int dtype, int mfma_shape, int workgroups, int passes, int zeros, hipStream_t stream);

}  // namespace beam
