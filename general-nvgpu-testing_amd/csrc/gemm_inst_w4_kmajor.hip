// The 256x256 tile of four 128x128 wavefronts (gemm_w4.h) with B stored [K][N], fp16 and bf16.
#include "gemm_w4.h"
#include "kernel_set.h"

namespace beam {

template <typename T, bool C_NT>
static hipError_t launch_w4_kmajor_t(const GemmParams& p, dim3 grid, hipStream_t stream) {
  using Tile = GemmW4<T, C_NT, false, 4, 8, 2, true>;
  auto kern = gemmrc_w4_kernel<T, C_NT, false, 4, 8, 2, true>;
  static bool configured = false;  // benign race: the attribute call is idempotent
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       Tile::LDS_BYTES);
    if (e != hipSuccess) return e;
    configured = true;
  }
  hipLaunchKernelGGL(kern, grid, dim3(Tile::NT), Tile::LDS_BYTES, stream, p);
  return hipGetLastError();
}

hipError_t launch_gemm_w4_kmajor(const GemmParams& p, int dtype, dim3 grid, hipStream_t stream) {
  if (p.c_streaming)
    return dtype == BEAM_BF16 ? launch_w4_kmajor_t<__bf16, true>(p, grid, stream) : launch_w4_kmajor_t<_Float16, true>(p, grid, stream);
  return dtype == BEAM_BF16 ? launch_w4_kmajor_t<__bf16, false>(p, grid, stream) : launch_w4_kmajor_t<_Float16, false>(p, grid, stream);
}

}  // namespace beam
