// The 256x256 tile of four 128x128 wavefronts (gemm_w4.h), fp16 and bf16.
#include "gemm_w4.h"
#include "kernel_set.h"

namespace beam {

template <typename T, bool C_NT, bool LN = false>
static hipError_t launch_w4_t(const GemmParams& p, dim3 grid, hipStream_t stream) {
  auto kern = gemmrc_w4_kernel<T, C_NT, LN>;
  static std::atomic<unsigned long long> configured{0};
  if (hipError_t e = allow_lds_once(configured, reinterpret_cast<const void*>(kern), GemmW4<T>::LDS_BYTES); e != hipSuccess) return e;
  hipLaunchKernelGGL(kern, grid, dim3(GemmW4<T>::NT), GemmW4<T>::LDS_BYTES, stream, p);
  return hipGetLastError();
}

hipError_t launch_gemm_w4(const GemmParams& p, int dtype, dim3 grid, hipStream_t stream) {
  if (p.c_streaming) return dtype == BEAM_BF16 ? launch_w4_t<__bf16, true>(p, grid, stream) : launch_w4_t<_Float16, true>(p, grid, stream);
  return dtype == BEAM_BF16 ? launch_w4_t<__bf16, false>(p, grid, stream) : launch_w4_t<_Float16, false>(p, grid, stream);
}

static_assert(kW4LnCompactTiles == GemmW4<_Float16, false, true>::kLnCompactTiles, "the host's bound is the kernel's");

hipError_t launch_gemm_w4_ln(const GemmParams& p, int dtype, dim3 grid, hipStream_t stream) {
  return dtype == BEAM_BF16 ? launch_w4_t<__bf16, false, true>(p, grid, stream) : launch_w4_t<_Float16, false, true>(p, grid, stream);
}

}  // namespace beam
