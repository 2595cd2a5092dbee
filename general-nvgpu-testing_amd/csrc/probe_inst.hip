// Measurement kernels that are not operators: see kEpiProbeLoads in gemm_kernel.h and BEAM_OP_PROBE_* in the C ABI.
#include "kernel_set.h"

namespace beam {

hipError_t launch_probe_splitk_loads(const GemmParams& p, int block_m, int block_n, dim3 grid, hipStream_t stream) {
  if (block_m == 64 && block_n == 128) {
    constexpr int DA = deep_a_slots(64, 128);
    return launch_gemm<_Float16, 64, 128, 2, 2, kEpiProbeLoads, DA, DA - 1>(p, grid, stream);
  }
  if (block_m == 64 && block_n == 64) {
    constexpr int DA = deep_a_slots(64, 64);
    return launch_gemm<_Float16, 64, 64, 2, 2, kEpiProbeLoads, DA, DA - 1>(p, grid, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace beam
