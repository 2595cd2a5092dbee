// gemmrc kernels for workgroup tile 64x128, wavefront tile 32x64 (all dtypes, epilogues, loaders).
#include "kernel_set.h"

namespace beam {
BEAM_DEFINE_SET(64, 128, 32, 64)
}  // namespace beam
