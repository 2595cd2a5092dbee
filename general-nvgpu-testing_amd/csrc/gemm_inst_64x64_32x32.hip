// gemmrc kernels for workgroup tile 64x64, wavefront tile 32x32 (all dtypes, epilogues, loaders).
#include "kernel_set.h"

namespace beam {
BEAM_DEFINE_SET(64, 64, 32, 32)
}  // namespace beam
