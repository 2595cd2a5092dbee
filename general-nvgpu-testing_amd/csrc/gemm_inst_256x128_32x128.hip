// gemmrc kernels for workgroup tile 256x128, wavefront tile 32x128 (all dtypes, epilogues, loaders).
#include "kernel_set.h"

namespace beam {
BEAM_DEFINE_SET(256, 128, 32, 128)
}  // namespace beam
