// gemmrc kernels for workgroup tile 128x256, wavefront tile 64x64 (all dtypes, epilogues, loaders).
#include "kernel_set.h"

namespace beam {
BEAM_DEFINE_SET(128, 256, 64, 64)
}  // namespace beam
