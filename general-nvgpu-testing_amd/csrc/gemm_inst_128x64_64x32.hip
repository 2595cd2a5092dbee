// gemmrc kernels for workgroup tile 128x64, wavefront tile 64x32 (all dtypes, epilogues, loaders).
#include "kernel_set.h"

namespace beam {
BEAM_DEFINE_SET(128, 64, 64, 32)
}  // namespace beam
