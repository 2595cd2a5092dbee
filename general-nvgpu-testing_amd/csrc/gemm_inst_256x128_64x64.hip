// gemmrc kernels for workgroup tile 256x128, wavefront tile 64x64 (all dtypes, epilogues, loaders).
#include "kernel_set.h"

namespace beam {
BEAM_DEFINE_SET(256, 128, 64, 64)
}  // namespace beam
