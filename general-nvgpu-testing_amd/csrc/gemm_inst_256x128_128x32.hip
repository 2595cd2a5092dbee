// gemmrc kernels for workgroup tile 256x128, wavefront tile 128x32 (all dtypes, epilogues, loaders).
#include "kernel_set.h"

namespace beam {
BEAM_DEFINE_SET(256, 128, 128, 32)
}  // namespace beam
