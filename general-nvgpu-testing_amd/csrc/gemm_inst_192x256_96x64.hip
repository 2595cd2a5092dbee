// gemmrc kernels for workgroup tile 192x256, wavefront tile 96x64 (all dtypes, epilogues, loaders).
#include "kernel_set.h"

namespace beam {
BEAM_DEFINE_SET(192, 256, 96, 64)
}  // namespace beam
