// gemmrc kernels for workgroup tile 224x256, wavefront tile 112x64 (all dtypes, epilogues, loaders).
#include "kernel_set.h"

namespace beam {
BEAM_DEFINE_SET(224, 256, 112, 64)
}  // namespace beam
