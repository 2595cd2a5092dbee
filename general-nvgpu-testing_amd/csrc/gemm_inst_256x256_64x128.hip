// gemmrc kernels for workgroup tile 256x256, wavefront tile 64x128 (all dtypes, epilogues, loaders).
#include "kernel_set.h"

namespace beam {
BEAM_DEFINE_SET(256, 256, 64, 128)
}  // namespace beam
