// Instantiates the LIF fire kernels of lif_kernels.h for float storage
// (fp32 arithmetic).  One translation unit per storage type keeps the build parallel.
#include "lif_kernels.h"

namespace snnlif {
SNNLIF_DEFINE_DTYPE(f32, float)
}  // namespace snnlif
