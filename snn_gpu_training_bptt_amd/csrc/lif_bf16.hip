// Instantiates the LIF fire kernels of lif_kernels.h for bf16_t storage
// (fp32 arithmetic).  One translation unit per storage type keeps the build parallel.
#include "lif_kernels.h"

namespace snnlif {
SNNLIF_DEFINE_DTYPE(bf16, bf16_t)
}  // namespace snnlif
