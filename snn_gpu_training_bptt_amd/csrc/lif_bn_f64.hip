// Batch-norm + fire kernels for double storage and arithmetic; see lif_bn_launch.h.
#include "lif_bn_launch.h"

SNNLIF_DEFINE_BN_DTYPE(f64, double)
