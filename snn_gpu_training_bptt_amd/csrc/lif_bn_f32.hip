// Batch-norm + fire kernels for float storage and arithmetic; see lif_bn_launch.h.
#include "lif_bn_launch.h"
#include "lif_bn_plain.h"
#include "lif_bn_stats.h"

SNNLIF_DEFINE_BN_DTYPE(f32, float)
SNNLIF_DEFINE_BN_STATS_DTYPE(f32, float)
SNNLIF_DEFINE_BN_PLAIN_DTYPE(f32, float)
