// Batch-norm + fire kernels for double storage and arithmetic; see lif_bn_launch.h.
#include "lif_bn_launch.h"
#include "lif_bn_plain.h"
#include "lif_bn_stats.h"

SNNLIF_DEFINE_BN_DTYPE(f64, double)
SNNLIF_DEFINE_BN_STATS_DTYPE(f64, double)
SNNLIF_DEFINE_BN_PLAIN_DTYPE(f64, double)
