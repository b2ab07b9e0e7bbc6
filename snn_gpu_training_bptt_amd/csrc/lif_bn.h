// Host-side interface of the batch-norm + fire kernels (lif_bn_kernels.h, lif_bn_f32.hip), shared
// with the C ABI in lif_abi.hip.
#ifndef SNNLIF_LIF_BN_H
#define SNNLIF_LIF_BN_H

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace snnlif {

// Number of batch slices each channel's reduction is split into (enough workgroups to fill the
// chip when there are few channels).
inline int bn_reduce_splits(int64_t B, int64_t C) {
    int64_t s = 2048 / (C > 0 ? C : 1);
    if (s < 1) s = 1;
    if (s > B) s = B;
    if (s > 65535) s = 65535;
    return static_cast<int>(s);
}

// floats: part_gy[N], part_gyx[N], split[2*S*C], coef[2*C]
inline size_t bn_backward_workspace_floats(int64_t B, int64_t C, int64_t HW) {
    const int S = bn_reduce_splits(B, C);
    return static_cast<size_t>(2 * B * C * HW) + static_cast<size_t>(2) * S * C +
           static_cast<size_t>(2 * C);
}

// from_ivar = false: stat is the variance and ivar is written; true: stat is the inverse standard
// deviation and ivar is not touched.
int bn_forward_f32(const float* x, const float* weight, const float* bias, const float* stat,
                   const float* mean, float* ivar, float* spike, bool from_ivar, int64_t T,
                   int64_t B, int64_t C, int64_t HW, float eps, float alpha, float thresh,
                   hipStream_t stream);

// The backward in its two halves (what a batch sharded over several GPUs runs on either side of the
// all-reduce of the two per-channel means): sweep 1 + channel reduction, then sweep 2.
// bn_backward_f32 is the two back to back.
int bn_backward_stats_f32(const float* x, const float* weight, const float* bias, const float* ivar,
                          const float* mean, const float* g, float* grad_weight, float* grad_bias,
                          float* mean_gxhat, float* mean_gxhatx, int64_t T, int64_t B, int64_t C,
                          int64_t HW, float alpha, float thresh, float beta, float interval,
                          float* workspace, hipStream_t stream);

int bn_backward_input_f32(const float* x, const float* weight, const float* bias, const float* ivar,
                          const float* mean, const float* g, const float* mean_gxhat,
                          const float* mean_gxhatx, float* gx, int64_t T, int64_t B, int64_t C,
                          int64_t HW, float alpha, float thresh, float beta, float interval,
                          hipStream_t stream);

int bn_backward_f32(const float* x, const float* weight, const float* bias, const float* ivar,
                    const float* mean, const float* g, float* gx, float* grad_weight,
                    float* grad_bias, int64_t T, int64_t B, int64_t C, int64_t HW, float alpha,
                    float thresh, float beta, float interval, float* workspace,
                    hipStream_t stream);

}  // namespace snnlif

#endif  // SNNLIF_LIF_BN_H
