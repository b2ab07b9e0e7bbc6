// Host-side interface of the batch-norm + fire kernels (lif_bn_kernels.h, lif_bn_launch.h, instantiated
// for float in lif_bn_f32.hip and for double in lif_bn_f64.hip), shared with the C ABI in lif_abi.hip.
#ifndef SNNLIF_LIF_BN_H
#define SNNLIF_LIF_BN_H

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace snnlif {

// Sweep 1 of the backward lays wavefronts over the (batch entry, channel) planes when a plane has at
// least this many positions (all lanes of a wavefront then share a channel and fold their sums by
// shuffles); smaller planes keep one lane per neuron in storage order.
constexpr int64_t kBnWavePlaneMin = 32;
inline bool bn_wave_partials(int64_t HW) { return HW >= kBnWavePlaneMin; }

// Partial sums sweep 1 leaves per quantity: one per wavefront (ceil(HW/64) per plane) or one per neuron.
inline size_t bn_partial_count(int64_t B, int64_t C, int64_t HW) {
    if (bn_wave_partials(HW)) return static_cast<size_t>(B * C) * static_cast<size_t>((HW + 63) / 64);
    return static_cast<size_t>(B * C * HW);
}

// Per-neuron partial sums are a [B, C*HW] matrix whose columns are summed over the batch in S slices
// (enough workgroups of kReduceBlock columns to fill the chip), then folded per channel.
constexpr int kReduceBlock = 256;
inline int bn_reduce_splits(int64_t B, int64_t CHW) {
    const int64_t groups = (CHW + kReduceBlock - 1) / kReduceBlock;
    int64_t s = (1024 + groups - 1) / groups;
    if (s > 64) s = 64;
    if (s > B) s = B;
    if (s < 1) s = 1;
    return static_cast<int>(s);
}

// Windows longer than this keep the membrane potential at the segment boundaries in device memory
// instead of LDS: sweep 1 in its workspace, sweep 2 in rows of the gradient it has yet to write.
constexpr int64_t kBnLdsBoundaryMaxT = 1024;
constexpr int64_t kBnSegment = 32;
inline size_t bn_boundary_elems(int64_t T, int64_t B, int64_t C, int64_t HW) {
    if (T <= kBnLdsBoundaryMaxT) return 0;
    return static_cast<size_t>((T + kBnSegment - 1) / kBnSegment) * static_cast<size_t>(B * C * HW);
}

// Workspace of the backward in elements of the scalar type:
// part_gy[P], part_gyx[P], split[2*S*C*HW] (per-neuron partials only), coef[2*C],
// boundary[ceil(T/32)*N] (T > 1024 only); P = bn_partial_count.
inline size_t bn_backward_workspace_elems(int64_t T, int64_t B, int64_t C, int64_t HW) {
    const size_t split = bn_wave_partials(HW)
                             ? 0
                             : static_cast<size_t>(2) * bn_reduce_splits(B, C * HW) * static_cast<size_t>(C * HW);
    return 2 * bn_partial_count(B, C, HW) + split + static_cast<size_t>(2 * C) +
           bn_boundary_elems(T, B, C, HW);
}

// Batch statistics (lif_bn_stats.h): threads per workgroup of the partial-sum kernels, the number of
// slices the rows of a small-plane tensor are dealt to (enough workgroups to fill the chip), partial
// sums per quantity (one per wavefront, or one per (slice, column)), and the workspace in doubles.
#ifndef SNNLIF_STATS_BLOCK
#define SNNLIF_STATS_BLOCK 256
#endif
constexpr int kStatsBlock = SNNLIF_STATS_BLOCK;
inline int bn_stats_row_slices(int64_t rows, int64_t CHW) {
    const int64_t groups = (CHW + kStatsBlock - 1) / kStatsBlock;
    int64_t s = (2048 + groups - 1) / groups;
    if (s > rows) s = rows;
    if (s > 1024) s = 1024;
    if (s < 1) s = 1;
    return static_cast<int>(s);
}
// Row slices of the plane-aligned statistics kernel: one per batch entry, fewer for windows shorter
// than the kernel's group of rows (so that every lane still sums a whole group).
// Rows of x a lane of the statistics kernels requests before it consumes the first: a read-only
// pass needs about twice as many requests in flight as the fire kernels (cold, [8,64,128,32,32]:
// 68 us with 8 rows, 55 us with 16; [8,128,128,32,32]: 131 / 99 us).
#ifndef SNNLIF_STATS_ROWS
#define SNNLIF_STATS_ROWS 16
#endif
inline int64_t bn_stats_wave_slices(int64_t T, int64_t B) {
    if (T >= SNNLIF_STATS_ROWS || B > 0x7fffffff / SNNLIF_STATS_ROWS) return B;  // (row counts stay in int)
    int64_t s = (T * B) / SNNLIF_STATS_ROWS;
    if (s > B) s = B;
    if (s < 1) s = 1;
    return s;
}
inline size_t bn_stats_partial_count(int64_t T, int64_t B, int64_t C, int64_t HW) {
    if (bn_wave_partials(HW)) return bn_partial_count(B, C, HW);
    return static_cast<size_t>(bn_stats_row_slices(T * B, C * HW)) * static_cast<size_t>(C * HW);
}
inline size_t bn_stats_workspace_elems(int64_t T, int64_t B, int64_t C, int64_t HW) {
    return 2 * bn_stats_partial_count(T, B, C, HW);
}

// Plain batch norm (lif_bn_plain.h).  Rows of the [T*B, C*HW] matrix a lane of the element-wise passes
// takes at a time, and a lane of the sums pass (x and g: twice as many requests in flight).  Measured
// at [8,64,128,32,32] fp32 with 16-byte lanes, input-gradient kernel: 2 rows 111 us, 4 rows 110, 6 rows
// 117, 8 rows 117-125, 16 rows 129; forward: 85 / 76 / 75 / 77 / 78; sums pass: 4 rows 107 us, 8 rows
// 84-87, 16 rows 88.
#ifndef SNNLIF_BN_PLAIN_ROWS
#define SNNLIF_BN_PLAIN_ROWS 4
#endif
#ifndef SNNLIF_BN_PLAIN_SUM_ROWS
#define SNNLIF_BN_PLAIN_SUM_ROWS 8
#endif
constexpr int kBnPlainRows = SNNLIF_BN_PLAIN_ROWS;
constexpr int kBnPlainSumRows = SNNLIF_BN_PLAIN_SUM_ROWS;
// Row slices of the sums pass: one group of kBnPlainSumRows rows per lane while that leaves few enough
// partial sums (at most 2^20 pairs; one per wavefront and slice, or one per column and slice), more
// rows per lane beyond.
inline int64_t bn_plain_slices(int64_t R, int64_t C, int64_t HW) {
    const int64_t per_slice = bn_wave_partials(HW) ? C * ((HW + 63) / 64) : C * HW;
    int64_t s = (R + kBnPlainSumRows - 1) / kBnPlainSumRows;
    const int64_t most = per_slice > 0 ? (int64_t(1) << 20) / per_slice : 1;
    if (s > most) s = most;
    if (s > 4096) s = 4096;
    if (s < 1) s = 1;
    return s;
}
// Workspace of the plain batch-norm backward in elements of the scalar type: the two partial-sum
// arrays ([S][C][ceil(HW/64)] each, or [S][C*HW] each) and the two per-channel means.
inline size_t bn_plain_workspace_elems(int64_t T, int64_t B, int64_t C, int64_t HW) {
    const int64_t per_slice = bn_wave_partials(HW) ? C * ((HW + 63) / 64) : C * HW;
    return static_cast<size_t>(2 * bn_plain_slices(T * B, C, HW) * per_slice + 2 * C);
}

enum class SpatialHint;  // lif_kernels.h

// What bn_stats_* writes (see below).
constexpr int kStatsVariance = 0, kStatsMoments = 1, kStatsSums = 2;

// The running statistics a layer keeps beside the batch statistics, advanced as the reference's layers do
// (snnlib/example/snnlib_op.py:79-80, 274-275): out = (in * keep) + (stat * gain), each product and the
// sum rounded in F like the framework's element-wise ops.  Null outputs: no update.
template <typename F>
struct RunningUpdate {
    const F* mean_in;
    const F* var_in;
    F* mean_out;
    F* var_out;
    F keep, gain_mean, gain_var;
};

// Per scalar type F (suffix f32 = float, f64 = double):
//   bn_stats_*           over (T, B, HW), per channel: mean and biased variance (mode kStatsVariance; with
//                        `running`, the layer's running pair is advanced in the same finish),
//                        E[x] and E[x^2] (kStatsMoments), or the plain sum into out_a alone (kStatsSums);
//   bn_moments_finish_*  mean = first * inv_world, var = second * inv_world - mean^2 from the moments a
//                        sharded batch has all-reduced, and the running pair, in one small kernel;
//   bn_forward_*         from_ivar = false: stat is the variance and ivar is written; true: stat is
//                        the inverse standard deviation and ivar is not touched.  keep_x: the caller's
//                        cache hint for x (lif_kernels.h).
//   bn_backward_stats_*  sweep 1 + channel reduction: parameter gradients and the two per-channel
//                        means (what a batch sharded over several GPUs runs before its all-reduce);
//   bn_backward_input_*  sweep 2: the input gradient from those means (after the all-reduce);
//   bn_backward_*        the two back to back, the means staged at the end of the workspace.
//   bn_plain_*           the batch norm without a fire recurrence: forward (var -> ivar, y), the
//                        backward's sums + channel reduction, its input gradient, and both back to back.
#define SNNLIF_DECLARE_BN_DTYPE(SUFFIX, F)                                                         \
    int bn_forward_##SUFFIX(const F* x, const F* weight, const F* bias, const F* stat,             \
                            const F* mean, F* ivar, F* spike, bool from_ivar, int64_t T,           \
                            int64_t B, int64_t C, int64_t HW, float eps, float alpha, float thresh,\
                            SpatialHint keep_x, hipStream_t stream);                               \
    int bn_stats_##SUFFIX(const F* x, F* out_a, F* out_b, int mode, int64_t T, int64_t B,          \
                          int64_t C, int64_t HW, double* workspace, hipStream_t stream,            \
                          const RunningUpdate<F>& running = RunningUpdate<F>{});                   \
    int bn_moments_finish_##SUFFIX(const F* first, const F* second, F* mean, F* var, F inv_world,  \
                                   const RunningUpdate<F>& running, int64_t C, hipStream_t stream);\
    int bn_backward_stats_##SUFFIX(const F* x, const F* weight, const F* bias, const F* ivar,      \
                                   const F* mean, const F* g, F* grad_weight, F* grad_bias,        \
                                   F* mean_gxhat, F* mean_gxhatx, int64_t T, int64_t B, int64_t C, \
                                   int64_t HW, float alpha, float thresh, float beta,              \
                                   float interval, F* workspace, hipStream_t stream);              \
    int bn_backward_input_##SUFFIX(const F* x, const F* weight, const F* bias, const F* ivar,      \
                                   const F* mean, const F* g, const F* mean_gxhat,                 \
                                   const F* mean_gxhatx, F* gx, int64_t T, int64_t B, int64_t C,   \
                                   int64_t HW, float alpha, float thresh, float beta,              \
                                   float interval, hipStream_t stream);                            \
    int bn_backward_##SUFFIX(const F* x, const F* weight, const F* bias, const F* ivar,            \
                             const F* mean, const F* g, F* gx, F* grad_weight, F* grad_bias,       \
                             int64_t T, int64_t B, int64_t C, int64_t HW, float alpha,             \
                             float thresh, float beta, float interval, F* workspace,               \
                             hipStream_t stream);

#define SNNLIF_DECLARE_BN_PLAIN_DTYPE(SUFFIX, F)                                                   \
    int bn_plain_forward_##SUFFIX(const F* x, const F* weight, const F* bias, const F* var,        \
                                  const F* mean, F* ivar, F* y, int64_t T, int64_t B, int64_t C,   \
                                  int64_t HW, float eps, hipStream_t stream);                      \
    int bn_plain_backward_stats_##SUFFIX(const F* x, const F* weight, const F* ivar,               \
                                         const F* mean, const F* g, F* grad_weight, F* grad_bias,  \
                                         F* mean_gxhat, F* mean_gxhatx, int64_t T, int64_t B,      \
                                         int64_t C, int64_t HW, F* workspace, hipStream_t stream); \
    int bn_plain_backward_input_##SUFFIX(const F* x, const F* weight, const F* ivar,               \
                                         const F* mean, const F* g, const F* mean_gxhat,           \
                                         const F* mean_gxhatx, F* gx, int64_t T, int64_t B,        \
                                         int64_t C, int64_t HW, hipStream_t stream);               \
    int bn_plain_backward_##SUFFIX(const F* x, const F* weight, const F* ivar, const F* mean,      \
                                   const F* g, F* gx, F* grad_weight, F* grad_bias, int64_t T,     \
                                   int64_t B, int64_t C, int64_t HW, F* workspace,                 \
                                   hipStream_t stream);

SNNLIF_DECLARE_BN_DTYPE(f32, float)
SNNLIF_DECLARE_BN_DTYPE(f64, double)
SNNLIF_DECLARE_BN_PLAIN_DTYPE(f32, float)
SNNLIF_DECLARE_BN_PLAIN_DTYPE(f64, double)
#undef SNNLIF_DECLARE_BN_DTYPE
#undef SNNLIF_DECLARE_BN_PLAIN_DTYPE

}  // namespace snnlif

#endif  // SNNLIF_LIF_BN_H
