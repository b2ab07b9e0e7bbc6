// Launchers of the batch-norm + fire kernels (fp32); see lif_bn_kernels.h.
#include "lif_bn_kernels.h"

namespace snnlif {

namespace {

template <bool FROM_IVAR>
int bn_forward_launch(const float* x, const float* weight, const float* bias, const float* stat,
                      const float* mean, float* ivar, float* spike, int64_t T, int64_t B, int64_t C,
                      int64_t HW, float eps, float alpha, float thresh, hipStream_t stream) {
    const int64_t N = B * C * HW;
    const int threads = forward_block(static_cast<size_t>(T) * static_cast<size_t>(N) * sizeof(float));
    const dim3 grid(grid_for(N, threads)), block(threads);
    const int Ti = static_cast<int>(T);
    constexpr int TC = SNNLIF_FWD_ROWS;
    if (T <= 4 && TC > 4) {
        launch_kernel(lif_bn_forward_kernel<4, false, FROM_IVAR>, grid, block, 0, stream, x,
                           weight, bias, stat, mean, ivar, spike, Ti, N, C, HW, eps, alpha, thresh);
    } else if (T <= TC) {
        launch_kernel(lif_bn_forward_kernel<TC, false, FROM_IVAR>, grid, block, 0, stream, x,
                           weight, bias, stat, mean, ivar, spike, Ti, N, C, HW, eps, alpha, thresh);
    } else {
        launch_kernel(lif_bn_forward_kernel<TC, true, FROM_IVAR>, grid, block, 0, stream, x,
                           weight, bias, stat, mean, ivar, spike, Ti, N, C, HW, eps, alpha, thresh);
    }
    return launch_status();
}

}  // namespace

int bn_forward_f32(const float* x, const float* weight, const float* bias, const float* stat,
                   const float* mean, float* ivar, float* spike, bool from_ivar, int64_t T,
                   int64_t B, int64_t C, int64_t HW, float eps, float alpha, float thresh,
                   hipStream_t stream) {
    if (from_ivar)
        return bn_forward_launch<true>(x, weight, bias, stat, mean, ivar, spike, T, B, C, HW, eps,
                                       alpha, thresh, stream);
    return bn_forward_launch<false>(x, weight, bias, stat, mean, ivar, spike, T, B, C, HW, eps, alpha,
                                    thresh, stream);
}

namespace {

// Small workgroup of the two backward sweeps (see backward_block): the sweeps carry more state per
// wavefront than the plain backward and single-wavefront groups cost them more than they gain.
constexpr int kBnSmallBlock = 128;

// Dynamic LDS of the segmented sweeps: one boundary value per segment and lane.
inline size_t bn_segment_lds_bytes(int64_t T, int threads) {
    return static_cast<size_t>((T + kSegment - 1) / kSegment) * threads * sizeof(float);
}

// Sweep 1 + channel reduction for windows of at most TW steps (SEGMENTED: of any length up to
// SNNLIF_BP_NO_WORKSPACE_MAX_T, in segments of TW = kSegment steps): parameter gradients and the two
// per-channel means the input-gradient sweep needs.
template <int TW, bool SEGMENTED = false>
int bn_backward_stats_window(const float* x, const float* weight, const float* bias,
                             const float* ivar, const float* mean, const float* g,
                             float* grad_weight, float* grad_bias, float* mean_gxhat,
                             float* mean_gxhatx, int64_t T, int64_t B, int64_t C, int64_t HW,
                             float alpha, float thresh, float beta, float interval,
                             float* workspace, hipStream_t stream) {
    const int64_t N = B * C * HW;
    const int S = bn_reduce_splits(B, C);
    float* part_gy = workspace;
    float* part_gyx = part_gy + N;
    float* split = part_gyx + N;
    const int threads = backward_block(static_cast<size_t>(T) * static_cast<size_t>(N) * sizeof(float), kBnSmallBlock);
    const dim3 block(threads);
    const int Ti = static_cast<int>(T);
    constexpr bool can_be_inexact = TW > 8;
    const bool exact = !SEGMENTED && (!can_be_inexact || (T == TW));
    const size_t lds = SEGMENTED ? bn_segment_lds_bytes(T, threads) : 0;

    // Planes with few positions (fully connected shapes) would leave most lanes of a plane-aligned
    // wavefront idle; they keep one lane per neuron and per-neuron partials.
    const bool wave = HW >= 32;
    const int64_t G = (HW + 63) / 64;
    const dim3 grid_partial(wave ? grid_for(B * C * G * 64, threads) : grid_for(N, threads));
    int rc;
#define SNNLIF_BN_PARTIAL(EXACT_, WAVE_)                                                          \
    launch_kernel(lif_bn_backward_partial_kernel<TW, EXACT_, WAVE_, SEGMENTED>, grid_partial, block, \
                  lds, stream, x, g, weight, bias, ivar, mean, part_gy, part_gyx, Ti, N, C, HW,   \
                  alpha, thresh, beta, interval)
    if constexpr (SEGMENTED) {
        if (wave) SNNLIF_BN_PARTIAL(false, true); else SNNLIF_BN_PARTIAL(false, false);
    } else if (exact) {
        if (wave) SNNLIF_BN_PARTIAL(true, true); else SNNLIF_BN_PARTIAL(true, false);
    } else if constexpr (can_be_inexact) {
        if (wave) SNNLIF_BN_PARTIAL(false, true); else SNNLIF_BN_PARTIAL(false, false);
    }
#undef SNNLIF_BN_PARTIAL
    rc = launch_status();
    if (rc != SNNLIF_OK) return rc;

    const float count = static_cast<float>(T * B * HW);
    if (wave) {
        launch_kernel(bn_channel_reduce_finalize_kernel, dim3(static_cast<unsigned>(C)),
                      dim3(kReduceBlock), 0, stream, part_gy, part_gyx, weight, grad_weight,
                      grad_bias, mean_gxhat, mean_gxhatx, B, C, G, count);
        return launch_status();
    }
    const int64_t bs = (B + S - 1) / S;
    launch_kernel(bn_channel_reduce_kernel, dim3(static_cast<unsigned>(C), S), dim3(kReduceBlock),
                  0, stream, part_gy, part_gyx, split, B, C, HW, bs, S);
    rc = launch_status();
    if (rc != SNNLIF_OK) return rc;
    launch_kernel(bn_channel_finalize_kernel,
                  dim3(static_cast<unsigned>((C + kReduceBlock - 1) / kReduceBlock)),
                  dim3(kReduceBlock), 0, stream, split, weight, grad_weight, grad_bias, mean_gxhat,
                  mean_gxhatx, C, S, count);
    return launch_status();
}

// Sweep 2 for windows of at most TW steps (SEGMENTED: as above).
template <int TW, bool SEGMENTED = false>
int bn_backward_input_window(const float* x, const float* weight, const float* bias,
                             const float* ivar, const float* mean, const float* g,
                             const float* mean_gxhat, const float* mean_gxhatx, float* gx, int64_t T,
                             int64_t B, int64_t C, int64_t HW, float alpha, float thresh, float beta,
                             float interval, hipStream_t stream) {
    const int64_t N = B * C * HW;
    const int threads = backward_block(static_cast<size_t>(T) * static_cast<size_t>(N) * sizeof(float), kBnSmallBlock);
    const dim3 grid(grid_for(N, threads)), block(threads);
    const int Ti = static_cast<int>(T);
    constexpr bool can_be_inexact = TW > 8;
    const bool exact = !SEGMENTED && (!can_be_inexact || (T == TW));
    if constexpr (SEGMENTED) {
        launch_kernel(lif_bn_backward_input_kernel<TW, false, true>, grid, block,
                      bn_segment_lds_bytes(T, threads), stream, x, g, weight, bias, ivar, mean, mean_gxhat,
                      mean_gxhatx, gx, Ti, N, C, HW, alpha, thresh, beta, interval);
    } else if (exact) {
        launch_kernel(lif_bn_backward_input_kernel<TW, true>, grid, block, 0, stream, x, g, weight,
                      bias, ivar, mean, mean_gxhat, mean_gxhatx, gx, Ti, N, C, HW, alpha, thresh,
                      beta, interval);
    } else if constexpr (can_be_inexact) {
        launch_kernel(lif_bn_backward_input_kernel<TW, false>, grid, block, 0, stream, x, g, weight,
                      bias, ivar, mean, mean_gxhat, mean_gxhatx, gx, Ti, N, C, HW, alpha, thresh,
                      beta, interval);
    }
    return launch_status();
}

}  // namespace

// Window lengths with a kernel instance of their own; any other T <= 32 runs in the next one up.
#define SNNLIF_BN_WINDOWS(X) X(1) X(2) X(3) X(4) X(5) X(6) X(7) X(8) X(10) X(12) X(16) X(20) X(24) X(28) X(32)

int bn_backward_stats_f32(const float* x, const float* weight, const float* bias, const float* ivar,
                          const float* mean, const float* g, float* grad_weight, float* grad_bias,
                          float* mean_gxhat, float* mean_gxhatx, int64_t T, int64_t B, int64_t C,
                          int64_t HW, float alpha, float thresh, float beta, float interval,
                          float* workspace, hipStream_t stream) {
#define SNNLIF_BN_WINDOW(TW)                                                                      \
    if (T <= TW)                                                                                  \
        return bn_backward_stats_window<TW>(x, weight, bias, ivar, mean, g, grad_weight, grad_bias, \
                                            mean_gxhat, mean_gxhatx, T, B, C, HW, alpha, thresh,   \
                                            beta, interval, workspace, stream);
    SNNLIF_BN_WINDOWS(SNNLIF_BN_WINDOW)
#undef SNNLIF_BN_WINDOW
    if (T <= SNNLIF_BP_NO_WORKSPACE_MAX_T)
        return bn_backward_stats_window<kSegment, true>(x, weight, bias, ivar, mean, g, grad_weight,
                                                        grad_bias, mean_gxhat, mean_gxhatx, T, B, C,
                                                        HW, alpha, thresh, beta, interval, workspace,
                                                        stream);
    return SNNLIF_ERR_UNSUPPORTED;
}

int bn_backward_input_f32(const float* x, const float* weight, const float* bias, const float* ivar,
                          const float* mean, const float* g, const float* mean_gxhat,
                          const float* mean_gxhatx, float* gx, int64_t T, int64_t B, int64_t C,
                          int64_t HW, float alpha, float thresh, float beta, float interval,
                          hipStream_t stream) {
#define SNNLIF_BN_WINDOW(TW)                                                                      \
    if (T <= TW)                                                                                  \
        return bn_backward_input_window<TW>(x, weight, bias, ivar, mean, g, mean_gxhat,           \
                                            mean_gxhatx, gx, T, B, C, HW, alpha, thresh, beta,    \
                                            interval, stream);
    SNNLIF_BN_WINDOWS(SNNLIF_BN_WINDOW)
#undef SNNLIF_BN_WINDOW
    if (T <= SNNLIF_BP_NO_WORKSPACE_MAX_T)
        return bn_backward_input_window<kSegment, true>(x, weight, bias, ivar, mean, g, mean_gxhat,
                                                        mean_gxhatx, gx, T, B, C, HW, alpha, thresh,
                                                        beta, interval, stream);
    return SNNLIF_ERR_UNSUPPORTED;
}

int bn_backward_f32(const float* x, const float* weight, const float* bias, const float* ivar,
                    const float* mean, const float* g, float* gx, float* grad_weight,
                    float* grad_bias, int64_t T, int64_t B, int64_t C, int64_t HW, float alpha,
                    float thresh, float beta, float interval, float* workspace,
                    hipStream_t stream) {
    // the two per-channel means live at the end of the workspace between the sweeps
    float* coef = workspace + bn_backward_workspace_floats(B, C, HW) - 2 * C;
    const int rc = bn_backward_stats_f32(x, weight, bias, ivar, mean, g, grad_weight, grad_bias,
                                         coef, coef + C, T, B, C, HW, alpha, thresh, beta, interval,
                                         workspace, stream);
    if (rc != SNNLIF_OK) return rc;
    return bn_backward_input_f32(x, weight, bias, ivar, mean, g, coef, coef + C, gx, T, B, C, HW,
                                 alpha, thresh, beta, interval, stream);
}

}  // namespace snnlif
