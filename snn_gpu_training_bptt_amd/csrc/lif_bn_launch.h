// Launchers of the batch-norm + fire kernels, templated on the scalar type F (float or double); see
// lif_bn_kernels.h.  SNNLIF_DEFINE_BN_DTYPE at the end stamps out the typed entry points that
// lif_bn.h declares; lif_bn_f32.hip and lif_bn_f64.hip hold one instantiation each.
#ifndef SNNLIF_LIF_BN_LAUNCH_H
#define SNNLIF_LIF_BN_LAUNCH_H

#include "lif_bn_kernels.h"

namespace snnlif {

template <typename F, bool FROM_IVAR, bool KEEP>
int bn_forward_launch(const F* x, const F* weight, const F* bias, const F* stat, const F* mean,
                      F* ivar, F* spike, int64_t T, int64_t B, int64_t C, int64_t HW, float eps,
                      float alpha, float thresh, hipStream_t stream) {
    const int64_t N = B * C * HW;
    const int threads = forward_block(static_cast<size_t>(T) * static_cast<size_t>(N) * sizeof(F));
    const dim3 grid(grid_for(N, threads)), block(threads);
    const int Ti = static_cast<int>(T);
    constexpr int TC = SNNLIF_FWD_ROWS;
    if (T <= 4 && TC > 4) {
        launch_kernel(lif_bn_forward_kernel<F, 4, false, FROM_IVAR, KEEP>, grid, block, 0, stream, x,
                      weight, bias, stat, mean, ivar, spike, Ti, N, C, HW, F(eps), F(alpha),
                      F(thresh));
    } else if (T <= TC) {
        launch_kernel(lif_bn_forward_kernel<F, TC, false, FROM_IVAR, KEEP>, grid, block, 0, stream, x,
                      weight, bias, stat, mean, ivar, spike, Ti, N, C, HW, F(eps), F(alpha),
                      F(thresh));
    } else {
        launch_kernel(lif_bn_forward_kernel<F, TC, true, FROM_IVAR, KEEP>, grid, block, 0, stream, x,
                      weight, bias, stat, mean, ivar, spike, Ti, N, C, HW, F(eps), F(alpha),
                      F(thresh));
    }
    return launch_status();
}

// from_ivar = false: stat is the variance and ivar is written; true: stat is the inverse standard
// deviation and ivar is not touched.  keep_x: the caller's cache hint; without one, tensors the
// memory-side cache is likely to hold anyway are kept and larger ones streamed, as in the plain fire.
template <typename F>
int bn_forward(const F* x, const F* weight, const F* bias, const F* stat, const F* mean, F* ivar,
               F* spike, bool from_ivar, int64_t T, int64_t B, int64_t C, int64_t HW, float eps,
               float alpha, float thresh, SpatialHint keep_x, hipStream_t stream) {
    const bool keep = keep_policy(
        keep_x, static_cast<size_t>(T) * static_cast<size_t>(B * C * HW) * sizeof(F));
#define SNNLIF_BN_FWD(FROM_IVAR, KEEP)                                                            \
    bn_forward_launch<F, FROM_IVAR, KEEP>(x, weight, bias, stat, mean, ivar, spike, T, B, C, HW, eps, \
                                          alpha, thresh, stream)
    if (from_ivar) return keep ? SNNLIF_BN_FWD(true, true) : SNNLIF_BN_FWD(true, false);
    return keep ? SNNLIF_BN_FWD(false, true) : SNNLIF_BN_FWD(false, false);
#undef SNNLIF_BN_FWD
}

// Small workgroup of the two backward sweeps (see backward_block): the sweeps carry more state per
// wavefront than the plain backward and single-wavefront groups cost them more than they gain.
constexpr int kBnSmallBlock = 128;

// Longest window for which a lane of the plane-aligned sweep 1 takes two batch entries (2 * T
// requests per entry: sixteen or more in flight from 4 steps on; windows of 7 steps and more have
// them on their own).
#ifndef SNNLIF_BN_PAIRED_MAX_T
#define SNNLIF_BN_PAIRED_MAX_T 6
#endif
constexpr int kBnPairedMaxT = SNNLIF_BN_PAIRED_MAX_T;

// Dynamic LDS of the segmented sweeps: one boundary value per segment and lane.
template <typename F>
inline size_t bn_segment_lds_bytes(int64_t T, int threads) {
    return static_cast<size_t>((T + kSegment - 1) / kSegment) * threads * sizeof(F);
}

// Sweep 1 + channel reduction for windows of at most TW steps (segmented walks: of any length, in
// segments of TW = kSegment steps): parameter gradients and the two per-channel means the
// input-gradient sweep needs.
template <typename F, int TW, TimeWalk WALK = TimeWalk::window>
int bn_backward_stats_window(const F* x, const F* weight, const F* bias, const F* ivar,
                             const F* mean, const F* g, F* grad_weight, F* grad_bias, F* mean_gxhat,
                             F* mean_gxhatx, int64_t T, int64_t B, int64_t C, int64_t HW, float alpha,
                             float thresh, float beta, float interval, F* workspace,
                             hipStream_t stream) {
    constexpr bool segmented = WALK != TimeWalk::window;
    const int64_t N = B * C * HW;
    const int S = bn_reduce_splits(B, C * HW);
    const size_t P = bn_partial_count(B, C, HW);
    F* part_gy = workspace;
    F* part_gyx = part_gy + P;
    F* split = part_gyx + P;
    // boundary potentials of a window too long for LDS: the tail of the workspace, [segment][N]
    F* far = workspace + bn_backward_workspace_elems(T, B, C, HW) - bn_boundary_elems(T, B, C, HW);
    const int threads =
        backward_block(static_cast<size_t>(T) * static_cast<size_t>(N) * sizeof(F), kBnSmallBlock);
    const dim3 block(threads);
    const int Ti = static_cast<int>(T);
    constexpr bool can_be_inexact = TW > 8;
    const bool exact = !segmented && (!can_be_inexact || (T == TW));
    const size_t lds = WALK == TimeWalk::segments_lds ? bn_segment_lds_bytes<F>(T, threads) : 0;

    // Planes with few positions (fully connected shapes) would leave most lanes of a plane-aligned
    // wavefront idle; they keep one lane per neuron and per-neuron partials.
    const bool wave = bn_wave_partials(HW);
    const int64_t G = (HW + 63) / 64;
    // windows of at most kBnPairedMaxT steps: a lane of the plane-aligned sweep takes two batch entries
    constexpr bool can_pair = !segmented && TW <= kBnPairedMaxT;
    const int64_t nb = (can_pair && wave && B % 2 == 0) ? 2 : 1;
    const dim3 grid_partial(wave ? grid_for((B / nb) * C * G * 64, threads) : grid_for(N, threads));
    int rc;
#define SNNLIF_BN_PARTIAL_NB(EXACT_, WAVE_, NB_)                                                   \
    launch_kernel(lif_bn_backward_partial_kernel<F, TW, EXACT_, WAVE_, WALK, NB_>, grid_partial,   \
                  block, lds, stream, x, g, weight, bias, ivar, mean, part_gy, part_gyx, far, Ti,  \
                  N, C, HW, F(alpha), F(thresh), F(beta), F(interval))
#define SNNLIF_BN_PARTIAL(EXACT_, WAVE_) SNNLIF_BN_PARTIAL_NB(EXACT_, WAVE_, 1)
    if constexpr (segmented) {
        if (wave) SNNLIF_BN_PARTIAL(false, true); else SNNLIF_BN_PARTIAL(false, false);
    } else if (exact) {
        if (nb == 2) {
            if constexpr (can_pair) SNNLIF_BN_PARTIAL_NB(true, true, 2);
        } else if (wave) {
            SNNLIF_BN_PARTIAL(true, true);
        } else {
            SNNLIF_BN_PARTIAL(true, false);
        }
    } else if constexpr (can_be_inexact) {
        if (wave) SNNLIF_BN_PARTIAL(false, true); else SNNLIF_BN_PARTIAL(false, false);
    }
#undef SNNLIF_BN_PARTIAL
#undef SNNLIF_BN_PARTIAL_NB
    rc = launch_status();
    if (rc != SNNLIF_OK) return rc;

    const F count = static_cast<F>(T * B * HW);
    if (wave) {
        launch_kernel(bn_channel_reduce_finalize_kernel<F>, dim3(static_cast<unsigned>(C)),
                      dim3(kReduceBlock), 0, stream, part_gy, part_gyx, weight, grad_weight,
                      grad_bias, mean_gxhat, mean_gxhatx, B / nb, C, G, count);
        return launch_status();
    }
    const int64_t CHW = C * HW;
    const int64_t bs = (B + S - 1) / S;
    launch_kernel(bn_column_reduce_kernel<F>,
                  dim3(static_cast<unsigned>((CHW + kReduceBlock - 1) / kReduceBlock), S),
                  dim3(kReduceBlock), 0, stream, part_gy, part_gyx, split, B, CHW, bs, S);
    rc = launch_status();
    if (rc != SNNLIF_OK) return rc;
    launch_kernel(bn_channel_finalize_kernel<F>,
                  dim3(static_cast<unsigned>((C + kReduceBlock / 64 - 1) / (kReduceBlock / 64))),
                  dim3(kReduceBlock), 0, stream, split, weight, grad_weight, grad_bias, mean_gxhat,
                  mean_gxhatx, C, HW, S, count);
    return launch_status();
}

// Sweep 2 for windows of at most TW steps (segmented walks: as above).
template <typename F, int TW, TimeWalk WALK = TimeWalk::window>
int bn_backward_input_window(const F* x, const F* weight, const F* bias, const F* ivar,
                             const F* mean, const F* g, const F* mean_gxhat, const F* mean_gxhatx,
                             F* gx, int64_t T, int64_t B, int64_t C, int64_t HW, float alpha,
                             float thresh, float beta, float interval, hipStream_t stream) {
    constexpr bool segmented = WALK != TimeWalk::window;
    const int64_t N = B * C * HW;
    const int threads =
        backward_block(static_cast<size_t>(T) * static_cast<size_t>(N) * sizeof(F), kBnSmallBlock);
    const dim3 grid(grid_for(N, threads)), block(threads);
    const int Ti = static_cast<int>(T);
    constexpr bool can_be_inexact = TW > 8;
    const bool exact = !segmented && (!can_be_inexact || (T == TW));
    if constexpr (segmented) {
        const size_t lds = WALK == TimeWalk::segments_lds ? bn_segment_lds_bytes<F>(T, threads) : 0;
        launch_kernel(lif_bn_backward_input_kernel<F, TW, false, WALK>, grid, block, lds, stream, x, g,
                      weight, bias, ivar, mean, mean_gxhat, mean_gxhatx, gx, Ti, N, C, HW, F(alpha),
                      F(thresh), F(beta), F(interval));
    } else if (exact) {
        launch_kernel(lif_bn_backward_input_kernel<F, TW, true>, grid, block, 0, stream, x, g, weight,
                      bias, ivar, mean, mean_gxhat, mean_gxhatx, gx, Ti, N, C, HW, F(alpha),
                      F(thresh), F(beta), F(interval));
    } else if constexpr (can_be_inexact) {
        launch_kernel(lif_bn_backward_input_kernel<F, TW, false>, grid, block, 0, stream, x, g,
                      weight, bias, ivar, mean, mean_gxhat, mean_gxhatx, gx, Ti, N, C, HW, F(alpha),
                      F(thresh), F(beta), F(interval));
    }
    return launch_status();
}

// Window lengths with a kernel instance of their own; any other T <= 32 runs in the next one up.
#define SNNLIF_BN_WINDOWS(X) X(1) X(2) X(3) X(4) X(5) X(6) X(7) X(8) X(10) X(12) X(16) X(20) X(24) X(28) X(32)

template <typename F>
int bn_backward_stats(const F* x, const F* weight, const F* bias, const F* ivar, const F* mean,
                      const F* g, F* grad_weight, F* grad_bias, F* mean_gxhat, F* mean_gxhatx,
                      int64_t T, int64_t B, int64_t C, int64_t HW, float alpha, float thresh,
                      float beta, float interval, F* workspace, hipStream_t stream) {
#define SNNLIF_BN_WINDOW(TW)                                                                       \
    if (T <= TW)                                                                                   \
        return bn_backward_stats_window<F, TW>(x, weight, bias, ivar, mean, g, grad_weight,        \
                                               grad_bias, mean_gxhat, mean_gxhatx, T, B, C, HW,    \
                                               alpha, thresh, beta, interval, workspace, stream);
    SNNLIF_BN_WINDOWS(SNNLIF_BN_WINDOW)
#undef SNNLIF_BN_WINDOW
    if (T <= kBnLdsBoundaryMaxT)
        return bn_backward_stats_window<F, kSegment, TimeWalk::segments_lds>(
            x, weight, bias, ivar, mean, g, grad_weight, grad_bias, mean_gxhat, mean_gxhatx, T, B, C,
            HW, alpha, thresh, beta, interval, workspace, stream);
    return bn_backward_stats_window<F, kSegment, TimeWalk::segments_memory>(
        x, weight, bias, ivar, mean, g, grad_weight, grad_bias, mean_gxhat, mean_gxhatx, T, B, C, HW,
        alpha, thresh, beta, interval, workspace, stream);
}

template <typename F>
int bn_backward_input(const F* x, const F* weight, const F* bias, const F* ivar, const F* mean,
                      const F* g, const F* mean_gxhat, const F* mean_gxhatx, F* gx, int64_t T,
                      int64_t B, int64_t C, int64_t HW, float alpha, float thresh, float beta,
                      float interval, hipStream_t stream) {
#define SNNLIF_BN_WINDOW(TW)                                                                       \
    if (T <= TW)                                                                                   \
        return bn_backward_input_window<F, TW>(x, weight, bias, ivar, mean, g, mean_gxhat,         \
                                               mean_gxhatx, gx, T, B, C, HW, alpha, thresh, beta,  \
                                               interval, stream);
    SNNLIF_BN_WINDOWS(SNNLIF_BN_WINDOW)
#undef SNNLIF_BN_WINDOW
    if (T <= kBnLdsBoundaryMaxT)
        return bn_backward_input_window<F, kSegment, TimeWalk::segments_lds>(
            x, weight, bias, ivar, mean, g, mean_gxhat, mean_gxhatx, gx, T, B, C, HW, alpha, thresh,
            beta, interval, stream);
    return bn_backward_input_window<F, kSegment, TimeWalk::segments_memory>(
        x, weight, bias, ivar, mean, g, mean_gxhat, mean_gxhatx, gx, T, B, C, HW, alpha, thresh, beta,
        interval, stream);
}

template <typename F>
int bn_backward(const F* x, const F* weight, const F* bias, const F* ivar, const F* mean, const F* g,
                F* gx, F* grad_weight, F* grad_bias, int64_t T, int64_t B, int64_t C, int64_t HW,
                float alpha, float thresh, float beta, float interval, F* workspace,
                hipStream_t stream) {
    // the two per-channel means live behind the partial sums in the workspace between the sweeps
    F* coef = workspace + bn_backward_workspace_elems(T, B, C, HW) - bn_boundary_elems(T, B, C, HW) -
              2 * C;
    const int rc = bn_backward_stats<F>(x, weight, bias, ivar, mean, g, grad_weight, grad_bias, coef,
                                        coef + C, T, B, C, HW, alpha, thresh, beta, interval,
                                        workspace, stream);
    if (rc != SNNLIF_OK) return rc;
    return bn_backward_input<F>(x, weight, bias, ivar, mean, g, coef, coef + C, gx, T, B, C, HW, alpha,
                                thresh, beta, interval, stream);
}

}  // namespace snnlif

// The entry points lif_bn.h declares for scalar type F under the name suffix SUFFIX.
#define SNNLIF_DEFINE_BN_DTYPE(SUFFIX, F)                                                          \
    namespace snnlif {                                                                             \
    int bn_forward_##SUFFIX(const F* x, const F* weight, const F* bias, const F* stat,             \
                            const F* mean, F* ivar, F* spike, bool from_ivar, int64_t T,           \
                            int64_t B, int64_t C, int64_t HW, float eps, float alpha, float thresh,\
                            SpatialHint keep_x, hipStream_t stream) {                              \
        return bn_forward<F>(x, weight, bias, stat, mean, ivar, spike, from_ivar, T, B, C, HW, eps,\
                             alpha, thresh, keep_x, stream);                                       \
    }                                                                                              \
    int bn_backward_stats_##SUFFIX(const F* x, const F* weight, const F* bias, const F* ivar,      \
                                   const F* mean, const F* g, F* grad_weight, F* grad_bias,        \
                                   F* mean_gxhat, F* mean_gxhatx, int64_t T, int64_t B, int64_t C, \
                                   int64_t HW, float alpha, float thresh, float beta,              \
                                   float interval, F* workspace, hipStream_t stream) {             \
        return bn_backward_stats<F>(x, weight, bias, ivar, mean, g, grad_weight, grad_bias,        \
                                    mean_gxhat, mean_gxhatx, T, B, C, HW, alpha, thresh, beta,     \
                                    interval, workspace, stream);                                  \
    }                                                                                              \
    int bn_backward_input_##SUFFIX(const F* x, const F* weight, const F* bias, const F* ivar,      \
                                   const F* mean, const F* g, const F* mean_gxhat,                 \
                                   const F* mean_gxhatx, F* gx, int64_t T, int64_t B, int64_t C,   \
                                   int64_t HW, float alpha, float thresh, float beta,              \
                                   float interval, hipStream_t stream) {                           \
        return bn_backward_input<F>(x, weight, bias, ivar, mean, g, mean_gxhat, mean_gxhatx, gx, T,\
                                    B, C, HW, alpha, thresh, beta, interval, stream);              \
    }                                                                                              \
    int bn_backward_##SUFFIX(const F* x, const F* weight, const F* bias, const F* ivar,            \
                             const F* mean, const F* g, F* gx, F* grad_weight, F* grad_bias,       \
                             int64_t T, int64_t B, int64_t C, int64_t HW, float alpha,             \
                             float thresh, float beta, float interval, F* workspace,               \
                             hipStream_t stream) {                                                 \
        return bn_backward<F>(x, weight, bias, ivar, mean, g, gx, grad_weight, grad_bias, T, B, C, \
                              HW, alpha, thresh, beta, interval, workspace, stream);               \
    }                                                                                              \
    }

#endif  // SNNLIF_LIF_BN_LAUNCH_H
