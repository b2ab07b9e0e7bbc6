/*
 * lif_oracle.c -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * Scalar CPU restatement of the reference's LIF "fire" kernels, used only as the checker in
 * tests/, in __graft_entry__.smoke() and in bench.py's cpu_baseline leg.  Nothing in the shipped
 * package may call it.  Build: `make -C oracle` (gcc -O2 -ffp-contract=off, no fast-math), which
 * keeps every product and sum individually rounded, as the reference's fp32 arithmetic is.
 *
 * Loop nest, indexing and operation order follow the reference one to one:
 *   forward  : snnlib/cuda/snn_kernel_fp.cu:37-52  (fire_s_fp_kernel)
 *              snnlib/cuda/snn_kernel_bp.cu:34-51  (fire_u_fp_kernel), :73-92 (fire_us_fp_kernel)
 *   backward : snnlib/cuda/snn_kernel_bp.cu:117-138 (fire_bp_kernel), driven as in
 *              fire_bp_cuda, snnlib/cuda/snn_kernel_bp.cu:141-168 (recompute mem, then reverse sweep)
 * Shapes are the reference's: T time steps, B batch entries, CHW neurons per entry, element
 * (t, b, i) at t*B*CHW + b*CHW + i (snnlib/cuda/snn_kernel_fp.cu:45).
 *
 * Parity pinning: the reference ships no golden vectors for this path.  These functions are
 * pinned in tests/test_oracle_pinning.py by closed forms (T=1, alpha=0, dyadic geometric sums,
 * always-spiking inputs, hand-derived T=2/T=3 gradients), by an independent exact-rounding
 * emulation in pure Python, and by agreement with autograd through oracle/gold_fire.py, which is
 * written from the reference's pure-PyTorch statement (snnlib/example/gold_op.py:17-44) rather than
 * from the kernels.
 */
#include <stdint.h>

#define LIF_ORACLE_DEFINE(SUFFIX, SCALAR)                                                          \
    /* mem and/or spike may be NULL */                                                             \
    void lif_oracle_forward_##SUFFIX(const SCALAR* spatial, SCALAR* mem, SCALAR* spike, int64_t T, \
                                     int64_t B, int64_t CHW, float alpha, float thresh) {          \
        const int64_t step_stride = B * CHW;                                                              \
        for (int64_t i = 0; i < CHW; i++) {                                                        \
            for (int64_t b = 0; b < B; b++) {                                                      \
                SCALAR potential = 0;                                                                \
                int fired = 0;                                                                   \
                for (int64_t t = 0; t < T; t++) {                                                  \
                    const int64_t at = t * step_stride + b * CHW + i;                                  \
                    potential = alpha * potential * (1 - fired) + spatial[at];                    \
                    fired = potential > thresh;                                                    \
                    if (mem) mem[at] = potential;                                                 \
                    if (spike) spike[at] = (SCALAR)fired;                                     \
                }                                                                                  \
            }                                                                                      \
        }                                                                                          \
    }                                                                                              \
                                                                                                   \
    /* reverse sweep over a given membrane tensor */                                               \
    void lif_oracle_reverse_##SUFFIX(const SCALAR* grad_spike, const SCALAR* mem,                  \
                                     SCALAR* grad_spatial, int64_t T, int64_t B, int64_t CHW,          \
                                     float alpha, float thresh, float beta, float interval) {      \
        const int64_t step_stride = B * CHW;                                                              \
        for (int64_t i = 0; i < CHW; i++) {                                                        \
            for (int64_t b = 0; b < B; b++) {                                                      \
                SCALAR carried = 0;                                                            \
                for (int64_t t = T - 1; t >= 0; t--) {                                             \
                    const int64_t at = t * step_stride + b * CHW + i;                                  \
                    const SCALAR u = mem[at];                                               \
                    SCALAR through_spike = 0;                                                        \
                    if ((u - thresh) < interval && (thresh - u) < interval) {              \
                        through_spike = grad_spike[at] - carried * alpha * u;             \
                    }                                                                              \
                    carried = through_spike * beta + carried * alpha * (u <= thresh);    \
                    grad_spatial[at] = carried;                                                 \
                }                                                                                  \
            }                                                                                      \
        }                                                                                          \
    }                                                                                              \
                                                                                                   \
    /* full backward: mem_scratch (T*B*CHW elements) receives the recomputed membrane potential */ \
    void lif_oracle_backward_##SUFFIX(const SCALAR* spatial, const SCALAR* grad_spike,             \
                                      SCALAR* grad_spatial, SCALAR* mem_scratch, int64_t T,        \
                                      int64_t B, int64_t CHW, float alpha, float thresh,           \
                                      float beta, float interval) {                                \
        lif_oracle_forward_##SUFFIX(spatial, mem_scratch, (SCALAR*)0, T, B, CHW, alpha, thresh);   \
        lif_oracle_reverse_##SUFFIX(grad_spike, mem_scratch, grad_spatial, T, B, CHW, alpha,       \
                                    thresh, beta, interval);                                       \
    }

LIF_ORACLE_DEFINE(f32, float)
LIF_ORACLE_DEFINE(f64, double)

/*
 * Batch-norm + fire (fp32 and fp64), following the reference's kernels:
 *   forward  : snnlib/cuda/snn_kernel_fp.cu:179-209 (bn_fire_s_fp_kernel; scale = weight / sqrt(var + eps),
 *              ivar = scale / weight)
 *   backward : snnlib/cuda/snn_kernel_bp.cu:448-478 (bn_fire_u_fp_kernel; scale = weight * ivar),
 *              :560-609 (bn_fire_bp_wb_kernel: float partial sums per (c,h,w) over b and t, the two
 *              mean-type ones divided by T*B), :640-676 (bn_fire_bp_x_kernel), driven as in
 *              bn_fire_bp_cuda :680-750, where the per-(c,h,w) partials are reduced over the spatial
 *              positions with at::mean / at::sum.  That last reduction has no defined order in the
 *              reference; here it is done in double and rounded once.
 * Shapes: x, g, outputs [T, B, C, HW]; weight, bias, var, mean, ivar, grad_weight, grad_bias [C].
 * Parity pinning: tests/test_oracle_pinning.py checks these against autograd through
 * torch.nn.functional.batch_norm + the gold fire loop (oracle/gold_fire.py: gold_bn_fire) and
 * against closed forms (identity statistics reduce to the plain fire op; T=1 reduces to the
 * textbook batch-norm backward with a masked upstream gradient).
 */
#include <math.h>
#include <stdlib.h>

#define LIF_ORACLE_BN_DEFINE(SUFFIX, REAL, WIDE, SQRT) \
void lif_oracle_bn_forward_##SUFFIX(const REAL* spatial, const REAL* weight, const REAL* bias,                        \
                               const REAL* var, const REAL* mean, REAL* ivar, REAL* mem,                              \
                               REAL* spike, int64_t T, int64_t B, int64_t C, int64_t HW,                              \
                               float eps_bn, float alpha, float thresh) {                                             \
    const int64_t CHW = C * HW, step_stride = B * CHW;                                                                \
    for (int64_t i = 0; i < CHW; i++) {                                                                               \
        const int64_t c = i / HW;                                                                                     \
        const REAL m = mean[c];                                                                                       \
        const REAL scale = weight[c] / SQRT(var[c] + eps_bn);                                                         \
        const REAL shift = bias[c];                                                                                   \
        ivar[c] = scale / weight[c];                                                                                  \
        for (int64_t b = 0; b < B; b++) {                                                                             \
            REAL potential = 0;                                                                                       \
            int fired = 0;                                                                                            \
            for (int64_t t = 0; t < T; t++) {                                                                         \
                const int64_t at = t * step_stride + b * CHW + i;                                                     \
                potential = alpha * potential * (1 - fired) + (spatial[at] - m) * scale + shift;                      \
                fired = potential > thresh;                                                                           \
                if (mem) mem[at] = potential;                                                                         \
                if (spike) spike[at] = (REAL)fired;                                                                   \
            }                                                                                                         \
        }                                                                                                             \
    }                                                                                                                 \
}                                                                                                                     \
                                                                                                                      \
void lif_oracle_bn_backward_##SUFFIX(const REAL* spatial, const REAL* weight, const REAL* bias,                       \
                                const REAL* ivar, const REAL* mean, const REAL* grad_spike,                           \
                                REAL* grad_spatial, REAL* grad_weight, REAL* grad_bias,                               \
                                int64_t T, int64_t B, int64_t C, int64_t HW, float alpha,                             \
                                float thresh, float beta, float interval) {                                           \
    const int64_t CHW = C * HW, step_stride = B * CHW;                                                                \
    REAL* mem = (REAL*)malloc(sizeof(REAL) * (size_t)(T * step_stride));                                              \
    REAL* p_xhat = (REAL*)malloc(sizeof(REAL) * (size_t)CHW);                                                         \
    REAL* p_xhatx = (REAL*)malloc(sizeof(REAL) * (size_t)CHW);                                                        \
    REAL* p_w = (REAL*)malloc(sizeof(REAL) * (size_t)CHW);                                                            \
    REAL* p_b = (REAL*)malloc(sizeof(REAL) * (size_t)CHW);                                                            \
                                                                                                                      \
    /* recompute the membrane potential with scale = weight * ivar */                                                 \
    for (int64_t i = 0; i < CHW; i++) {                                                                               \
        const int64_t c = i / HW;                                                                                     \
        const REAL m = mean[c], scale = weight[c] * ivar[c], shift = bias[c];                                         \
        for (int64_t b = 0; b < B; b++) {                                                                             \
            REAL potential = 0;                                                                                       \
            int fired = 0;                                                                                            \
            for (int64_t t = 0; t < T; t++) {                                                                         \
                const int64_t at = t * step_stride + b * CHW + i;                                                     \
                potential = alpha * potential * (1 - fired) + (spatial[at] - m) * scale + shift;                      \
                fired = potential > thresh;                                                                           \
                mem[at] = potential;                                                                                  \
            }                                                                                                         \
        }                                                                                                             \
    }                                                                                                                 \
    /* partial sums per (c, h, w) */                                                                                  \
    for (int64_t i = 0; i < CHW; i++) {                                                                               \
        const int64_t c = i / HW;                                                                                     \
        const REAL m = mean[c], w = weight[c], iv = ivar[c];                                                          \
        REAL sum_b = 0, sum_w = 0, sum_xhat = 0, sum_xhatx = 0;                                                       \
        for (int64_t b = 0; b < B; b++) {                                                                             \
            REAL carried = 0;                                                                                         \
            for (int64_t t = T - 1; t >= 0; t--) {                                                                    \
                const int64_t at = t * step_stride + b * CHW + i;                                                     \
                const REAL u = mem[at];                                                                               \
                REAL through_spike = 0;                                                                               \
                if ((u - thresh) < interval && (thresh - u) < interval) {                                             \
                    through_spike = grad_spike[at] - carried * alpha * u;                                             \
                }                                                                                                     \
                carried = through_spike * beta + carried * alpha * (u <= thresh);                                     \
                const REAL x_bn = (spatial[at] - m) * iv;                                                             \
                sum_b += carried;                                                                                     \
                sum_w += carried * x_bn;                                                                              \
                sum_xhat += carried * w;                                                                              \
                sum_xhatx += carried * w * x_bn;                                                                      \
            }                                                                                                         \
        }                                                                                                             \
        p_b[i] = sum_b;                                                                                               \
        p_w[i] = sum_w;                                                                                               \
        p_xhat[i] = sum_xhat / (T * B);                                                                               \
        p_xhatx[i] = sum_xhatx / (T * B);                                                                             \
    }                                                                                                                 \
    /* reduce over the spatial positions of each channel; then the input gradient */                                  \
    for (int64_t c = 0; c < C; c++) {                                                                                 \
        WIDE acc_b = 0, acc_w = 0, acc_xhat = 0, acc_xhatx = 0;                                                       \
        for (int64_t k = 0; k < HW; k++) {                                                                            \
            acc_b += p_b[c * HW + k];                                                                                 \
            acc_w += p_w[c * HW + k];                                                                                 \
            acc_xhat += p_xhat[c * HW + k];                                                                           \
            acc_xhatx += p_xhatx[c * HW + k];                                                                         \
        }                                                                                                             \
        grad_bias[c] = (REAL)acc_b;                                                                                   \
        grad_weight[c] = (REAL)acc_w;                                                                                 \
        const REAL g_xhat = (REAL)(acc_xhat / (WIDE)HW);                                                              \
        const REAL g_xhatx = (REAL)(acc_xhatx / (WIDE)HW);                                                            \
        const REAL m = mean[c], w = weight[c], iv = ivar[c];                                                          \
        for (int64_t k = 0; k < HW; k++) {                                                                            \
            const int64_t i = c * HW + k;                                                                             \
            for (int64_t b = 0; b < B; b++) {                                                                         \
                REAL carried = 0;                                                                                     \
                for (int64_t t = T - 1; t >= 0; t--) {                                                                \
                    const int64_t at = t * step_stride + b * CHW + i;                                                 \
                    const REAL u = mem[at];                                                                           \
                    REAL through_spike = 0;                                                                           \
                    if ((u - thresh) < interval && (thresh - u) < interval) {                                         \
                        through_spike = grad_spike[at] - carried * alpha * u;                                         \
                    }                                                                                                 \
                    carried = through_spike * beta + carried * alpha * (u <= thresh);                                 \
                    grad_spatial[at] = carried * w * iv - iv * ((spatial[at] - m) * iv * g_xhatx + g_xhat);           \
                }                                                                                                     \
            }                                                                                                         \
        }                                                                                                             \
    }                                                                                                                 \
    free(mem); free(p_xhat); free(p_xhatx); free(p_w); free(p_b);                                                     \
}                                                                                                                     

/* fp32 as the reference trains; fp64 with the same loops in double (the reference's double dispatch keeps
 * the per-channel statistics in float temporaries, snnlib/cuda/snn_kernel_bp.cu:563; this restatement and
 * the device code do not narrow them).  Sums across positions: one precision up, rounded once. */
LIF_ORACLE_BN_DEFINE(f32, float, double, sqrtf)
LIF_ORACLE_BN_DEFINE(f64, double, long double, sqrt)

/*
 * Plain batch norm (no fire recurrence), fp32 and fp64, following the reference's kernels:
 *   forward  : snnlib/cuda/snn_kernel_fp.cu:102-121 (bn_fp_kernel: scale = weight / sqrt(var + eps),
 *              ivar = scale / weight, y = (x - mean) * scale + bias)
 *   backward : snnlib/cuda/snn_kernel_bp.cu:202-234 (bn_bp_wb_kernel: partial sums per (c,h,w) over b and
 *              t, t descending, the two mean-type ones divided by T*B), :263-283 (bn_bp_x_kernel),
 *              driven as in bn_bp_cuda :288-345 (at::mean / at::sum of the partials over the positions
 *              of a channel: no defined order in the reference; one precision up here, rounded once).
 * Parity pinning (tests/test_oracle_pinning.py): the forward against torch.nn.functional.batch_norm
 * with given statistics, the backward against autograd through the training-mode batch norm in
 * float64 (the textbook formula), and against hand-computed values on a two-channel case.
 */
#define LIF_ORACLE_PLAIN_BN_DEFINE(SUFFIX, REAL, WIDE, SQRT) \
void lif_oracle_plain_bn_forward_##SUFFIX(const REAL* x, const REAL* weight, const REAL* bias,                        \
                                     const REAL* var, const REAL* mean, REAL* ivar, REAL* y,                          \
                                     int64_t T, int64_t B, int64_t C, int64_t HW, float eps_bn) {                     \
    const int64_t CHW = C * HW, step_stride = B * CHW;                                                                \
    for (int64_t i = 0; i < CHW; i++) {                                                                               \
        const int64_t c = i / HW;                                                                                     \
        const REAL m = mean[c];                                                                                       \
        const REAL scale = weight[c] / SQRT(var[c] + eps_bn);                                                         \
        const REAL shift = bias[c];                                                                                   \
        ivar[c] = scale / weight[c];                                                                                  \
        for (int64_t b = 0; b < B; b++) {                                                                             \
            for (int64_t t = 0; t < T; t++) {                                                                         \
                const int64_t at = t * step_stride + b * CHW + i;                                                     \
                y[at] = (x[at] - m) * scale + shift;                                                                  \
            }                                                                                                         \
        }                                                                                                             \
    }                                                                                                                 \
}                                                                                                                     \
                                                                                                                      \
void lif_oracle_plain_bn_backward_##SUFFIX(const REAL* x, const REAL* weight, const REAL* ivar,                       \
                                      const REAL* mean, const REAL* grad_y, REAL* grad_x,                             \
                                      REAL* grad_weight, REAL* grad_bias, int64_t T, int64_t B,                       \
                                      int64_t C, int64_t HW) {                                                        \
    const int64_t CHW = C * HW, step_stride = B * CHW;                                                                \
    REAL* p_xhat = (REAL*)malloc(sizeof(REAL) * (size_t)CHW);                                                         \
    REAL* p_xhatx = (REAL*)malloc(sizeof(REAL) * (size_t)CHW);                                                        \
    REAL* p_w = (REAL*)malloc(sizeof(REAL) * (size_t)CHW);                                                            \
    REAL* p_b = (REAL*)malloc(sizeof(REAL) * (size_t)CHW);                                                            \
    for (int64_t i = 0; i < CHW; i++) {                                                                               \
        const int64_t c = i / HW;                                                                                     \
        const REAL m = mean[c], w = weight[c], iv = ivar[c];                                                          \
        REAL sum_b = 0, sum_w = 0, sum_xhat = 0, sum_xhatx = 0;                                                       \
        for (int64_t b = 0; b < B; b++) {                                                                             \
            for (int64_t t = T - 1; t >= 0; t--) {                                                                    \
                const int64_t at = t * step_stride + b * CHW + i;                                                     \
                const REAL gy = grad_y[at];                                                                           \
                const REAL x_bn = (x[at] - m) * iv;                                                                   \
                sum_b += gy;                                                                                          \
                sum_w += gy * x_bn;                                                                                   \
                sum_xhat += gy * w;                                                                                   \
                sum_xhatx += gy * w * x_bn;                                                                           \
            }                                                                                                         \
        }                                                                                                             \
        p_b[i] = sum_b;                                                                                               \
        p_w[i] = sum_w;                                                                                               \
        p_xhat[i] = sum_xhat / (T * B);                                                                               \
        p_xhatx[i] = sum_xhatx / (T * B);                                                                             \
    }                                                                                                                 \
    for (int64_t c = 0; c < C; c++) {                                                                                 \
        WIDE acc_b = 0, acc_w = 0, acc_xhat = 0, acc_xhatx = 0;                                                       \
        for (int64_t k = 0; k < HW; k++) {                                                                            \
            acc_b += p_b[c * HW + k];                                                                                 \
            acc_w += p_w[c * HW + k];                                                                                 \
            acc_xhat += p_xhat[c * HW + k];                                                                           \
            acc_xhatx += p_xhatx[c * HW + k];                                                                         \
        }                                                                                                             \
        grad_bias[c] = (REAL)acc_b;                                                                                   \
        grad_weight[c] = (REAL)acc_w;                                                                                 \
        const REAL g_xhat = (REAL)(acc_xhat / (WIDE)HW);                                                              \
        const REAL g_xhatx = (REAL)(acc_xhatx / (WIDE)HW);                                                            \
        const REAL m = mean[c], w = weight[c], iv = ivar[c];                                                          \
        for (int64_t k = 0; k < HW; k++) {                                                                            \
            const int64_t i = c * HW + k;                                                                             \
            for (int64_t b = 0; b < B; b++) {                                                                         \
                for (int64_t t = T - 1; t >= 0; t--) {                                                                \
                    const int64_t at = t * step_stride + b * CHW + i;                                                 \
                    grad_x[at] = grad_y[at] * w * iv - iv * ((x[at] - m) * iv * g_xhatx + g_xhat);                    \
                }                                                                                                     \
            }                                                                                                         \
        }                                                                                                             \
    }                                                                                                                 \
    free(p_xhat); free(p_xhatx); free(p_w); free(p_b);                                                                \
}

LIF_ORACLE_PLAIN_BN_DEFINE(f32, float, double, sqrtf)
LIF_ORACLE_PLAIN_BN_DEFINE(f64, double, long double, sqrt)
