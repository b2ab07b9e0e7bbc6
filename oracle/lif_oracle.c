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
 * Batch-norm + fire (fp32), following the reference's kernels:
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

void lif_oracle_bn_forward_f32(const float* spatial, const float* weight, const float* bias,
                               const float* var, const float* mean, float* ivar, float* mem,
                               float* spike, int64_t T, int64_t B, int64_t C, int64_t HW,
                               float eps_bn, float alpha, float thresh) {
    const int64_t CHW = C * HW, step_stride = B * CHW;
    for (int64_t i = 0; i < CHW; i++) {
        const int64_t c = i / HW;
        const float m = mean[c];
        const float scale = weight[c] / sqrtf(var[c] + eps_bn);
        const float shift = bias[c];
        ivar[c] = scale / weight[c];
        for (int64_t b = 0; b < B; b++) {
            float potential = 0;
            int fired = 0;
            for (int64_t t = 0; t < T; t++) {
                const int64_t at = t * step_stride + b * CHW + i;
                potential = alpha * potential * (1 - fired) + (spatial[at] - m) * scale + shift;
                fired = potential > thresh;
                if (mem) mem[at] = potential;
                if (spike) spike[at] = (float)fired;
            }
        }
    }
}

void lif_oracle_bn_backward_f32(const float* spatial, const float* weight, const float* bias,
                                const float* ivar, const float* mean, const float* grad_spike,
                                float* grad_spatial, float* grad_weight, float* grad_bias,
                                int64_t T, int64_t B, int64_t C, int64_t HW, float alpha,
                                float thresh, float beta, float interval) {
    const int64_t CHW = C * HW, step_stride = B * CHW;
    float* mem = (float*)malloc(sizeof(float) * (size_t)(T * step_stride));
    float* p_xhat = (float*)malloc(sizeof(float) * (size_t)CHW);
    float* p_xhatx = (float*)malloc(sizeof(float) * (size_t)CHW);
    float* p_w = (float*)malloc(sizeof(float) * (size_t)CHW);
    float* p_b = (float*)malloc(sizeof(float) * (size_t)CHW);

    /* recompute the membrane potential with scale = weight * ivar */
    for (int64_t i = 0; i < CHW; i++) {
        const int64_t c = i / HW;
        const float m = mean[c], scale = weight[c] * ivar[c], shift = bias[c];
        for (int64_t b = 0; b < B; b++) {
            float potential = 0;
            int fired = 0;
            for (int64_t t = 0; t < T; t++) {
                const int64_t at = t * step_stride + b * CHW + i;
                potential = alpha * potential * (1 - fired) + (spatial[at] - m) * scale + shift;
                fired = potential > thresh;
                mem[at] = potential;
            }
        }
    }
    /* partial sums per (c, h, w) */
    for (int64_t i = 0; i < CHW; i++) {
        const int64_t c = i / HW;
        const float m = mean[c], w = weight[c], iv = ivar[c];
        float sum_b = 0, sum_w = 0, sum_xhat = 0, sum_xhatx = 0;
        for (int64_t b = 0; b < B; b++) {
            float carried = 0;
            for (int64_t t = T - 1; t >= 0; t--) {
                const int64_t at = t * step_stride + b * CHW + i;
                const float u = mem[at];
                float through_spike = 0;
                if ((u - thresh) < interval && (thresh - u) < interval) {
                    through_spike = grad_spike[at] - carried * alpha * u;
                }
                carried = through_spike * beta + carried * alpha * (u <= thresh);
                const float x_bn = (spatial[at] - m) * iv;
                sum_b += carried;
                sum_w += carried * x_bn;
                sum_xhat += carried * w;
                sum_xhatx += carried * w * x_bn;
            }
        }
        p_b[i] = sum_b;
        p_w[i] = sum_w;
        p_xhat[i] = sum_xhat / (T * B);
        p_xhatx[i] = sum_xhatx / (T * B);
    }
    /* reduce over the spatial positions of each channel; then the input gradient */
    for (int64_t c = 0; c < C; c++) {
        double acc_b = 0, acc_w = 0, acc_xhat = 0, acc_xhatx = 0;
        for (int64_t k = 0; k < HW; k++) {
            acc_b += p_b[c * HW + k];
            acc_w += p_w[c * HW + k];
            acc_xhat += p_xhat[c * HW + k];
            acc_xhatx += p_xhatx[c * HW + k];
        }
        grad_bias[c] = (float)acc_b;
        grad_weight[c] = (float)acc_w;
        const float g_xhat = (float)(acc_xhat / (double)HW);
        const float g_xhatx = (float)(acc_xhatx / (double)HW);
        const float m = mean[c], w = weight[c], iv = ivar[c];
        for (int64_t k = 0; k < HW; k++) {
            const int64_t i = c * HW + k;
            for (int64_t b = 0; b < B; b++) {
                float carried = 0;
                for (int64_t t = T - 1; t >= 0; t--) {
                    const int64_t at = t * step_stride + b * CHW + i;
                    const float u = mem[at];
                    float through_spike = 0;
                    if ((u - thresh) < interval && (thresh - u) < interval) {
                        through_spike = grad_spike[at] - carried * alpha * u;
                    }
                    carried = through_spike * beta + carried * alpha * (u <= thresh);
                    grad_spatial[at] = carried * w * iv - iv * ((spatial[at] - m) * iv * g_xhatx + g_xhat);
                }
            }
        }
    }
    free(mem); free(p_xhat); free(p_xhatx); free(p_w); free(p_b);
}
