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
