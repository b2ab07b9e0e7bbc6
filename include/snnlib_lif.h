/*
 * snnlib_lif.h -- C ABI of libsnnlif_gfx950.so: the LIF "fire" forward / backward operators
 * of snnlib as hand-written HIP kernels for MI355X (gfx950).
 *
 * The library is the device-side half of the Python extension module `snnlib`
 * (reference binding table: snnlib/cuda/snn.cpp:798-830).  Every entry point below replaces one
 * host launcher of the reference; the `snnlib` module (csrc/snnlib_ext.cpp) allocates the output
 * tensors and forwards raw device pointers here, exactly where the reference's pybind forwarders
 * (snnlib/cuda/snn.cpp:11-17, 270-279) call their *_cuda launchers.
 *
 * Conventions shared by all entry points
 *   - Tensors are dense row-major [T, N]: T time steps, N = B*C*H*W (or B*C) neurons; element
 *     (t, n) sits at index t*N + n (reference indexing: snnlib/cuda/snn_kernel_fp.cu:45 with
 *     b*CHW + i folded into n -- neurons are independent, so the batch axis needs no loop).
 *     The batch-norm entry points need the channel of a neuron and therefore take the neuron axis
 *     as B, C, HW (N = B*C*HW, neuron (b, c, k) at (b*C + c)*HW + k); per-channel vectors are [C].
 *   - All pointers are DEVICE pointers on the current HIP device.  Inputs are only read; outputs
 *     are fully overwritten.  Nothing is allocated, nothing is kept between calls, so calls are
 *     thread-safe and may be issued on any stream (also under HIP graph capture: only kernel
 *     launches are enqueued).  Scratch memory, where an entry point needs any, is the caller's
 *     `workspace` argument.
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).  Calls only enqueue
 *     work; they never synchronise.
 *   - `dtype` selects the storage type of every tensor argument (see SNNLIF_DTYPE_*; the fire entry
 *     points also take a cache hint, SNNLIF_KEEP_SPATIAL or SNNLIF_STREAM_SPATIAL, or-ed into it).  Arithmetic
 *     is IEEE fp32 for F32 and BF16 storage and fp64 for F64 storage, in the reference's operation
 *     order, without fused multiply-add contraction.
 *   - Return value: SNNLIF_OK (0), a negative SNNLIF_ERR_* argument error, or a positive
 *     hipError_t value reported by the launch.  T == 0 or N == 0 is a successful no-op.
 */
#ifndef SNNLIB_LIF_H
#define SNNLIB_LIF_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* 2: cache hints in `dtype`, snnlif_fire_bp_strided, snnlif_bn_stats, snnlif_bn_fire_bp_static and
 *    SNNLIF_ERR_SCRATCH, the plain batch-norm entry points (snnlif_bn_fp, snnlif_bn_bp and its halves).
 *    A library of version 1 rejects hinted dtypes with SNNLIF_ERR_DTYPE and lacks those symbols.
 * 3: snnlif_channel_sum, snnlif_bn_stats_running, snnlif_bn_moments_finish. */
#define SNNLIF_ABI_VERSION 3

/* Storage types. */
#define SNNLIF_DTYPE_F32  0 /* float storage, fp32 arithmetic (the reference's training dtype) */
#define SNNLIF_DTYPE_F64  1 /* double storage, fp64 arithmetic */
#define SNNLIF_DTYPE_BF16 2 /* bfloat16 storage, fp32 arithmetic, round-to-nearest-even stores */

/*
 * Cache hints, or-ed into the `dtype` argument of snnlif_fire_s_fp, snnlif_fire_us_fp, snnlif_fire_bp,
 * snnlif_fire_bp_strided, snnlif_bn_fire_s_fp and snnlif_bn_fire_s_recompute (accepted and without effect
 * elsewhere; both at once: SNNLIF_ERR_DTYPE).  Results never depend on them.
 * No counterpart in the reference.
 *   SNNLIF_KEEP_SPATIAL    the caller will read `spatial` again soon -- the backward runs straight after
 *       the forward, or the same input current is used step after step.  `spatial` is loaded with the
 *       default cache policy, so that the 256 MB memory-side cache may keep it for its next reader,
 *       and the launch shape is the one that serves cache hits best.
 *   SNNLIF_STREAM_SPATIAL  it will not: `spatial` is streamed from HBM with the non-temporal hint like
 *       every other tensor, and the launch shape is the one that streams best.  This is the case of a
 *       network, where whole layers run between a layer's forward and its backward.
 *   neither                tensors of more than 32 MiB are streamed, smaller ones kept (a tensor that
 *       small is likely to be cache-resident whatever lies between its two readers).
 */
#define SNNLIF_KEEP_SPATIAL   0x100
#define SNNLIF_STREAM_SPATIAL 0x200

/* Return codes (hipError_t values are positive). */
#define SNNLIF_OK              0
#define SNNLIF_ERR_ARG        -1 /* NULL pointer with non-empty shape, negative T or N, T*N overflow */
#define SNNLIF_ERR_DTYPE      -2 /* dtype is not one of SNNLIF_DTYPE_* */
#define SNNLIF_ERR_WORKSPACE  -3 /* workspace missing or smaller than snnlif_fire_bp_workspace_bytes() */
#define SNNLIF_ERR_ALIGN      -4 /* a pointer is not aligned to its element size */
#define SNNLIF_ERR_SCRATCH    -6 /* shape needs more than SNNLIF_STATIC_SCRATCH_BYTES (snnlif_bn_fire_bp_static) */
#define SNNLIF_ERR_UNSUPPORTED -5 /* valid arguments this entry point does not implement (bf16 in the batch-norm ones) */

/* Every T up to this keeps the whole recomputed membrane potential in registers in the backward
 * (one kernel, 12 bytes per neuron-step in fp32) whatever the storage type; so do longer windows up to
 * 111 steps in fp32 (71 in fp64; bf16: up to 63, and multiples of 8 up to 104). */
#define SNNLIF_BP_FUSED_MAX_T 32
/* Largest T for which snnlif_fire_bp needs no workspace: up to here longer windows are processed
 * in register-sized segments whose boundary potentials live in LDS (16 bytes per neuron-step). */
#define SNNLIF_BP_NO_WORKSPACE_MAX_T 1024

/* Size of the fixed device array snnlif_bn_fire_bp_static works in (held once per GPU the library
 * runs on, for the life of the process). */
#define SNNLIF_STATIC_SCRATCH_BYTES (16u << 20)

/* ABI version of the loaded library (== SNNLIF_ABI_VERSION it was built with). */
int snnlif_abi_version(void);

/* Code-object target the kernels were compiled for ("gfx950"). */
const char* snnlif_target_arch(void);

/* Static, human-readable text for a return code of this library (negative codes) or of HIP
 * (positive codes). Never NULL. */
const char* snnlif_strerror(int code);

/*
 * Arms timing for the next snnlif_* entry point called from this thread (two hipEvent_t created with
 * timing enabled, passed as void*; either may be NULL; two NULLs disarm).
 * Entry points that launch one kernel (snnlif_fire_s_fp, snnlif_fire_us_fp, snnlif_fire_bp up to
 * SNNLIF_BP_NO_WORKSPACE_MAX_T steps, snnlif_bn_fire_s_fp, snnlif_bn_fire_s_recompute,
 * snnlif_bn_fire_bp_dist2) get the events attached to that dispatch -- `start_event` completes when
 * the kernel begins, `stop_event` when it has finished -- so hipEventElapsedTime(start, stop) is the
 * kernel's own duration, without the dispatch gaps an interval between two hipEventRecord markers
 * contains.  A start event costs a few microseconds of stream time per dispatch, a stop event alone
 * none: stop events on consecutive launches give completion-to-completion intervals that add up to the
 * wall clock (kernel duration plus dispatch gap), which is how bench.py times a saturated stream.  Entry points that launch several kernels (snnlif_bn_stats, snnlif_bn_fire_bp and its
 * _static and _dist1 forms, snnlif_fire_bp beyond SNNLIF_BP_NO_WORKSPACE_MAX_T steps) record
 * `start_event` on the stream before their first kernel and `stop_event` after their last: the whole
 * operation, gaps between its kernels included.
 * The arming is consumed by that one call whatever its outcome: a call that returns an argument error
 * or finds an empty shape leaves the events unrecorded and the timer disarmed.  Not meant for use under
 * HIP graph capture.  No counterpart in the reference (which has no timing hooks); for benchmarks and
 * profilers built on this ABI.
 */
int snnlif_time_next_kernel(void* start_event, void* stop_event);

/*
 * Fire forward: spikes only.
 *   u[t] = (alpha * u[t-1]) * (1 - s[t-1]) + x[t],   s[t] = u[t] > thresh,   u[-1] = s[-1] = 0
 *   spike[t] = s[t] as 0.0 / 1.0 in the storage dtype.
 * Replaces fire_s_fp_cuda + fire_s_fp_kernel (snnlib/cuda/snn_kernel_fp.cu:15-73), bound as
 * snnlib.fire_s_fp (snnlib/cuda/snn.cpp:11-17, 799).
 */
int snnlif_fire_s_fp(const void* spatial, void* spike, int dtype, int64_t T, int64_t N,
                     float alpha, float thresh, void* stream);

/*
 * Fire forward: membrane potential and spikes.  Same recurrence; mem[t] = u[t], spike[t] = s[t].
 * Either output may be NULL to skip it (mem only = the reference's fire_u_fp_kernel,
 * snnlib/cuda/snn_kernel_bp.cu:15-52; both = fire_us_fp_kernel, snnlib/cuda/snn_kernel_bp.cu:54-93,
 * which the reference launches from fire_fc_bp_cuda :1089 and fire_conv_bp_cuda :1372).
 */
int snnlif_fire_us_fp(const void* spatial, void* mem, void* spike, int dtype, int64_t T, int64_t N,
                      float alpha, float thresh, void* stream);

/*
 * Bytes of device workspace snnlif_fire_bp needs for this shape: 0 when
 * T <= SNNLIF_BP_NO_WORKSPACE_MAX_T (membrane potential recomputed on chip), otherwise
 * T*N*sizeof(arithmetic type) for the recomputed membrane potential (the reference always
 * allocates this tensor: `mem`, snnlib/cuda/snn_kernel_bp.cu:154).  Returns 0 for invalid arguments.
 */
size_t snnlif_fire_bp_workspace_bytes(int dtype, int64_t T, int64_t N);

/*
 * Fire backward: gradient of the loss w.r.t. the input current, given the input current saved by
 * the forward and the gradient w.r.t. the spikes.  Recomputes u[t] from `spatial`, then for
 * t = T-1 .. 0 with gu = 0 initially:
 *   gs = ((u[t]-thresh) < interval && (thresh-u[t]) < interval) ? grad_spike[t] - (gu*alpha)*u[t] : 0
 *   gu = gs*beta + (gu*alpha) * (u[t] <= thresh);      grad_spatial[t] = gu
 * Replaces fire_bp_cuda + fire_u_fp_kernel + fire_bp_kernel
 * (snnlib/cuda/snn_kernel_bp.cu:15-52, 95-168), bound as snnlib.fire_bp
 * (snnlib/cuda/snn.cpp:270-279, 813).
 * `workspace` may be NULL when snnlif_fire_bp_workspace_bytes() is 0; otherwise it must point to at
 * least that many bytes of device memory aligned to 16 bytes, private to this call until the
 * stream has run it.
 */
int snnlif_fire_bp(const void* spatial, const void* grad_spike, void* grad_spatial, int dtype,
                   int64_t T, int64_t N, float alpha, float thresh, float beta, float interval,
                   void* workspace, size_t workspace_bytes, void* stream);

/*
 * snnlif_fire_bp for a gradient whose time rows are `grad_row_stride` elements apart instead of N:
 *   grad_row_stride == N  the dense [T,N] gradient (exactly snnlif_fire_bp);
 *   grad_row_stride == 0  one row of N values that stands for every time step: what autograd hands to
 *                         the fire op after `spike.mean(dim=0)` or `spike.sum(dim=0)` (a stride-0
 *                         expansion over time; the pattern of the reference's own snnlib/test_fire.py:22-30).
 *                         The reference's binding makes such a gradient dense first
 *                         (snnlib/cuda/snn.cpp:270-279 requires contiguous inputs); here it is read in
 *                         place, N values instead of T*N;
 *   grad_row_stride >  N  rows of a wider tensor.
 * Any other value (negative, or 0 < stride < N: overlapping rows) is SNNLIF_ERR_ARG.  `grad_spatial` is
 * dense and must not overlap `grad_spike`.  Everything else as snnlif_fire_bp; same results bit for bit
 * as snnlif_fire_bp on the gradient made dense.
 */
int snnlif_fire_bp_strided(const void* spatial, const void* grad_spike, void* grad_spatial, int dtype,
                           int64_t T, int64_t N, int64_t grad_row_stride, float alpha, float thresh,
                           float beta, float interval, void* workspace, size_t workspace_bytes,
                           void* stream);

/* Bytes of device workspace snnlif_bn_stats needs (partial sums: two doubles per wavefront when
 * HW >= 32, two per (row slice, channel position) otherwise).  0 for invalid arguments. */
size_t snnlif_bn_stats_workspace_bytes(int dtype, int64_t T, int64_t B, int64_t C, int64_t HW);

/*
 * Per-channel batch statistics of a [T, B, C, HW] activation over (T, B, HW), fp32 or fp64 (bf16:
 * SNNLIF_ERR_UNSUPPORTED); `mean` and `var` are [C] of the storage type.
 *   raw_moments == 0:  mean[c] = E[x],  var[c] = E[(x - mean[c])^2]  (biased: divided by T*B*HW)
 *   raw_moments != 0:  mean[c] = E[x],  var[c] = E[x^2]              (what a sharded batch all-reduces)
 * Replaces the framework reductions the reference's layers run before every batch-norm op:
 * torch.var_mean(x, dim_bn, unbiased=False) (snnlib/example/snnlib_op.py:44, 78, 122, 184) and torch.mean(x), torch.mean(x**2) of the sharded layers (snnlib/example/snnlib_op.py:265-266,
 * 328-329, 388-389).  One pass over the tensor; sums are taken of x minus the channel's first element, in
 * double precision throughout, and added up per channel in a fixed order (reproducible results).  `spatial` is
 * loaded with the default cache policy, so a tensor that fits the memory-side cache is still there
 * for the batch-norm op that follows.  T, B or HW of zero with C > 0 is SNNLIF_ERR_ARG (a channel
 * without elements has no statistics).  `workspace`: snnlif_bn_stats_workspace_bytes() bytes, 16-byte
 * aligned, private to the call until the stream has run it.
 */
int snnlif_bn_stats(const void* spatial, void* mean, void* var, int dtype, int64_t T, int64_t B,
                    int64_t C, int64_t HW, int raw_moments, void* workspace, size_t workspace_bytes,
                    void* stream);

/*
 * snnlif_bn_stats (mean and biased variance) together with the layer's running statistics: what the
 * reference's layers do after torch.var_mean in training mode (snnlib/example/snnlib_op.py:44-46, 78-80,
 * 122-124, 184-186),
 *   new_running_mean[c] = (running_mean[c] * keep) + (mean[c] * gain_mean)
 *   new_running_var[c]  = (running_var[c]  * keep) + (var[c]  * gain_var)
 * with keep = 0.9, gain_mean = 0.1, gain_var = 0.1 * n / (n - 1) there.  The factors are rounded to the
 * storage type once and every product and sum is rounded in it, so the results carry the bits of the
 * framework's element-wise expression; they are formed in the last step of the statistics pass (no
 * further kernel: six small launches per layer and step less).  new_running_* may alias running_*.
 * Arguments, workspace and errors as for snnlif_bn_stats; all seven tensors are required.
 */
int snnlif_bn_stats_running(const void* spatial, void* mean, void* var, const void* running_mean,
                            const void* running_var, void* new_running_mean, void* new_running_var,
                            double keep, double gain_mean, double gain_var, int dtype, int64_t T,
                            int64_t B, int64_t C, int64_t HW, void* workspace, size_t workspace_bytes,
                            void* stream);

/*
 * Statistics of a batch sharded over `world_size` ranks from its all-reduced raw moments, as the
 * reference's sharded layers form them (snnlib/example/snnlib_op.py:271-275, 334-338, 394-398):
 *   mean[c] = first[c] / world_size;   var[c] = second[c] / world_size - mean[c]^2
 * and, when the four running pointers are given, the running pair as in snnlif_bn_stats_running (keep =
 * 0.95, gains 0.05 and 0.05 * n / (n - 1) there).  The division is a product with 1 / world_size rounded
 * to the storage type and the square a product, as the framework evaluates them: same bits as the
 * reference's ten small element-wise launches, in one.  [C] vectors of fp32 or fp64; world_size >= 1.
 */
int snnlif_bn_moments_finish(const void* first, const void* second, void* mean, void* var,
                             const void* running_mean, const void* running_var,
                             void* new_running_mean, void* new_running_var, double world_size,
                             double keep, double gain_mean, double gain_var, int dtype, int64_t C,
                             void* stream);

/*
 * Per-channel sum of a [T, B, C, HW] gradient over (T, B, HW), fp32 or fp64 (bf16:
 * SNNLIF_ERR_UNSUPPORTED); `sum` is [C] of the storage type.  The bias gradient of the layers that end
 * in a convolution: replaces at::sum(grad_conv, dim_conv) in bn_fire_conv_bp_cuda, its _dist2 form,
 * fire_conv_bp_cuda and conv_bp_cuda (snnlib/cuda/snn_kernel_bp.cu:1261, 1338, 1401, 1435) for the
 * dim_conv the reference's layers pass, (0, 1, 3, 4), every axis but the channel's (snnlib/example/snnlib_func.py:182, 215, 247, 357).
 * The pass of snnlif_bn_stats with another last step: summed in double precision in a fixed order
 * (reproducible), `grad` loaded with the default cache policy.  T, B or HW of zero with C > 0 is
 * SNNLIF_ERR_ARG.  `workspace`: snnlif_bn_stats_workspace_bytes() bytes, 16-byte aligned, private to
 * the call until the stream has run it.
 */
int snnlif_channel_sum(const void* grad, void* sum, int dtype, int64_t T, int64_t B, int64_t C,
                       int64_t HW, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Batch-norm + fire forward (dtype SNNLIF_DTYPE_F32 or SNNLIF_DTYPE_F64, which also is the type of the
 * per-channel vectors; SNNLIF_DTYPE_BF16: SNNLIF_ERR_UNSUPPORTED).  In fp64 the per-channel statistics
 * stay in double (the reference's double dispatch narrows them to float inside its kernels,
 * snnlib/cuda/snn_kernel_fp.cu:184).
 * Tensors are [T, B, C, HW] (HW = 1 for [T, B, C]); weight, bias, var, mean, ivar are [C].
 *   scale[c] = weight[c] / sqrt(var[c] + eps);   ivar[c] = scale[c] / weight[c]
 *   u[t] = (alpha*u[t-1])*(1-s[t-1]) + (x[t] - mean[c])*scale[c] + bias[c];   s[t] = u[t] > thresh
 * Replaces bn_fire_s_fp_cuda + bn_fire_s_fp_kernel (snnlib/cuda/snn_kernel_fp.cu:157-240), bound as
 * snnlib.bn_fire_s_fp (snnlib/cuda/snn.cpp:800).
 */
int snnlif_bn_fire_s_fp(const void* spatial, const void* weight, const void* bias, const void* var,
                        const void* mean, void* ivar, void* spike, int dtype, int64_t T, int64_t B,
                        int64_t C, int64_t HW, float eps, float alpha, float thresh, void* stream);

/*
 * Spikes of the batch-norm + fire layer recomputed from saved statistics, the way the backward of
 * the fused layers sees them: scale[c] = weight[c] * ivar[c] (not weight / sqrt(var + eps)), same
 * recurrence as snnlif_bn_fire_s_fp, fp32 or fp64.  Replaces bn_fire_us_fp_kernel
 * (snnlib/cuda/snn_kernel_bp.cu:481-530) as used by bn_fire_fc_bp_cuda (:890) and bn_fire_conv_bp_cuda
 * (:1215); the membrane potential it also writes there is not needed here because
 * snnlif_bn_fire_bp recomputes it in registers.
 */
int snnlif_bn_fire_s_recompute(const void* spatial, const void* weight, const void* bias,
                               const void* ivar, const void* mean, void* spike, int dtype, int64_t T,
                               int64_t B, int64_t C, int64_t HW, float alpha, float thresh,
                               void* stream);

/* Bytes of device workspace snnlif_bn_fire_bp needs: two partial sums of the storage type per
 * wavefront of sweep 1 (ceil(HW/64) wavefronts per (batch entry, channel) plane) when HW >= 32, two
 * per neuron plus their batch-sliced column sums otherwise, per-channel staging, and for
 * T > SNNLIF_BP_NO_WORKSPACE_MAX_T one membrane potential per 32-step segment and neuron.
 * 0 for invalid arguments. */
size_t snnlif_bn_fire_bp_workspace_bytes(int dtype, int64_t T, int64_t B, int64_t C, int64_t HW);

/*
 * Batch-norm + fire backward (fp32 or fp64; any T; windows longer than SNNLIF_BP_FUSED_MAX_T are cut
 * into 32-step segments and read x twice per sweep, with the membrane potential at the segment
 * boundaries in LDS up to SNNLIF_BP_NO_WORKSPACE_MAX_T steps and in device memory beyond).
 * With u recomputed from scale[c] = weight[c]*ivar[c], gy the fire reverse chain (see
 * snnlif_fire_bp), xhat = (x - mean[c])*ivar[c] and M = T*B*HW:
 *   grad_bias[c] = sum gy;   grad_weight[c] = sum gy*xhat
 *   grad_spatial = (gy*weight[c])*ivar[c]
 *                  - ivar[c]*((xhat*(weight[c]*grad_weight[c]/M)) + weight[c]*grad_bias[c]/M)
 * Replaces bn_fire_bp_cuda and its three kernels (snnlib/cuda/snn_kernel_bp.cu:432-479, 533-750),
 * bound as snnlib.bn_fire_bp (snnlib/cuda/snn.cpp:814).  `workspace` must hold
 * snnlif_bn_fire_bp_workspace_bytes() bytes, 16-byte aligned, private to the call until the
 * stream has run it.  Per-channel sums are formed in a fixed order: results are reproducible.
 */
int snnlif_bn_fire_bp(const void* spatial, const void* weight, const void* bias, const void* ivar,
                      const void* mean, const void* grad_spike, void* grad_spatial,
                      void* grad_weight, void* grad_bias, int dtype, int64_t T, int64_t B, int64_t C,
                      int64_t HW, float alpha, float thresh, float beta, float interval,
                      void* workspace, size_t workspace_bytes, void* stream);

/*
 * snnlif_bn_fire_bp for callers that can neither allocate device memory nor hand in a workspace: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference.  Same arguments, checks, kernels and results (bit for bit)
 * as snnlif_bn_fire_bp, minus the workspace: the partial sums live in a fixed device array of
 * SNNLIF_STATIC_SCRATCH_BYTES that the library holds once per GPU.  Shapes for which
 * snnlif_bn_fire_bp_workspace_bytes() exceeds that size return SNNLIF_ERR_SCRATCH and launch nothing
 * (at fp32: more than about 2 million wavefront partials B*C*ceil(HW/64) when HW >= 32, or about
 * 2 million neurons B*C*HW when HW < 32).  The call allocates and frees nothing.  The first call made
 * with a given device current resolves that device's copy of the array (make it outside graph
 * capture); all calls on one GPU share the array, so two calls whose kernels may overlap on that GPU
 * (different streams without an ordering between them) race -- order them.  Nothing needs to be
 * cleared between calls: every value read from the array is written earlier in the same call.
 */
int snnlif_bn_fire_bp_static(const void* spatial, const void* weight, const void* bias,
                             const void* ivar, const void* mean, const void* grad_spike,
                             void* grad_spatial, void* grad_weight, void* grad_bias, int dtype,
                             int64_t T, int64_t B, int64_t C, int64_t HW, float alpha, float thresh,
                             float beta, float interval, void* stream);

/*
 * The same backward in the two halves that a batch sharded over several GPUs runs on either side of
 * an all-reduce (fp32 or fp64, any T, shapes and workspace as snnlif_bn_fire_bp; B is the local batch).
 *
 * snnlif_bn_fire_bp_dist1: the local parameter gradients and the local per-channel means
 *   mean_gxhat[c]  = weight[c] * (sum gy)      / (T*B*HW)
 *   mean_gxhatx[c] = weight[c] * (sum gy*xhat) / (T*B*HW)
 * Replaces bn_fire_bp_cuda_dist1 (snnlib/cuda/snn_kernel_bp.cu:753-809), bound as
 * snnlib.bn_fire_bp_dist1 (snnlib/cuda/snn.cpp:826) and run inside bn_fire_fc_bp_cuda_dist1 (:966-1061)
 * and bn_fire_conv_bp_cuda_dist1 (:1265-1340).
 *
 * snnlif_bn_fire_bp_dist2: the input gradient from the two means averaged over all ranks,
 *   grad_spatial = (gy*weight[c])*ivar[c] - ivar[c]*((xhat*grad_xhatx[c]) + grad_xhat[c])
 * Needs no workspace (beyond SNNLIF_BP_NO_WORKSPACE_MAX_T steps it parks the segment boundary potentials in
 * rows of grad_spatial that it overwrites later in the same call).  Replaces bn_fire_bp_cuda_dist2 (snnlib/cuda/snn_kernel_bp.cu:811-854), bound
 * as snnlib.bn_fire_bp_dist2 (snnlib/cuda/snn.cpp:827).
 *
 * dist1 followed by dist2 on the same arrays is snnlif_bn_fire_bp, bit for bit.  The all-reduce
 * between them is the caller's.
 */
int snnlif_bn_fire_bp_dist1(const void* spatial, const void* weight, const void* bias,
                            const void* ivar, const void* mean, const void* grad_spike,
                            void* mean_gxhat, void* mean_gxhatx, void* grad_weight, void* grad_bias,
                            int dtype, int64_t T, int64_t B, int64_t C, int64_t HW, float alpha,
                            float thresh, float beta, float interval, void* workspace,
                            size_t workspace_bytes, void* stream);

int snnlif_bn_fire_bp_dist2(const void* spatial, const void* weight, const void* bias,
                            const void* ivar, const void* mean, const void* grad_spike,
                            const void* grad_xhat, const void* grad_xhatx, void* grad_spatial,
                            int dtype, int64_t T, int64_t B, int64_t C, int64_t HW, float alpha,
                            float thresh, float beta, float interval, void* stream);

/*
 * Plain batch norm of a [T, B, C, HW] activation with given per-channel statistics (fp32 or fp64; bf16:
 * SNNLIF_ERR_UNSUPPORTED); weight, bias, var, mean, ivar are [C].
 *   scale[c] = weight[c] / sqrt(var[c] + eps);   ivar[c] = scale[c] / weight[c]
 *   y_bn = (x_bn - mean[c]) * scale[c] + bias[c]
 * One pass, 8 bytes per element.  Replaces bn_fp_cuda + bn_fp_kernel (snnlib/cuda/snn_kernel_fp.cu:81-150),
 * bound as snnlib.bn_fp (snnlib/cuda/snn.cpp:30-40).
 */
int snnlif_bn_fp(const void* x_bn, const void* weight, const void* bias, const void* var,
                 const void* mean, void* ivar, void* y_bn, int dtype, int64_t T, int64_t B, int64_t C,
                 int64_t HW, float eps, void* stream);

/* Bytes of device workspace snnlif_bn_bp and snnlif_bn_bp_dist1 need: two partial sums of the storage
 * type per wavefront and row slice of the sums pass when HW >= 32, two per column and row slice
 * otherwise, and two per-channel means.  0 for invalid arguments. */
size_t snnlif_bn_bp_workspace_bytes(int dtype, int64_t T, int64_t B, int64_t C, int64_t HW);

/*
 * Plain batch-norm backward with the statistics the forward saved (fp32 or fp64).  With
 * xhat = (x_bn - mean[c])*ivar[c] and M = T*B*HW:
 *   grad_bias[c] = sum grad_y;   grad_weight[c] = sum grad_y*xhat
 *   grad_x_bn = (grad_y*weight[c])*ivar[c]
 *               - ivar[c]*((xhat*(weight[c]*grad_weight[c]/M)) + weight[c]*grad_bias[c]/M)
 * Two passes over (x_bn, grad_y) around a per-channel reduction in a fixed order (reproducible
 * results): 20 bytes per element.  Replaces bn_bp_cuda with bn_bp_wb_kernel and bn_bp_x_kernel
 * (snnlib/cuda/snn_kernel_bp.cu:176-345), bound as snnlib.bn_bp (snnlib/cuda/snn.cpp:293-304).  `workspace`:
 * snnlif_bn_bp_workspace_bytes() bytes, 16-byte aligned, private to the call until the stream has run it.
 */
int snnlif_bn_bp(const void* x_bn, const void* weight, const void* ivar, const void* mean,
                 const void* grad_y_bn, void* grad_x_bn, void* grad_weight, void* grad_bias, int dtype,
                 int64_t T, int64_t B, int64_t C, int64_t HW, void* workspace, size_t workspace_bytes,
                 void* stream);

/*
 * The two halves of snnlif_bn_bp for a batch sharded over several GPUs (B is the local batch):
 * snnlif_bn_bp_dist1 leaves the local parameter gradients and the local means
 *   mean_gxhat[c] = weight[c]*(sum grad_y)/(T*B*HW),  mean_gxhatx[c] = weight[c]*(sum grad_y*xhat)/(T*B*HW)
 * (8 bytes per element); snnlif_bn_bp_dist2 forms the input gradient from the two means averaged over
 * all ranks (12 bytes per element, no workspace).  dist1 followed by dist2 on the same arrays is
 * snnlif_bn_bp, bit for bit; the all-reduce between them is the caller's.  Replace bn_bp_cuda_dist1 and
 * bn_bp_cuda_dist2 (snnlib/cuda/snn_kernel_bp.cu:348-425), bound as snnlib.bn_bp_dist1 / bn_bp_dist2
 * (snnlib/cuda/snn.cpp:317-355).
 */
int snnlif_bn_bp_dist1(const void* x_bn, const void* weight, const void* ivar, const void* mean,
                       const void* grad_y_bn, void* mean_gxhat, void* mean_gxhatx, void* grad_weight,
                       void* grad_bias, int dtype, int64_t T, int64_t B, int64_t C, int64_t HW,
                       void* workspace, size_t workspace_bytes, void* stream);

int snnlif_bn_bp_dist2(const void* x_bn, const void* weight, const void* ivar, const void* mean,
                       const void* grad_y_bn, const void* grad_xhat, const void* grad_xhatx,
                       void* grad_x_bn, int dtype, int64_t T, int64_t B, int64_t C, int64_t HW,
                       void* stream);

#ifdef __cplusplus
}
#endif

#endif /* SNNLIB_LIF_H */
