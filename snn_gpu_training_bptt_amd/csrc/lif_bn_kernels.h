// Batch-norm + LIF fire kernels (F = float or double; one neuron per lane) for MI355X: the
// per-channel affine of a batch norm is applied to the input current inside the fire recurrence,
// forward and backward.
//
// Reference: snnlib/cuda/snn_kernel_fp.cu:157-240 (bn_fire_s_fp_kernel + launcher) and
// snnlib/cuda/snn_kernel_bp.cu:432-479 (bn_fire_u_fp_kernel), :533-610 (bn_fire_bp_wb_kernel),
// :613-677 (bn_fire_bp_x_kernel), :680-750 (bn_fire_bp_cuda).
//
//   forward   y = (x - mean[c]) * (weight[c] / sqrt(var[c] + eps)) + bias[c]   folded as
//             u = (alpha*u)*(1-s) + (x - mean[c]) * scale[c] + bias[c];  s = u > thresh
//             ivar[c] = scale[c] / weight[c]
//   backward  gy[t] = the fire reverse chain on u recomputed with scale[c] = weight[c] * ivar[c]
//             xhat  = (x - mean[c]) * ivar[c]
//             grad_bias[c]   = sum gy            grad_weight[c] = sum gy * xhat      (over T,B,H,W)
//             gxhat[c]  = weight[c] * grad_bias[c]   / M      gxhatx[c] = weight[c] * grad_weight[c] / M
//             gx = (gy * weight[c]) * ivar[c] - ivar[c] * ((xhat * gxhatx[c]) + gxhat[c]),  M = T*B*H*W
//
// Mapping.  Same lanes as the plain fire kernels (one neuron per lane, time in registers).  The
// backward needs per-channel sums over everything before any input gradient can be formed, so it
// is two sweeps over (x, g) with a reduction between them:
//   1. lif_bn_backward_partial_kernel: reverse chain per neuron, sums over its T steps, and -- for
//      planes of at least 32 positions, over which wavefronts are laid so that all 64 lanes share a
//      channel -- over the wavefront by shuffles: two floats per wavefront (per neuron otherwise);
//   2. bn_channel_reduce_finalize_kernel (or bn_column_reduce_kernel + bn_channel_finalize_kernel
//      for per-neuron partials): per-channel sums of those partials (wavefront shuffles, then LDS
//      across the waves of a workgroup, for the per-wavefront form; column sums over the batch
//      for the per-neuron form), in an order fixed by the launch geometry -> bit-reproducible results;
//   3. lif_bn_backward_input_kernel: the chain again (x and g re-read: 8 B per neuron-step, the
//      same as storing and re-loading gy would cost) and the input gradient.
// Windows of more than 32 steps run both sweeps in 32-step segments with the membrane potential at
// the segment boundaries kept aside (bn_reverse_segmented): x is then read twice per sweep.  Up to
// 1024 steps the boundary values live in LDS; beyond, sweep 1 keeps them in its workspace and sweep 2
// in rows of the input gradient that it has not written yet (a lane only ever touches its own column).
// HBM traffic: forward 8 B, backward 20 B (+ at most 16/T B) per neuron-step up to 32 steps, 28 B
// beyond; the reference moves 8 and 36.
#ifndef SNNLIF_LIF_BN_KERNELS_H
#define SNNLIF_LIF_BN_KERNELS_H

#include "lif_bn.h"
#include "lif_kernels.h"

namespace snnlif {

__device__ __forceinline__ float real_sqrt(float v) { return sqrtf(v); }
__device__ __forceinline__ double real_sqrt(double v) { return sqrt(v); }


// Channel of a neuron column in a [B, C, HW] neuron axis.
__device__ __forceinline__ int channel_of(int64_t col, int64_t C, int64_t HW, bool small) {
    if (small) {  // everything fits 32 bits: cheap unsigned division
        const uint32_t q = static_cast<uint32_t>(col) / static_cast<uint32_t>(HW);
        return static_cast<int>(q % static_cast<uint32_t>(C));
    }
    return static_cast<int>((col / HW) % C);
}

// ---------------------------------------------------------------------------------------------
// Forward: spikes.  FROM_IVAR = false: `stat` is the variance, scale = weight / sqrt(var + eps), and
// the inverse standard deviation scale / weight is published per channel (the layer's forward).
// FROM_IVAR = true: `stat` is that inverse standard deviation, scale = weight * ivar, nothing is
// published (how the backward of the fused layers recomputes the spikes, as the reference's
// bn_fire_us_fp_kernel does, snnlib/cuda/snn_kernel_bp.cu:481-530).
// ---------------------------------------------------------------------------------------------
// KEEP: x is loaded with the default cache policy (a caller that reads x again soon), otherwise with
// the non-temporal hint like the spikes.  Cold, right after the statistics pass over the same x, the
// streamed form measures 79-83 % of the HBM peak on 128-256 MiB tensors where the kept one reaches
// 64-78 %; all 8 wavefronts per SIMD resident serve both best.
#ifndef SNNLIF_BN_FWD_WAVES
#define SNNLIF_BN_FWD_WAVES 8
#endif
template <typename F, int TC, bool MULTI, bool FROM_IVAR, bool KEEP>
__global__ void __launch_bounds__(kFwdBlock) SNNLIF_WAVES_PER_SIMD(SNNLIF_BN_FWD_WAVES)
lif_bn_forward_kernel(const F* __restrict__ x, const F* __restrict__ weight,
                      const F* __restrict__ bias, const F* __restrict__ stat,
                      const F* __restrict__ mean, F* __restrict__ ivar,
                      F* __restrict__ spike, int T, int64_t N, int64_t C, int64_t HW, F eps,
                      F alpha, F thresh) {
    const bool small = N <= 0xffffffffll;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t col = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; col < N;
         col += stride) {
        const int c = channel_of(col, C, HW, small);
        const F m = mean[c];
        const F wgt = weight[c];
        const F scale = FROM_IVAR ? wgt * stat[c] : wgt / real_sqrt(stat[c] + eps);
        const F b = bias[c];
        // first neuron of the channel in batch entry 0 publishes the channel's ivar
        if (!FROM_IVAR && col == static_cast<int64_t>(c) * HW) ivar[c] = scale / wgt;

        F u = F(0), s = F(0);
        Pack<F, 1> cur[TC];
        Pack<F, 1> nxt[MULTI ? TC : 1];
#pragma unroll
        for (int k = 0; k < TC; ++k) {
            if (k < T) cur[k] = load_pack<F, 1, !KEEP>(x + static_cast<int64_t>(k) * N + col);
        }
        for (int t0 = 0; t0 < T; t0 += TC) {
            if (MULTI && t0 + TC < T) {
#pragma unroll
                for (int k = 0; k < TC; ++k) {
                    const int t = t0 + TC + k;
                    if (t < T)
                        nxt[MULTI ? k : 0] =
                            load_pack<F, 1, !KEEP>(x + static_cast<int64_t>(t) * N + col);
                }
            }
#pragma unroll
            for (int k = 0; k < TC; ++k) {
                const int t = t0 + k;
                if (t < T) {
                    u = (alpha * u) * (F(1) - s) + (cur[k].e[0] - m) * scale + b;
                    s = (u > thresh) ? F(1) : F(0);
                    Pack<F, 1> so;
                    so.e[0] = s;
                    store_pack<F, 1>(spike + static_cast<int64_t>(t) * N + col, so);
                }
            }
            if (!MULTI) break;
            if (t0 + TC < T) {
#pragma unroll
                for (int k = 0; k < TC; ++k) cur[k] = nxt[MULTI ? k : 0];
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Shared front half of both backward sweeps, for one register window of at most TW steps whose
// first row the pointers x / g name: load the window, recompute u from the state (uc, sc) carried
// in from the step before it, run the reverse chain from the gradient gu carried in from the step
// after it.  Calls emit(t, gy, x_t) for t = rows-1 .. 0 (t counts from the window's first row).  On
// exit uc / sc are the state after the window and gu the gradient at its first step.
// ---------------------------------------------------------------------------------------------
template <typename F, int TW, bool EXACT, typename Emit>
__device__ __forceinline__ void bn_reverse_window(const F* __restrict__ x,
                                                  const F* __restrict__ g, int rows, int64_t N,
                                                  int64_t col, F m, F scale, F b,
                                                  F& uc, F& sc, F& gu, F alpha,
                                                  F thresh, F beta, F interval,
                                                  Emit&& emit) {
    F xin[TW], gin[TW], u[TW];
#pragma unroll
    for (int t = 0; t < TW; ++t) {
        xin[t] = F(0);
        if (EXACT || t < rows)
            xin[t] = load_pack<F, 1, false>(x + static_cast<int64_t>(t) * N + col).e[0];
    }
#pragma unroll
    for (int t = TW - 1; t >= 0; --t) {
        gin[t] = F(0);
        if (EXACT || t < rows)
            gin[t] = load_pack<F, 1, true>(g + static_cast<int64_t>(t) * N + col).e[0];
    }
#pragma unroll
    for (int t = 0; t < TW; ++t) {
        uc = (alpha * uc) * (F(1) - sc) + (xin[t] - m) * scale + b;
        sc = (uc > thresh) ? F(1) : F(0);
        u[t] = uc;
    }
#pragma unroll
    for (int t = TW - 1; t >= 0; --t) {
        if (EXACT || t < rows) {
            lif_reverse_step<F>(gu, u[t], gin[t], alpha, thresh, beta, interval);
            emit(t, gu, xin[t]);
        }
    }
}

// The whole time axis as one window (T <= TW).
template <typename F, int TW, bool EXACT, typename Emit>
__device__ __forceinline__ void bn_reverse_chain(const F* __restrict__ x,
                                                 const F* __restrict__ g, int T, int64_t N,
                                                 int64_t col, F m, F scale, F b,
                                                 F alpha, F thresh, F beta,
                                                 F interval, Emit&& emit) {
    F uc = F(0), sc = F(0), gu = F(0);
    bn_reverse_window<F, TW, EXACT>(x, g, T, N, col, m, scale, b, uc, sc, gu, alpha, thresh, beta,
                                 interval, emit);
}

// Time axes longer than one register window, in segments of kSegment steps, the way
// lif_backward_segmented_kernel does it: forward over all but the last segment keeping the membrane
// potential at each boundary in a slot of this lane's own, then the segments last to first.  The slot
// of segment `seg` (the potential after step seg*kSegment - 1, seg >= 1) is
// boundary[seg * bstride + boff]: dynamic LDS ([segment][blockDim.x]: bstride = blockDim.x, boff =
// threadIdx.x) or device memory ([segment][N]: bstride = N, boff = col; or rows of the gradient still
// to be written).  emit gets the absolute time step.
template <typename F, typename Emit>
__device__ __forceinline__ void bn_reverse_segmented(const F* __restrict__ x,
                                                     const F* __restrict__ g, int T, int64_t N,
                                                     int64_t col, F m, F scale, F b,
                                                     F alpha, F thresh, F beta,
                                                     F interval, F* boundary, int64_t bstride,
                                                     int64_t boff, Emit&& emit) {
    const int nseg = (T + kSegment - 1) / kSegment;
    constexpr int ROWS = 8;
    static_assert(kSegment % ROWS == 0, "a segment is a whole number of forward groups");
    F uc = F(0), sc = F(0), gu = F(0);
    for (int seg = 0; seg + 1 < nseg; ++seg) {
        for (int t0 = seg * kSegment; t0 < (seg + 1) * kSegment; t0 += ROWS) {
            F rows[ROWS];
#pragma unroll
            for (int k = 0; k < ROWS; ++k)
                rows[k] = load_pack<F, 1, false>(x + static_cast<int64_t>(t0 + k) * N + col).e[0];
#pragma unroll
            for (int k = 0; k < ROWS; ++k) {
                uc = (alpha * uc) * (F(1) - sc) + (rows[k] - m) * scale + b;
                sc = (uc > thresh) ? F(1) : F(0);
            }
        }
        boundary[static_cast<int64_t>(seg + 1) * bstride + boff] = uc;
    }
    {
        const int t0 = (nseg - 1) * kSegment;
        const int64_t off = static_cast<int64_t>(t0) * N;
        bn_reverse_window<F, kSegment, false>(x + off, g + off, T - t0, N, col, m, scale, b, uc, sc, gu,
                                           alpha, thresh, beta, interval,
                                           [&](int t, F gy, F xt) { emit(t0 + t, gy, xt); });
    }
    for (int seg = nseg - 2; seg >= 0; --seg) {
        uc = seg == 0 ? F(0) : boundary[static_cast<int64_t>(seg) * bstride + boff];
        sc = (seg != 0 && uc > thresh) ? F(1) : F(0);
        const int t0 = seg * kSegment;
        const int64_t off = static_cast<int64_t>(t0) * N;
        bn_reverse_window<F, kSegment, true>(x + off, g + off, kSegment, N, col, m, scale, b, uc, sc, gu,
                                          alpha, thresh, beta, interval,
                                          [&](int t, F gy, F xt) { emit(t0 + t, gy, xt); });
    }
}

// How a kernel instance walks time: the whole window in registers, or in segments with the boundary
// potentials in LDS or in device memory.
enum class TimeWalk { window, segments_lds, segments_memory };

// Dispatch between them; segmented kernels are instantiated with TW = kSegment.  `far` is the
// device-memory boundary array (TimeWalk::segments_memory) with its stride and this lane's offset.
template <typename F, int TW, bool EXACT, TimeWalk WALK, typename Emit>
__device__ __forceinline__ void bn_reverse(const F* __restrict__ x, const F* __restrict__ g,
                                           int T, int64_t N, int64_t col, F m, F scale,
                                           F b, F alpha, F thresh, F beta,
                                           F interval, F* lds_boundary, F* far, int64_t far_stride,
                                           int64_t far_offset, Emit&& emit) {
    if constexpr (WALK == TimeWalk::segments_lds) {
        bn_reverse_segmented<F>(x, g, T, N, col, m, scale, b, alpha, thresh, beta, interval, lds_boundary,
                                static_cast<int64_t>(blockDim.x), static_cast<int64_t>(threadIdx.x), emit);
    } else if constexpr (WALK == TimeWalk::segments_memory) {
        bn_reverse_segmented<F>(x, g, T, N, col, m, scale, b, alpha, thresh, beta, interval, far,
                                far_stride, far_offset, emit);
    } else {
        bn_reverse_chain<F, TW, EXACT>(x, g, T, N, col, m, scale, b, alpha, thresh, beta, interval, emit);
    }
}

// Sum over the 64 lanes of a wavefront; lane 0 holds the result.
template <typename F>
__device__ __forceinline__ F wave_sum(F v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off, 64);
    return v;
}

// Sweep 1: sums over time of gy and gy * xhat.
// WAVE = false: one lane per neuron in storage order, one pair of floats per neuron.
// WAVE = true: wavefronts are laid over the (batch entry, channel) planes -- G = ceil(HW/64)
// wavefronts per plane, the last one partly idle when HW is not a multiple of 64 -- so all lanes of
// a wavefront share a channel and their sums are folded by shuffles: one pair of floats per
// wavefront, part_* indexed [plane][chunk] (B*C*G entries).  NB > 1 (short windows, B a multiple of
// NB): a lane takes the same position of NB batch entries B/NB apart, so that a read-only sweep whose
// window gives a lane fewer than sixteen requests keeps that many in flight all the same; the
// planes then number (B/NB)*C.
// `far`: [segment][N] boundary potentials in the workspace (TimeWalk::segments_memory only).
template <typename F, int TW, bool EXACT, bool WAVE, TimeWalk WALK = TimeWalk::window, int NB = 1>
__global__ void __launch_bounds__(kBwdBlock) SNNLIF_WAVES_PER_SIMD(backward_waves(TW))
lif_bn_backward_partial_kernel(const F* __restrict__ x, const F* __restrict__ g,
                               const F* __restrict__ weight, const F* __restrict__ bias,
                               const F* __restrict__ ivar, const F* __restrict__ mean,
                               F* __restrict__ part_gy, F* __restrict__ part_gyx, F* __restrict__ far,
                               int T, int64_t N, int64_t C, int64_t HW, F alpha, F thresh,
                               F beta, F interval) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    F* boundary = reinterpret_cast<F*>(lds_raw);  // used by TimeWalk::segments_lds only
    const bool small = N <= 0xffffffffll;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    if (WAVE) {
        const int64_t G = (HW + 63) / 64;
        const int64_t planes = (N / HW) / NB;     // (B/NB) * C
        const int64_t lanes = planes * G * 64;    // padded lane space: planes * G wavefronts
        for (int64_t pc = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; pc < lanes;
             pc += stride) {
            const int64_t wave = pc >> 6;
            const int64_t plane = wave / G;
            const int64_t k = (wave - plane * G) * 64 + (pc & 63);  // position inside the plane
            const int c = static_cast<int>(plane % C);
            F acc_gy = F(0), acc_gyx = F(0);
            if (k < HW) {
                const F m = mean[c], iv = ivar[c];
                const F scale = weight[c] * iv;
                const F b = bias[c];
#pragma unroll
                for (int j = 0; j < NB; ++j) {
                    const int64_t col = (plane + j * planes) * HW + k;
                    bn_reverse<F, TW, EXACT, WALK>(x, g, T, N, col, m, scale, b, alpha, thresh, beta,
                                                   interval, boundary, far, N, col,
                                                   [&](int, F gy, F xt) {
                                                       const F xhat = (xt - m) * iv;
                                                       acc_gy += gy;
                                                       acc_gyx += gy * xhat;
                                                   });
                }
            }
            acc_gy = wave_sum(acc_gy);
            acc_gyx = wave_sum(acc_gyx);
            if ((pc & 63) == 0) {
                part_gy[wave] = acc_gy;
                part_gyx[wave] = acc_gyx;
            }
        }
    } else {
        for (int64_t col = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; col < N;
             col += stride) {
            const int c = channel_of(col, C, HW, small);
            const F m = mean[c], iv = ivar[c];
            const F scale = weight[c] * iv;
            const F b = bias[c];
            F acc_gy = F(0), acc_gyx = F(0);
            bn_reverse<F, TW, EXACT, WALK>(x, g, T, N, col, m, scale, b, alpha, thresh, beta,
                                           interval, boundary, far, N, col, [&](int, F gy, F xt) {
                                               const F xhat = (xt - m) * iv;
                                               acc_gy += gy;
                                               acc_gyx += gy * xhat;
                                           });
            part_gy[col] = acc_gy;
            part_gyx[col] = acc_gyx;
        }
    }
}

// Sweep 2: input gradient.  mean_gxhat[C], mean_gxhatx[C]: the per-channel means that sweep 1 and
// the channel reduction produced (averaged over the ranks first when the batch is sharded).
// With TimeWalk::segments_memory the boundary potential of segment seg >= 1 is parked in row
// seg*kSegment - 1 of gx, column of this lane: that row belongs to segment seg - 1, which this lane
// writes only after it has consumed the value (segments are swept last to first).
template <typename F, int TW, bool EXACT, TimeWalk WALK = TimeWalk::window>
__global__ void __launch_bounds__(kBwdBlock) SNNLIF_WAVES_PER_SIMD(backward_waves(TW))
lif_bn_backward_input_kernel(const F* __restrict__ x, const F* __restrict__ g,
                             const F* __restrict__ weight, const F* __restrict__ bias,
                             const F* __restrict__ ivar, const F* __restrict__ mean,
                             const F* __restrict__ mean_gxhat,
                             const F* __restrict__ mean_gxhatx, F* __restrict__ gx, int T,
                             int64_t N, int64_t C, int64_t HW, F alpha, F thresh, F beta,
                             F interval) {
    extern __shared__ __align__(16) unsigned char lds_raw[];
    F* boundary = reinterpret_cast<F*>(lds_raw);  // used by TimeWalk::segments_lds only
    const bool small = N <= 0xffffffffll;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t v = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; v < N;
         v += stride) {
        const int64_t col = N - 1 - v;  // opposite direction to sweep 1: its tail is still cached
        const int c = channel_of(col, C, HW, small);
        const F m = mean[c], iv = ivar[c], wgt = weight[c];
        const F scale = wgt * iv;
        const F b = bias[c];
        const F gxhat = mean_gxhat[c], gxhatx = mean_gxhatx[c];
        bn_reverse<F, TW, EXACT, WALK>(
            x, g, T, N, col, m, scale, b, alpha, thresh, beta, interval, boundary, gx,
            static_cast<int64_t>(kSegment) * N, col - N, [&](int t, F gy, F xt) {
                Pack<F, 1> out;
                out.e[0] = gy * wgt * iv - iv * ((xt - m) * iv * gxhatx + gxhat);
                store_pack<F, 1>(gx + static_cast<int64_t>(t) * N + col, out);
            });
    }
}

// ---------------------------------------------------------------------------------------------
// Reduction of the per-neuron partials, a [B, CHW] matrix per quantity: workgroup (blockIdx.x,
// blockIdx.y = s) adds up the batch entries [s*bs, min(B, (s+1)*bs)) of its kReduceBlock columns,
// one column (channel, position) per lane -- consecutive lanes read consecutive addresses, and the
// order of the sum is fixed by the geometry alone.  split = {gy[S][CHW], gyx[S][CHW]}.
// ---------------------------------------------------------------------------------------------
template <typename F>
__global__ void __launch_bounds__(kReduceBlock)
bn_column_reduce_kernel(const F* __restrict__ part_gy, const F* __restrict__ part_gyx,
                        F* __restrict__ split, int64_t B, int64_t CHW, int64_t bs, int S) {
    const int64_t j = static_cast<int64_t>(blockIdx.x) * kReduceBlock + threadIdx.x;
    if (j >= CHW) return;
    const int s = blockIdx.y;
    const int64_t b0 = static_cast<int64_t>(s) * bs;
    const int64_t b1 = (b0 + bs < B) ? (b0 + bs) : B;
    F a = F(0), ax = F(0);
    for (int64_t b = b0; b < b1; ++b) {
        a += part_gy[b * CHW + j];
        ax += part_gyx[b * CHW + j];
    }
    split[static_cast<int64_t>(s) * CHW + j] = a;
    split[(static_cast<int64_t>(S) + s) * CHW + j] = ax;
}

// Whole reduction of one channel in one workgroup, for partials that are few (the wave-summed
// form): sums the B*G entries of channel c (G entries per batch entry), then writes the parameter
// gradients and the two coefficients of the input-gradient sweep.
template <typename F>
__global__ void __launch_bounds__(kReduceBlock)
bn_channel_reduce_finalize_kernel(const F* __restrict__ part_gy,
                                  const F* __restrict__ part_gyx,
                                  const F* __restrict__ weight, F* __restrict__ grad_weight,
                                  F* __restrict__ grad_bias, F* __restrict__ mean_gxhat,
                                  F* __restrict__ mean_gxhatx, int64_t B, int64_t C, int64_t G,
                                  F count) {
    const int c = blockIdx.x;
    const int64_t n = B * G;
    F a = F(0), ax = F(0);
    for (int64_t e = threadIdx.x; e < n; e += kReduceBlock) {
        const int64_t b = e / G, i = e % G;
        const int64_t at = (b * C + c) * G + i;
        a += part_gy[at];
        ax += part_gyx[at];
    }
    __shared__ F lds[2][kReduceBlock / 64];
    a = wave_sum(a);
    ax = wave_sum(ax);
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    if (lane == 0) {
        lds[0][wave] = a;
        lds[1][wave] = ax;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        F ta = F(0), tax = F(0);
#pragma unroll
        for (int w = 0; w < kReduceBlock / 64; ++w) {
            ta += lds[0][w];
            tax += lds[1][w];
        }
        grad_bias[c] = ta;
        grad_weight[c] = tax;
        const F wgt = weight[c];
        mean_gxhat[c] = (ta * wgt) / count;
        mean_gxhatx[c] = (tax * wgt) / count;
    }
}

// One wavefront per channel: lane l adds entries l, l + 64, ... of the channel's S*HW partial sums
// (slice-major), the wavefront folds its lanes by shuffles -- an order fixed by S and HW alone -- and
// lane 0 emits the parameter gradients and the two coefficients the input-gradient sweep needs.
// (One lane per channel walking the S*HW entries one after the other took 68 us for 512 channels of 16
// positions in 32 slices: a chain of dependent memory round trips.)
template <typename F>
__global__ void __launch_bounds__(kReduceBlock)
bn_channel_finalize_kernel(const F* __restrict__ split, const F* __restrict__ weight,
                           F* __restrict__ grad_weight, F* __restrict__ grad_bias,
                           F* __restrict__ mean_gxhat, F* __restrict__ mean_gxhatx,
                           int64_t C, int64_t HW, int S, F count) {
    const int64_t c = static_cast<int64_t>(blockIdx.x) * (kReduceBlock / 64) + threadIdx.x / 64;
    if (c >= C) return;  // whole wavefronts leave together
    const int lane = threadIdx.x % 64;
    const int64_t CHW = C * HW;
    const int64_t n = static_cast<int64_t>(S) * HW;
    F a = F(0), ax = F(0);
    for (int64_t e = lane; e < n; e += 64) {
        const int64_t s = e / HW, i = e - s * HW;
        a += split[s * CHW + c * HW + i];
        ax += split[(static_cast<int64_t>(S) + s) * CHW + c * HW + i];
    }
    a = wave_sum(a);
    ax = wave_sum(ax);
    if (lane != 0) return;
    grad_bias[c] = a;
    grad_weight[c] = ax;
    const F wgt = weight[c];
    mean_gxhat[c] = (a * wgt) / count;
    mean_gxhatx[c] = (ax * wgt) / count;
}

}  // namespace snnlif

#endif  // SNNLIF_LIF_BN_KERNELS_H
