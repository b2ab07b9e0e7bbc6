// Plain batch norm of a [T, B, C, HW] activation for MI355X (F = float or double): the layer without
// a fire recurrence behind it, forward and backward, and the two halves of the backward that a batch
// sharded over several GPUs runs on either side of its all-reduce.
//
// Reference: snnlib/cuda/snn_kernel_fp.cu:81-150 (bn_fp_kernel + bn_fp_cuda) and
// snnlib/cuda/snn_kernel_bp.cu:176-236 (bn_bp_wb_kernel), :240-285 (bn_bp_x_kernel), :288-345 (bn_bp_cuda),
// :348-425 (bn_bp_cuda_dist1 / _dist2).
//
//   forward   scale[c] = weight[c] / sqrt(var[c] + eps);   ivar[c] = scale[c] / weight[c]
//             y = (x - mean[c]) * scale[c] + bias[c]
//   backward  xhat = (x - mean[c]) * ivar[c],   M = T*B*HW
//             grad_bias[c] = sum g;   grad_weight[c] = sum g * xhat          (over T, B, HW)
//             gxhat[c] = weight[c] * grad_bias[c] / M;   gxhatx[c] = weight[c] * grad_weight[c] / M
//             gx = (g * weight[c]) * ivar[c] - ivar[c] * ((xhat * gxhatx[c]) + gxhat[c])
//
// Mapping.  Time and batch are the same thing to a batch norm: the tensor is a matrix of R = T*B rows
// of C*HW elements.  Nothing is carried from row to row, so every pass is cut along both axes:
//   * element-wise passes (forward, input gradient): a lane owns V consecutive positions of a row
//     (16 bytes when C*HW and the base addresses allow, else one element), takes kBnPlainRows
//     consecutive rows of them and requests them all before it consumes the first; the channel of each
//     position and its per-channel constants are worked out once per lane.  8 bytes per element
//     forward (R x, W y), 12 backward (R x, R g, W gx).
//   * sums (backward, before any input gradient can be formed): planes of at least 32 positions are
//     covered by whole wavefronts (ceil(HW/64) per plane, all lanes of one share a channel); a lane adds
//     up g and g*xhat over the rows of its slice, the wavefront folds its lanes by shuffles and leaves
//     one pair of sums, and bn_channel_reduce_finalize_kernel (lif_bn_kernels.h) adds them per channel
//     in a fixed order.  Smaller planes (fully connected shapes): a lane per column of the matrix and
//     row slice, partial sums per (slice, column), folded by bn_channel_finalize_kernel.  8 bytes per
//     element (R x, R g).
// The reference moves 8 bytes forward and 28 backward (its second kernel re-reads both tensors and the
// per-position partial sums go through at::sum / at::mean); here 8 and 20.
#ifndef SNNLIF_LIF_BN_PLAIN_H
#define SNNLIF_LIF_BN_PLAIN_H

#include "lif_bn.h"
#include "lif_bn_kernels.h"

namespace snnlif {

// Rows a lane of the element-wise passes requests before it consumes the first (kBnPlainRows, lif_bn.h),
// threads per workgroup, wavefronts per SIMD.
#ifndef SNNLIF_BN_PLAIN_BLOCK
#define SNNLIF_BN_PLAIN_BLOCK 256
#endif
#ifndef SNNLIF_BN_PLAIN_WAVES
#define SNNLIF_BN_PLAIN_WAVES 8
#endif
// Bytes per lane and memory instruction of the element-wise passes.
#ifndef SNNLIF_BN_PLAIN_LANE_BYTES
#define SNNLIF_BN_PLAIN_LANE_BYTES 16
#endif
// Cache policy of the sums pass (1 = non-temporal loads): x with the default policy, the gradient
// streamed.  The input-gradient pass reads both again straight away; what the 256 MB memory-side cache
// can keep for it is one tensor's worth, and with only x competing for it the second pass finds more.
// Measured at [8,64,128,32,32] fp32 (sums + input-gradient kernel, us): both default 87 + 125, gradient
// streamed 84 + 117, both streamed 81 + 134.
#ifndef SNNLIF_BN_PLAIN_SUM_STREAM_X
#define SNNLIF_BN_PLAIN_SUM_STREAM_X 0
#endif
#ifndef SNNLIF_BN_PLAIN_SUM_STREAM_G
#define SNNLIF_BN_PLAIN_SUM_STREAM_G 1
#endif
// The input-gradient pass takes its tiles from the last to the first (1) or in storage order (0).
#ifndef SNNLIF_BN_PLAIN_INPUT_DESCENDING
#define SNNLIF_BN_PLAIN_INPUT_DESCENDING 1
#endif
// Threads per workgroup of the sums pass.
#ifndef SNNLIF_BN_PLAIN_SUM_BLOCK
#define SNNLIF_BN_PLAIN_SUM_BLOCK 256
#endif
constexpr int kBnPlainBlock = SNNLIF_BN_PLAIN_BLOCK;
constexpr int kBnPlainSumBlock = SNNLIF_BN_PLAIN_SUM_BLOCK;

// Channel constants of the V positions a lane owns.
template <typename F, int V>
struct BnLaneChannels {
    int c[V];
    __device__ __forceinline__ void locate(int64_t first, int64_t HW, int64_t CHW) {
        const bool small = CHW <= 0xffffffffll;
#pragma unroll
        for (int j = 0; j < V; ++j) {
            c[j] = small ? static_cast<int>(static_cast<uint32_t>(first + j) / static_cast<uint32_t>(HW))
                         : static_cast<int>((first + j) / HW);
        }
    }
};

// ---------------------------------------------------------------------------------------------
// Forward.  The matrix is cut into tiles of ROWS rows by blockDim.x packs of V positions, numbered row
// slice by row slice (`across` tiles per slice); a workgroup takes tile blockIdx.x (and further ones a
// whole grid apart when the launch was capped).  The lane that holds position 0 of a channel in row 0
// publishes the channel's inverse standard deviation.
// ---------------------------------------------------------------------------------------------
template <typename F, int V, int ROWS>
__global__ void __launch_bounds__(kBnPlainBlock) SNNLIF_WAVES_PER_SIMD(SNNLIF_BN_PLAIN_WAVES)
bn_plain_forward_kernel(const F* __restrict__ x, const F* __restrict__ weight,
                        const F* __restrict__ bias, const F* __restrict__ var,
                        const F* __restrict__ mean, F* __restrict__ ivar, F* __restrict__ y,
                        int64_t R, int64_t CHW, int64_t HW, int64_t across, int64_t tiles, F eps) {
  for (int64_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
    const int64_t slice = tile / across;
    const int64_t first = ((tile - slice * across) * blockDim.x + threadIdx.x) * V;
    if (first >= CHW) continue;
    const int64_t r0 = slice * ROWS;

    Pack<F, V> in[ROWS];
#pragma unroll
    for (int k = 0; k < ROWS; ++k) {
        in[k] = zero_pack<F, V>();
        if (r0 + k < R) in[k] = load_pack<F, V, true>(x + (r0 + k) * CHW + first);
    }

    BnLaneChannels<F, V> ch;
    ch.locate(first, HW, CHW);
    F m[V], scale[V], b[V];
#pragma unroll
    for (int j = 0; j < V; ++j) {
        const F wgt = weight[ch.c[j]];
        m[j] = mean[ch.c[j]];
        scale[j] = wgt / real_sqrt(var[ch.c[j]] + eps);
        b[j] = bias[ch.c[j]];
        if (r0 == 0 && first + j == static_cast<int64_t>(ch.c[j]) * HW) ivar[ch.c[j]] = scale[j] / wgt;
    }

#pragma unroll
    for (int k = 0; k < ROWS; ++k) {
        if (r0 + k < R) {
            Pack<F, V> out;
#pragma unroll
            for (int j = 0; j < V; ++j) out.e[j] = (in[k].e[j] - m[j]) * scale[j] + b[j];
            store_pack<F, V>(y + (r0 + k) * CHW + first, out);
        }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Input gradient from the two per-channel means.  Same tiles as the forward, taken from the last to
// the first: right behind the sums pass (which walks the tensors upwards with the default cache
// policy) the end of x and g is what the memory-side cache still holds.
// ---------------------------------------------------------------------------------------------
template <typename F, int V, int ROWS>
__global__ void __launch_bounds__(kBnPlainBlock) SNNLIF_WAVES_PER_SIMD(SNNLIF_BN_PLAIN_WAVES)
bn_plain_input_kernel(const F* __restrict__ x, const F* __restrict__ g,
                      const F* __restrict__ weight, const F* __restrict__ ivar,
                      const F* __restrict__ mean, const F* __restrict__ mean_gxhat,
                      const F* __restrict__ mean_gxhatx, F* __restrict__ gx, int64_t R,
                      int64_t CHW, int64_t HW, int64_t across, int64_t tiles) {
  for (int64_t turn = blockIdx.x; turn < tiles; turn += gridDim.x) {
    const int64_t tile = SNNLIF_BN_PLAIN_INPUT_DESCENDING ? tiles - 1 - turn : turn;
    const int64_t slice = tile / across;
    const int64_t first = ((tile - slice * across) * blockDim.x + threadIdx.x) * V;
    if (first >= CHW) continue;
    const int64_t r0 = slice * ROWS;

    Pack<F, V> xin[ROWS], gin[ROWS];
#pragma unroll
    for (int k = 0; k < ROWS; ++k) {
        xin[k] = zero_pack<F, V>();
        gin[k] = zero_pack<F, V>();
        if (r0 + k < R) {
            xin[k] = load_pack<F, V, true>(x + (r0 + k) * CHW + first);
            gin[k] = load_pack<F, V, true>(g + (r0 + k) * CHW + first);
        }
    }

    BnLaneChannels<F, V> ch;
    ch.locate(first, HW, CHW);
    F m[V], iv[V], wgt[V], gxhat[V], gxhatx[V];
#pragma unroll
    for (int j = 0; j < V; ++j) {
        m[j] = mean[ch.c[j]];
        iv[j] = ivar[ch.c[j]];
        wgt[j] = weight[ch.c[j]];
        gxhat[j] = mean_gxhat[ch.c[j]];
        gxhatx[j] = mean_gxhatx[ch.c[j]];
    }

#pragma unroll
    for (int k = 0; k < ROWS; ++k) {
        if (r0 + k < R) {
            Pack<F, V> out;
#pragma unroll
            for (int j = 0; j < V; ++j)
                out.e[j] = gin[k].e[j] * wgt[j] * iv[j] -
                           iv[j] * ((xin[k].e[j] - m[j]) * iv[j] * gxhatx[j] + gxhat[j]);
            store_pack<F, V>(gx + (r0 + k) * CHW + first, out);
        }
    }
  }
}

// Adds the kBnPlainSumRows rows [r, r + kBnPlainSumRows) of one column (rows past `end` count as zero
// gradient) to the running sums of g and g * xhat.
template <typename F>
__device__ __forceinline__ void bn_plain_add_rows(const F* __restrict__ x, const F* __restrict__ g,
                                                  int64_t r, int64_t end, int64_t CHW, int64_t at,
                                                  F m, F iv, F& acc_g, F& acc_gx) {
    F xin[kBnPlainSumRows], gin[kBnPlainSumRows];
#pragma unroll
    for (int k = 0; k < kBnPlainSumRows; ++k) {
        xin[k] = F(0);
        gin[k] = F(0);
        if (r + k < end) {
            xin[k] = load_pack<F, 1, SNNLIF_BN_PLAIN_SUM_STREAM_X != 0>(x + (r + k) * CHW + at).e[0];
            gin[k] = load_pack<F, 1, SNNLIF_BN_PLAIN_SUM_STREAM_G != 0>(g + (r + k) * CHW + at).e[0];
        }
    }
#pragma unroll
    for (int k = 0; k < kBnPlainSumRows; ++k) {
        const F xhat = (xin[k] - m) * iv;
        acc_g += gin[k];
        acc_gx += gin[k] * xhat;
    }
}

// ---------------------------------------------------------------------------------------------
// Sums, planes of at least 32 positions.  Lane space [slice][channel][chunk][64]: wavefront
// (s, c, i) covers positions [64 i, 64 i + 64) of channel c in the rows [s * rps, (s + 1) * rps) and
// leaves part_*[(s * C + c) * G + i].
// ---------------------------------------------------------------------------------------------
template <typename F>
__global__ void __launch_bounds__(kBnPlainSumBlock) SNNLIF_WAVES_PER_SIMD(SNNLIF_BN_PLAIN_WAVES)
bn_plain_sums_wave_kernel(const F* __restrict__ x, const F* __restrict__ g,
                          const F* __restrict__ ivar, const F* __restrict__ mean,
                          F* __restrict__ part_g, F* __restrict__ part_gx, int64_t R, int64_t rps,
                          int64_t S, int64_t C, int64_t HW, int64_t G) {
    const int64_t lanes = S * C * G * 64;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    const int64_t CHW = C * HW;
    for (int64_t pc = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; pc < lanes;
         pc += stride) {
        const int64_t wave = pc >> 6;
        const int64_t plane = wave / G;  // slice * C + channel
        const int64_t k = (wave - plane * G) * 64 + (pc & 63);
        const int64_t s = plane / C;
        const int c = static_cast<int>(plane - s * C);
        F acc_g = F(0), acc_gx = F(0);
        if (k < HW) {
            const F m = mean[c], iv = ivar[c];
            const int64_t at = static_cast<int64_t>(c) * HW + k;
            const int64_t begin = s * rps;
            const int64_t end = (begin + rps < R) ? begin + rps : R;
            for (int64_t r = begin; r < end; r += kBnPlainSumRows)
                bn_plain_add_rows<F>(x, g, r, end, CHW, at, m, iv, acc_g, acc_gx);
        }
        acc_g = wave_sum(acc_g);
        acc_gx = wave_sum(acc_gx);
        if ((pc & 63) == 0) {
            part_g[wave] = acc_g;
            part_gx[wave] = acc_gx;
        }
    }
}

// Sums, smaller planes: workgroup (blockIdx.x, blockIdx.y = s) sums the rows of slice s in its columns;
// split = {g[S][CHW], g*xhat[S][CHW]}, the layout bn_channel_finalize_kernel folds.
template <typename F>
__global__ void __launch_bounds__(kBnPlainSumBlock)
bn_plain_sums_column_kernel(const F* __restrict__ x, const F* __restrict__ g,
                            const F* __restrict__ ivar, const F* __restrict__ mean,
                            F* __restrict__ split, int64_t R, int64_t rps, int S, int64_t CHW,
                            int64_t HW) {
    const int64_t j = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (j >= CHW) return;
    const int s = blockIdx.y;
    const int64_t c = j / HW;
    const F m = mean[c], iv = ivar[c];
    const int64_t begin = static_cast<int64_t>(s) * rps;
    const int64_t end = (begin + rps < R) ? begin + rps : R;
    F acc_g = F(0), acc_gx = F(0);
    for (int64_t r = begin; r < end; r += kBnPlainSumRows)
        bn_plain_add_rows<F>(x, g, r, end, CHW, j, m, iv, acc_g, acc_gx);
    split[static_cast<int64_t>(s) * CHW + j] = acc_g;
    split[(static_cast<int64_t>(S) + s) * CHW + j] = acc_gx;
}

// ---------------------------------------------------------------------------------------------
// Host side.
// ---------------------------------------------------------------------------------------------

// Widest lanes (in elements) of the element-wise passes for which rows and base addresses stay aligned.
template <typename F>
inline int bn_plain_vec(int64_t CHW, const void* const* ptrs, int n) {
    constexpr int maxv = SNNLIF_BN_PLAIN_LANE_BYTES / static_cast<int>(sizeof(F)) < 1
                             ? 1
                             : SNNLIF_BN_PLAIN_LANE_BYTES / static_cast<int>(sizeof(F));
    int v = maxv;
    while (v > 1) {
        bool ok = (CHW % v) == 0;
        for (int i = 0; ok && i < n; ++i) ok = aligned_to(ptrs[i], sizeof(F) * v);
        if (ok) break;
        v >>= 1;
    }
    return v;
}

// Tiles of the element-wise passes: `across` per row slice, `tiles` in all.
struct BnPlainTiles {
    int64_t across, tiles;
};
inline BnPlainTiles bn_plain_tiles(int64_t R, int64_t CHW, int v) {
    const int64_t packs = (CHW + v - 1) / v;
    const int64_t across = (packs + kBnPlainBlock - 1) / kBnPlainBlock;
    return BnPlainTiles{across, across * ((R + kBnPlainRows - 1) / kBnPlainRows)};
}
inline dim3 bn_plain_grid(const BnPlainTiles& t) {
    return dim3(static_cast<unsigned>(t.tiles < kMaxGrid ? (t.tiles < 1 ? 1 : t.tiles) : kMaxGrid));
}

template <typename F>
int bn_plain_forward(const F* x, const F* weight, const F* bias, const F* var, const F* mean, F* ivar,
                     F* y, int64_t T, int64_t B, int64_t C, int64_t HW, float eps,
                     hipStream_t stream) {
    const int64_t R = T * B, CHW = C * HW;
    const void* ptrs[2] = {x, y};
    const int v = bn_plain_vec<F>(CHW, ptrs, 2);
    constexpr int maxv = 16 / static_cast<int>(sizeof(F));
    return with_vec<maxv>(v, [&](auto vc) {
        constexpr int V = decltype(vc)::value;
        const BnPlainTiles t = bn_plain_tiles(R, CHW, V);
        launch_kernel(bn_plain_forward_kernel<F, V, kBnPlainRows>, bn_plain_grid(t),
                      dim3(kBnPlainBlock), 0, stream, x, weight, bias, var, mean, ivar, y, R, CHW, HW,
                      t.across, t.tiles, F(eps));
        return launch_status();
    });
}

template <typename F>
int bn_plain_backward_input(const F* x, const F* weight, const F* ivar, const F* mean, const F* g,
                            const F* mean_gxhat, const F* mean_gxhatx, F* gx, int64_t T, int64_t B,
                            int64_t C, int64_t HW, hipStream_t stream) {
    const int64_t R = T * B, CHW = C * HW;
    const void* ptrs[3] = {x, g, gx};
    const int v = bn_plain_vec<F>(CHW, ptrs, 3);
    constexpr int maxv = 16 / static_cast<int>(sizeof(F));
    return with_vec<maxv>(v, [&](auto vc) {
        constexpr int V = decltype(vc)::value;
        const BnPlainTiles t = bn_plain_tiles(R, CHW, V);
        launch_kernel(bn_plain_input_kernel<F, V, kBnPlainRows>, bn_plain_grid(t),
                      dim3(kBnPlainBlock), 0, stream, x, g, weight, ivar, mean, mean_gxhat,
                      mean_gxhatx, gx, R, CHW, HW, t.across, t.tiles);
        return launch_status();
    });
}

// Sums + channel reduction: parameter gradients and the two per-channel means.  workspace:
// bn_plain_workspace_elems() values.
template <typename F>
int bn_plain_backward_stats(const F* x, const F* weight, const F* ivar, const F* mean, const F* g,
                            F* grad_weight, F* grad_bias, F* mean_gxhat, F* mean_gxhatx, int64_t T,
                            int64_t B, int64_t C, int64_t HW, F* workspace, hipStream_t stream) {
    const int64_t R = T * B, CHW = C * HW;
    const int64_t S = bn_plain_slices(R, C, HW);
    const int64_t rps = (R + S - 1) / S;
    const F count = static_cast<F>(R * HW);
    if (bn_wave_partials(HW)) {
        const int64_t G = (HW + 63) / 64;
        F* part_g = workspace;
        F* part_gx = workspace + S * C * G;
        launch_kernel(bn_plain_sums_wave_kernel<F>, dim3(grid_for(S * C * G * 64, kBnPlainSumBlock)),
                      dim3(kBnPlainSumBlock), 0, stream, x, g, ivar, mean, part_g, part_gx, R, rps, S, C,
                      HW, G);
        int rc = launch_status();
        if (rc != SNNLIF_OK) return rc;
        launch_kernel(bn_channel_reduce_finalize_kernel<F>, dim3(static_cast<unsigned>(C)),
                      dim3(kReduceBlock), 0, stream, part_g, part_gx, weight, grad_weight, grad_bias,
                      mean_gxhat, mean_gxhatx, S, C, G, count);
        return launch_status();
    }
    F* split = workspace;
    launch_kernel(bn_plain_sums_column_kernel<F>,
                  dim3(static_cast<unsigned>((CHW + kBnPlainSumBlock - 1) / kBnPlainSumBlock),
                       static_cast<unsigned>(S)),
                  dim3(kBnPlainSumBlock), 0, stream, x, g, ivar, mean, split, R, rps, static_cast<int>(S),
                  CHW, HW);
    int rc = launch_status();
    if (rc != SNNLIF_OK) return rc;
    launch_kernel(bn_channel_finalize_kernel<F>,
                  dim3(static_cast<unsigned>((C + kReduceBlock / 64 - 1) / (kReduceBlock / 64))),
                  dim3(kReduceBlock), 0, stream, split, weight, grad_weight, grad_bias, mean_gxhat,
                  mean_gxhatx, C, HW, static_cast<int>(S), count);
    return launch_status();
}

template <typename F>
int bn_plain_backward(const F* x, const F* weight, const F* ivar, const F* mean, const F* g, F* gx,
                      F* grad_weight, F* grad_bias, int64_t T, int64_t B, int64_t C, int64_t HW,
                      F* workspace, hipStream_t stream) {
    // the two per-channel means live behind the partial sums in the workspace between the passes
    F* coef = workspace + bn_plain_workspace_elems(T, B, C, HW) - 2 * C;
    const int rc = bn_plain_backward_stats<F>(x, weight, ivar, mean, g, grad_weight, grad_bias, coef,
                                              coef + C, T, B, C, HW, workspace, stream);
    if (rc != SNNLIF_OK) return rc;
    return bn_plain_backward_input<F>(x, weight, ivar, mean, g, coef, coef + C, gx, T, B, C, HW,
                                      stream);
}

}  // namespace snnlif

// The entry points lif_bn.h declares for the plain batch norm, scalar type F, name suffix SUFFIX.
#define SNNLIF_DEFINE_BN_PLAIN_DTYPE(SUFFIX, F)                                                    \
    namespace snnlif {                                                                             \
    int bn_plain_forward_##SUFFIX(const F* x, const F* weight, const F* bias, const F* var,        \
                                  const F* mean, F* ivar, F* y, int64_t T, int64_t B, int64_t C,   \
                                  int64_t HW, float eps, hipStream_t stream) {                     \
        return bn_plain_forward<F>(x, weight, bias, var, mean, ivar, y, T, B, C, HW, eps, stream); \
    }                                                                                              \
    int bn_plain_backward_stats_##SUFFIX(const F* x, const F* weight, const F* ivar,               \
                                         const F* mean, const F* g, F* grad_weight, F* grad_bias,  \
                                         F* mean_gxhat, F* mean_gxhatx, int64_t T, int64_t B,      \
                                         int64_t C, int64_t HW, F* workspace,                      \
                                         hipStream_t stream) {                                     \
        return bn_plain_backward_stats<F>(x, weight, ivar, mean, g, grad_weight, grad_bias,        \
                                          mean_gxhat, mean_gxhatx, T, B, C, HW, workspace, stream);\
    }                                                                                              \
    int bn_plain_backward_input_##SUFFIX(const F* x, const F* weight, const F* ivar,               \
                                         const F* mean, const F* g, const F* mean_gxhat,           \
                                         const F* mean_gxhatx, F* gx, int64_t T, int64_t B,        \
                                         int64_t C, int64_t HW, hipStream_t stream) {              \
        return bn_plain_backward_input<F>(x, weight, ivar, mean, g, mean_gxhat, mean_gxhatx, gx,   \
                                          T, B, C, HW, stream);                                    \
    }                                                                                              \
    int bn_plain_backward_##SUFFIX(const F* x, const F* weight, const F* ivar, const F* mean,      \
                                   const F* g, F* gx, F* grad_weight, F* grad_bias, int64_t T,     \
                                   int64_t B, int64_t C, int64_t HW, F* workspace,                 \
                                   hipStream_t stream) {                                           \
        return bn_plain_backward<F>(x, weight, ivar, mean, g, gx, grad_weight, grad_bias, T, B, C, \
                                    HW, workspace, stream);                                        \
    }                                                                                              \
    }

#endif  // SNNLIF_LIF_BN_PLAIN_H
