// Per-channel batch statistics of a [T, B, C, HW] activation for MI355X: mean and biased variance over
// (T, B, HW), or the first two raw moments E[x], E[x^2] that a batch sharded over several GPUs
// all-reduces, or the plain per-channel sum (F = float or double).
//
// Reference: the layers compute these with framework reductions before calling the native op --
// torch.var_mean(x, dim_bn, unbiased=False) in snnlib/example/snnlib_op.py:44, 78, 122, 184
// and torch.mean(x), torch.mean(x**2) in the sharded layers, snnlib/example/snnlib_op.py:265-266,
// 328-329, 388-389.  On MI355X the framework's Welford reduction over a [8,64,128,32,32] tensor runs at
// 0.7 TB/s and costs five times the fused batch-norm + fire forward it feeds, so the statistics get a
// kernel of their own.  The per-channel sum is the bias gradient of the layers with a convolution,
// at::sum(grad_conv, dim_conv) in snnlib/cuda/snn_kernel_bp.cu:1261, 1338, 1401, 1435 (on a
// [8,64,128,32,32] gradient the framework's reduction takes 148 us where this pass takes 43).
//
// One pass over x (4 bytes per neuron-step in fp32), HBM-bound, two kernels:
//   1. partial sums.  Planes of at least 32 positions: wavefronts are laid over the (batch entry,
//      channel) planes as in sweep 1 of the batch-norm backward (ceil(HW/64) wavefronts per plane,
//      all lanes of a wavefront share a channel); a lane adds up its neuron's T values (requested
//      sixteen at a time, summed in double; windows of fewer than sixteen steps: the values of several
//      batch entries, so that sixteen requests are in flight all the same), the wavefront
//      folds the 64 lanes by shuffles and leaves one pair of sums (doubles, whatever the storage type).  Smaller planes (fully
//      connected shapes): one lane per (channel, position) column of the [T*B, C*HW] matrix, the rows
//      dealt round-robin to S slices of workgroups; consecutive lanes read consecutive addresses.
//   2. one workgroup per channel adds the partial sums in double precision, in an order fixed by the
//      launch geometry (results are reproducible), and writes the two statistics.
// Sums are taken of d = x - K[c] with K[c] the channel's first element (t = 0, b = 0, position 0):
// a shift by any sample of the channel keeps sum(d)^2/n and sum(d^2) of comparable size, so that
// var = (sum(d^2) - sum(d)^2/n)/n does not cancel even when |mean| >> sqrt(var) (the textbook shifted
// two-sum formula); mean = K + sum(d)/n.  d, d^2 and every sum are formed in double precision (the
// subtraction is then exact for fp32 storage), so a shift that happens to be an outlier -- D standard
// deviations from the mean -- costs about 1e-16 * D^2 of relative accuracy in the variance, not
// 6e-8 * D^2 as squares taken in fp32 would.
#ifndef SNNLIF_LIF_BN_STATS_H
#define SNNLIF_LIF_BN_STATS_H

#include "lif_bn.h"
#include "lif_bn_kernels.h"

namespace snnlif {

// Rows requested before the first is consumed, and wavefronts per SIMD of the partial-sum kernels.
// (SNNLIF_STATS_ROWS: lif_bn.h, which also sizes the row slices by it.)
#ifndef SNNLIF_STATS_WAVES
#define SNNLIF_STATS_WAVES 8
#endif
constexpr int kStatsRows = SNNLIF_STATS_ROWS;

// Bytes per load of a lane of the plane-aligned kernel.  One element per lane, as in the fire
// kernels: measured on MI355X at [8,64,128,32,32] with nothing cached, dword lanes read at 72 % of
// the HBM peak, 8-byte lanes at 62 %, 16-byte lanes at 57-68 % depending on the workgroup size.
#ifndef SNNLIF_STATS_LANE_BYTES
#define SNNLIF_STATS_LANE_BYTES 4
#endif

// Adds kStatsRows x V values to the running sums of d and d*d, d = value - shift, all in double.
template <typename F, int V>
__device__ __forceinline__ void stats_add_group(const Pack<F, V> (&v)[kStatsRows], double shift,
                                                double& acc_d, double& acc_dd) {
#pragma unroll
    for (int r = 0; r < kStatsRows; ++r) {
#pragma unroll
        for (int j = 0; j < V; ++j) {
            const double d = static_cast<double>(v[r].e[j]) - shift;
            acc_d += d;
            acc_dd += d * d;
        }
    }
}

template <typename F, int V>
__device__ __forceinline__ Pack<F, V> stats_fill(F value) {
    Pack<F, V> p;
#pragma unroll
    for (int j = 0; j < V; ++j) p.e[j] = value;
    return p;
}

// Planes of at least 32 positions.  A wavefront covers 64*V consecutive positions of one channel
// (G = ceil(HW / (64*V)) wavefronts per plane; HW is a multiple of V) and sums a set of rows of the
// [rows = T*B, C*HW] matrix (row t*B + b) there; part_* indexed [slice][channel][chunk].
//   SLICED = false (windows of at least kStatsRows steps): S = B slices, slice b = the T rows of
//       batch entry b, `step` = B*C*HW elements apart, kStatsRows at a time;
//   SLICED = true (shorter windows): S = rows / kStatsRows slices of consecutive rows (slice s = rows
//       [s * rps, (s + 1) * rps), rps = ceil(rows / S)), so that a lane still has kStatsRows requests in
//       flight: it sums the values of several batch entries.  `step` = C*HW.
template <typename F, int V, bool SLICED>
__global__ void __launch_bounds__(kStatsBlock) SNNLIF_WAVES_PER_SIMD(SNNLIF_STATS_WAVES)
bn_stats_wave_kernel(const F* __restrict__ x, double* __restrict__ part_d,
                     double* __restrict__ part_dd, int rows, int64_t step, int64_t C, int64_t HW,
                     int64_t G, int64_t S) {
    const int64_t lanes = S * C * G * 64;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t pc = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; pc < lanes;
         pc += stride) {
        const int64_t wave = pc >> 6;
        const int64_t plane = wave / G;  // slice * C + channel
        const int64_t k = ((wave - plane * G) * 64 + (pc & 63)) * V;
        const int c = static_cast<int>(plane % C);
        double acc_d = 0.0, acc_dd = 0.0;
        if (k < HW) {
            const double shift = static_cast<double>(x[static_cast<int64_t>(c) * HW]);
            // first row of the slice; its further rows are `step` elements apart
            const int64_t slice = plane / C;
            const int rps = SLICED ? static_cast<int>((rows + S - 1) / S) : rows;
            const int64_t first = SLICED ? slice * rps : 0;
            const F* col = SLICED ? x + first * step + static_cast<int64_t>(c) * HW + k : x + plane * HW + k;
            const int64_t hop = step;
            const int left = rows - static_cast<int>(first);
            const int count = SLICED ? (left < rps ? (left < 0 ? 0 : left) : rps) : rows;
            int t0 = 0;
            for (; t0 + kStatsRows <= count; t0 += kStatsRows) {  // whole groups: straight-line loads
                Pack<F, V> v[kStatsRows];
#pragma unroll
                for (int r = 0; r < kStatsRows; ++r)
                    v[r] = load_pack<F, V, false>(col + static_cast<int64_t>(t0 + r) * hop);
                stats_add_group<F, V>(v, shift, acc_d, acc_dd);
            }
            if (t0 < count) {
                Pack<F, V> v[kStatsRows];
#pragma unroll
                for (int r = 0; r < kStatsRows; ++r) {
                    v[r] = stats_fill<F, V>(x[static_cast<int64_t>(c) * HW]);  // rows past the end: d = 0
                    if (t0 + r < count)
                        v[r] = load_pack<F, V, false>(col + static_cast<int64_t>(t0 + r) * hop);
                }
                stats_add_group<F, V>(v, shift, acc_d, acc_dd);
            }
        }
        acc_d = wave_sum(acc_d);
        acc_dd = wave_sum(acc_dd);
        if ((pc & 63) == 0) {
            part_d[wave] = acc_d;
            part_dd[wave] = acc_dd;
        }
    }
}

// Planes of fewer than 32 positions: the tensor as a [rows = T*B, CHW] matrix.  Workgroup
// (blockIdx.x, blockIdx.y = slice s) sums rows s, s+S, s+2S, ... of its 256 columns.
// part_* indexed [slice][column].
template <typename F>
__global__ void __launch_bounds__(kStatsBlock)
bn_stats_column_kernel(const F* __restrict__ x, double* __restrict__ part_d,
                       double* __restrict__ part_dd, int64_t rows, int64_t CHW, int64_t HW, int S) {
    const int64_t j = static_cast<int64_t>(blockIdx.x) * kStatsBlock + threadIdx.x;
    if (j >= CHW) return;
    const int s = blockIdx.y;
    const F first_of_channel = x[(j / HW) * HW];
    const double shift = static_cast<double>(first_of_channel);
    double acc_d = 0.0, acc_dd = 0.0;
    for (int64_t r0 = s; r0 < rows; r0 += static_cast<int64_t>(S) * kStatsRows) {
        Pack<F, 1> v[kStatsRows];
#pragma unroll
        for (int q = 0; q < kStatsRows; ++q) {
            const int64_t r = r0 + static_cast<int64_t>(q) * S;
            v[q] = stats_fill<F, 1>(first_of_channel);
            if (r < rows) v[q] = load_pack<F, 1, false>(x + r * CHW + j);
        }
        stats_add_group<F, 1>(v, shift, acc_d, acc_dd);
    }
    part_d[static_cast<int64_t>(s) * CHW + j] = acc_d;
    part_dd[static_cast<int64_t>(s) * CHW + j] = acc_dd;
}

// One workgroup per channel: adds the channel's partial sums in double and writes
//   mode kStatsVariance:  out_a = mean,  out_b = biased variance
//   mode kStatsMoments:   out_a = E[x],  out_b = E[x^2]
//   mode kStatsSums:      out_a = sum of x,  out_b not touched
// Wave layout: entries (b*C + c)*G + i for b < B, i < G.  Column layout: entries s*CHW + c*HW + i for
// s < S, i < HW.  Both are "outer" groups of "inner" consecutive entries, outer_stride apart.
template <typename F>
__global__ void __launch_bounds__(kReduceBlock)
bn_stats_finalize_kernel(const F* __restrict__ x, const double* __restrict__ part_d,
                         const double* __restrict__ part_dd, F* __restrict__ out_a,
                         F* __restrict__ out_b, int64_t HW, int64_t outer, int64_t inner,
                         int64_t outer_stride, double count, int mode, RunningUpdate<F> running) {
    const int c = blockIdx.x;
    const int64_t base = static_cast<int64_t>(c) * inner;
    const int64_t n = outer * inner;
    double a = 0.0, aa = 0.0;
    for (int64_t e = threadIdx.x; e < n; e += kReduceBlock) {
        const int64_t at = (e / inner) * outer_stride + base + (e % inner);
        a += part_d[at];
        aa += part_dd[at];
    }
    __shared__ double lds[2][kReduceBlock / 64];
    a = wave_sum(a);
    aa = wave_sum(aa);
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    if (lane == 0) {
        lds[0][wave] = a;
        lds[1][wave] = aa;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        double sd = 0.0, sdd = 0.0;
#pragma unroll
        for (int w = 0; w < kReduceBlock / 64; ++w) {
            sd += lds[0][w];
            sdd += lds[1][w];
        }
        const double shift = static_cast<double>(x[static_cast<int64_t>(c) * HW]);
        if (mode == kStatsSums) {  // the plain sum: out_b is not written
            out_a[c] = static_cast<F>(shift * count + sd);
            return;
        }
        const double mean_d = sd / count;
        double var = (sdd - sd * mean_d) / count;
        if (var < 0.0) var = 0.0;
        const double mean = shift + mean_d;
        const F mean_f = static_cast<F>(mean);
        const F second_f = static_cast<F>(mode == kStatsMoments ? var + mean * mean : var);
        out_a[c] = mean_f;
        out_b[c] = second_f;
        if (running.mean_out != nullptr) {  // (mode kStatsVariance) from the rounded statistics, as a reader of out_* would
            running.mean_out[c] = running.mean_in[c] * running.keep + mean_f * running.gain_mean;
            running.var_out[c] = running.var_in[c] * running.keep + second_f * running.gain_var;
        }
    }
}

template <typename F>
int bn_stats(const F* x, F* out_a, F* out_b, int mode, int64_t T, int64_t B, int64_t C,
             int64_t HW, double* workspace, hipStream_t stream, const RunningUpdate<F>& running) {
    const int64_t N = B * C * HW;
    const size_t P = bn_stats_partial_count(T, B, C, HW);
    double* part_d = workspace;
    double* part_dd = workspace + P;
    const double count = static_cast<double>(T) * static_cast<double>(B) * static_cast<double>(HW);
    if (bn_wave_partials(HW)) {
        // widest lanes for which rows, planes and the base address stay aligned and a wavefront
        // still has work for most of its lanes (the partial-sum arrays are sized for V = 1, the
        // case with the most wavefronts per plane)
        constexpr int maxv = SNNLIF_STATS_LANE_BYTES / static_cast<int>(sizeof(F)) < 1
                                 ? 1
                                 : SNNLIF_STATS_LANE_BYTES / static_cast<int>(sizeof(F));
        int v = maxv;
        while (v > 1 && (HW % v != 0 || HW < 64 * v || !aligned_to(x, sizeof(F) * v))) v >>= 1;
        const int64_t G = (HW + 64 * v - 1) / (64 * v);
        const int64_t S = bn_stats_wave_slices(T, B);
        const dim3 grid(grid_for(S * C * G * 64, kStatsBlock)), block(kStatsBlock);
        const int rc = with_vec<maxv>(v, [&](auto vc) {
            constexpr int V = decltype(vc)::value;
            if (S == B)  // slice b = batch entry b: its T rows, N elements apart
                launch_kernel(bn_stats_wave_kernel<F, V, false>, grid, block, 0, stream, x, part_d,
                              part_dd, static_cast<int>(T), N, C, HW, G, S);
            else  // row s of the [T*B, C*HW] matrix starts slice s
                launch_kernel(bn_stats_wave_kernel<F, V, true>, grid, block, 0, stream, x, part_d,
                              part_dd, static_cast<int>(T * B), C * HW, C, HW, G, S);
            return launch_status();
        });
        if (rc != SNNLIF_OK) return rc;
        launch_kernel(bn_stats_finalize_kernel<F>, dim3(static_cast<unsigned>(C)), dim3(kReduceBlock),
                      0, stream, x, part_d, part_dd, out_a, out_b, HW, S, G, C * G, count, mode, running);
        return launch_status();
    }
    const int64_t rows = T * B, CHW = C * HW;
    const int S = bn_stats_row_slices(rows, CHW);
    launch_kernel(bn_stats_column_kernel<F>,
                  dim3(static_cast<unsigned>((CHW + kStatsBlock - 1) / kStatsBlock), S),
                  dim3(kStatsBlock), 0, stream, x, part_d, part_dd, rows, CHW, HW, S);
    int rc = launch_status();
    if (rc != SNNLIF_OK) return rc;
    launch_kernel(bn_stats_finalize_kernel<F>, dim3(static_cast<unsigned>(C)), dim3(kReduceBlock), 0,
                  stream, x, part_d, part_dd, out_a, out_b, HW, static_cast<int64_t>(S), HW, CHW, count,
                  mode, running);
    return launch_status();
}

// Statistics of a sharded batch from its all-reduced moments, as the reference's sharded layers form
// them (snnlib/example/snnlib_op.py:271-275): mean = first / world, var = second / world - mean^2 (the
// framework divides by a scalar as a multiplication by its reciprocal, and squares by a product), and
// the running pair.  One lane per channel.
template <typename F>
__global__ void __launch_bounds__(kReduceBlock)
bn_moments_finish_kernel(const F* __restrict__ first, const F* __restrict__ second,
                         F* __restrict__ mean, F* __restrict__ var, F inv_world,
                         RunningUpdate<F> running, int64_t C) {
    const int64_t c = static_cast<int64_t>(blockIdx.x) * kReduceBlock + threadIdx.x;
    if (c >= C) return;
    const F m = first[c] * inv_world;
    const F v = second[c] * inv_world - m * m;
    mean[c] = m;
    var[c] = v;
    if (running.mean_out != nullptr) {
        running.mean_out[c] = running.mean_in[c] * running.keep + m * running.gain_mean;
        running.var_out[c] = running.var_in[c] * running.keep + v * running.gain_var;
    }
}

template <typename F>
int bn_moments_finish(const F* first, const F* second, F* mean, F* var, F inv_world,
                      const RunningUpdate<F>& running, int64_t C, hipStream_t stream) {
    launch_kernel(bn_moments_finish_kernel<F>,
                  dim3(static_cast<unsigned>((C + kReduceBlock - 1) / kReduceBlock)), dim3(kReduceBlock),
                  0, stream, first, second, mean, var, inv_world, running, C);
    return launch_status();
}

}  // namespace snnlif

#define SNNLIF_DEFINE_BN_STATS_DTYPE(SUFFIX, F)                                                    \
    namespace snnlif {                                                                             \
    int bn_stats_##SUFFIX(const F* x, F* out_a, F* out_b, int mode, int64_t T, int64_t B,          \
                          int64_t C, int64_t HW, double* workspace, hipStream_t stream,            \
                          const RunningUpdate<F>& running) {                                       \
        return bn_stats<F>(x, out_a, out_b, mode, T, B, C, HW, workspace, stream, running);        \
    }                                                                                              \
    int bn_moments_finish_##SUFFIX(const F* first, const F* second, F* mean, F* var, F inv_world,  \
                                   const RunningUpdate<F>& running, int64_t C,                     \
                                   hipStream_t stream) {                                           \
        return bn_moments_finish<F>(first, second, mean, var, inv_world, running, C, stream);      \
    }                                                                                              \
    }

#endif  // SNNLIF_LIF_BN_STATS_H
