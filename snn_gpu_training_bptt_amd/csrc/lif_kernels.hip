// LIF "fire" forward / backward kernels for MI355X (gfx950, CDNA4) and their C ABI.
//
// What is computed (reference: snnlib/cuda/snn_kernel_fp.cu:37-52, snnlib/cuda/snn_kernel_bp.cu:34-51
// and :117-138; pure-PyTorch statement of the same maths: snnlib/example/gold_op.py:17-44):
//
//   forward, per neuron, u = s = 0 before t = 0:
//       u = (alpha * u) * (1 - s) + x[t];   s = (u > thresh);   spike[t] = s;   (mem[t] = u)
//   backward, per neuron, gu = 0 before t = T-1, walking t downwards:
//       gs = in_window(u[t]) ? g[t] - (gu * alpha) * u[t] : 0
//       gu = gs * beta + (gu * alpha) * (u[t] <= thresh);   gx[t] = gu
//       in_window(u) = (u - thresh) < interval && (thresh - u) < interval
//
// How it is mapped to the machine (nothing here follows the reference's launch geometry, which
// gives one thread a (c,h,w) position and makes it loop serially over the batch):
//   * Tensors are viewed as [T, N] with N = all neurons of the batch.  Neurons are independent and
//     time is the only dependency, so a lane owns V consecutive neurons and walks T itself: the
//     membrane potential, the spike flag and the running gradient never leave VGPRs.
//   * V is chosen so that one lane moves 16 bytes per access (float4 / double2 / 8 x bf16): a
//     64-lane wavefront touches 1 KiB of consecutive addresses per time step, and all T rows (which
//     are N*sizeof apart) are requested before the first value is consumed, so a wavefront keeps
//     T KiB in flight.  That, not occupancy, is what covers HBM latency.
//   * The backward recomputes u[0..T-1] from x into registers (T <= 32) instead of writing a
//     membrane tensor to HBM and reading it back: 12 bytes per neuron-step instead of 20.
//     Gradient rows are streamed in reverse time order through a double-buffered register window.
//   * The op is element-wise and HBM-bound: no LDS, no cross-lane traffic, no MFMA.  Every byte is
//     touched once, so loads and stores carry the non-temporal hint to keep L2 lines for others.
//   * Built with -ffp-contract=off: each product and sum is rounded on its own, as PyTorch's
//     element-wise CPU/GPU ops do, which makes spikes, potentials and gradients bit-identical to
//     the per-op rounded reference arithmetic.
//
// Longer windows (T > 32) use the same forward kernel to write u to a caller-provided workspace
// and a streaming reverse kernel that reads it back.

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

#include "snnlib_lif.h"

#ifndef SNNLIF_BLOCK
#define SNNLIF_BLOCK 256
#endif
#ifndef SNNLIF_NT_LOAD
#define SNNLIF_NT_LOAD 1
#endif
#ifndef SNNLIF_NT_STORE
#define SNNLIF_NT_STORE 1
#endif
// Rows of the gradient held in flight per buffer of the backward's reverse sweep.
#ifndef SNNLIF_BWD_GCHUNK
#define SNNLIF_BWD_GCHUNK 8
#endif

namespace {

constexpr int kBlock = SNNLIF_BLOCK;

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// bfloat16 as raw bits; conversions are done by hand so the rounding is spelled out.
struct bf16_t {
    uint16_t bits;
};

template <int BYTES> struct RawOf;
template <> struct RawOf<2>  { using type = uint16_t; };
template <> struct RawOf<4>  { using type = uint32_t; };
template <> struct RawOf<8>  { using type = u32x2; };
template <> struct RawOf<16> { using type = u32x4; };

// V consecutive elements of storage type S, moved with one memory instruction.
template <typename S, int V>
struct Pack {
    using raw_t = typename RawOf<sizeof(S) * V>::type;
    union {
        raw_t raw;
        S e[V];
    };
};

template <typename S, int V>
__device__ __forceinline__ Pack<S, V> load_pack(const S* p) {
    using raw_t = typename Pack<S, V>::raw_t;
    Pack<S, V> r;
#if SNNLIF_NT_LOAD
    r.raw = __builtin_nontemporal_load(reinterpret_cast<const raw_t*>(p));
#else
    r.raw = *reinterpret_cast<const raw_t*>(p);
#endif
    return r;
}

template <typename S, int V>
__device__ __forceinline__ void store_pack(S* p, const Pack<S, V>& v) {
    using raw_t = typename Pack<S, V>::raw_t;
#if SNNLIF_NT_STORE
    __builtin_nontemporal_store(v.raw, reinterpret_cast<raw_t*>(p));
#else
    *reinterpret_cast<raw_t*>(p) = v.raw;
#endif
}

// Storage type -> arithmetic type and conversions.
template <typename S> struct Arith;
template <> struct Arith<float> {
    using type = float;
    static constexpr int kMaxVec = 4;
    __device__ static __forceinline__ float load(float v) { return v; }
    __device__ static __forceinline__ float store(float v) { return v; }
};
template <> struct Arith<double> {
    using type = double;
    static constexpr int kMaxVec = 2;
    __device__ static __forceinline__ double load(double v) { return v; }
    __device__ static __forceinline__ double store(double v) { return v; }
};
template <> struct Arith<bf16_t> {
    using type = float;
    static constexpr int kMaxVec = 8;
    __device__ static __forceinline__ float load(bf16_t v) {
        return __uint_as_float(static_cast<uint32_t>(v.bits) << 16);
    }
    // Round to nearest, ties to even; every NaN becomes the canonical quiet NaN 0x7FC0.
    __device__ static __forceinline__ bf16_t store(float f) {
        uint32_t u = __float_as_uint(f);
        bf16_t r;
        if ((u & 0x7fffffffu) > 0x7f800000u) {
            r.bits = 0x7fc0;
        } else {
            u += 0x7fffu + ((u >> 16) & 1u);
            r.bits = static_cast<uint16_t>(u >> 16);
        }
        return r;
    }
};

// One forward step for one neuron, in the reference's association:
// ((alpha * u) * (1 - s)) + x, then the strict comparison.
template <typename C>
__device__ __forceinline__ void lif_step(C& u, C& s, C x, C alpha, C thresh) {
    u = (alpha * u) * (C(1) - s) + x;
    s = (u > thresh) ? C(1) : C(0);
}

// One reverse step for one neuron, given the membrane potential u of that step and the incoming
// spike gradient g; gu is the gradient carried from step t+1 and becomes the result of step t.
template <typename C>
__device__ __forceinline__ void lif_reverse_step(C& gu, C u, C g, C alpha, C thresh, C beta,
                                                 C interval) {
    const C gua = gu * alpha;
    C gs = C(0);
    if ((u - thresh) < interval && (thresh - u) < interval) {
        gs = g - gua * u;
    }
    gu = gs * beta + gua * ((u <= thresh) ? C(1) : C(0));
}

// ---------------------------------------------------------------------------------------------
// Forward.  S: storage type of x / spike, M: storage type of the membrane output (S for the
// public op, the arithmetic type when it is the backward's workspace), V: neurons per lane,
// TC: rows requested before the first is consumed.  A window longer than TC is streamed with the
// next TC rows already in flight while the current ones are processed.
// ---------------------------------------------------------------------------------------------
template <typename S, typename M, int V, int TC, bool WRITE_U, bool WRITE_S>
__global__ void __launch_bounds__(kBlock)
lif_forward_kernel(const S* __restrict__ x, M* __restrict__ mem, S* __restrict__ spike, int T,
                   int64_t N, int64_t nvec, typename Arith<S>::type alpha,
                   typename Arith<S>::type thresh) {
    using C = typename Arith<S>::type;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
    for (int64_t v = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; v < nvec;
         v += stride) {
        const int64_t col = v * V;
        C u[V], s[V];
#pragma unroll
        for (int j = 0; j < V; ++j) {
            u[j] = C(0);
            s[j] = C(0);
        }
        Pack<S, V> cur[TC], nxt[TC];
#pragma unroll
        for (int k = 0; k < TC; ++k) {
            if (k < T) cur[k] = load_pack<S, V>(x + static_cast<int64_t>(k) * N + col);
        }
        for (int t0 = 0; t0 < T; t0 += TC) {
            if (t0 + TC < T) {
#pragma unroll
                for (int k = 0; k < TC; ++k) {
                    const int t = t0 + TC + k;
                    if (t < T) nxt[k] = load_pack<S, V>(x + static_cast<int64_t>(t) * N + col);
                }
            }
#pragma unroll
            for (int k = 0; k < TC; ++k) {
                const int t = t0 + k;
                if (t < T) {
                    Pack<M, V> mo;
                    Pack<S, V> so;
#pragma unroll
                    for (int j = 0; j < V; ++j) {
                        lif_step<C>(u[j], s[j], Arith<S>::load(cur[k].e[j]), alpha, thresh);
                        if (WRITE_U) mo.e[j] = Arith<M>::store(u[j]);
                        if (WRITE_S) so.e[j] = Arith<S>::store(s[j]);
                    }
                    const int64_t off = static_cast<int64_t>(t) * N + col;
                    if (WRITE_U) store_pack<M, V>(mem + off, mo);
                    if (WRITE_S) store_pack<S, V>(spike + off, so);
                }
            }
            if (t0 + TC < T) {
#pragma unroll
                for (int k = 0; k < TC; ++k) cur[k] = nxt[k];
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Fused backward for T <= TMAX: recompute u[0..T-1] into registers, then sweep t downwards.
// Gradient rows are fetched GC at a time, the newest time steps first; the fetch of the next
// (earlier) group is issued before the current group is consumed.
// ---------------------------------------------------------------------------------------------
template <typename S, int V, int TMAX>
__global__ void __launch_bounds__(kBlock)
lif_backward_fused_kernel(const S* __restrict__ x, const S* __restrict__ g, S* __restrict__ gx,
                          int T, int64_t N, int64_t nvec, typename Arith<S>::type alpha,
                          typename Arith<S>::type thresh, typename Arith<S>::type beta,
                          typename Arith<S>::type interval) {
    using C = typename Arith<S>::type;
    constexpr int GC = (TMAX < SNNLIF_BWD_GCHUNK) ? TMAX : SNNLIF_BWD_GCHUNK;
    constexpr int NCH = TMAX / GC;
    static_assert(TMAX % GC == 0, "TMAX must be a multiple of the gradient chunk");

    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
    for (int64_t v = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; v < nvec;
         v += stride) {
        const int64_t col = v * V;

        Pack<S, V> xin[TMAX];
#pragma unroll
        for (int t = 0; t < TMAX; ++t) {
            if (t < T) xin[t] = load_pack<S, V>(x + static_cast<int64_t>(t) * N + col);
        }
        Pack<S, V> gbuf[2][GC];
#pragma unroll
        for (int k = 0; k < GC; ++k) {
            const int t = (NCH - 1) * GC + k;
            if (t < T) gbuf[(NCH - 1) & 1][k] = load_pack<S, V>(g + static_cast<int64_t>(t) * N + col);
        }

        C u[TMAX][V];
        {
            C uc[V], sc[V];
#pragma unroll
            for (int j = 0; j < V; ++j) {
                uc[j] = C(0);
                sc[j] = C(0);
            }
#pragma unroll
            for (int t = 0; t < TMAX; ++t) {
                if (t < T) {
#pragma unroll
                    for (int j = 0; j < V; ++j) {
                        lif_step<C>(uc[j], sc[j], Arith<S>::load(xin[t].e[j]), alpha, thresh);
                        u[t][j] = uc[j];
                    }
                }
            }
        }

        C gu[V];
#pragma unroll
        for (int j = 0; j < V; ++j) gu[j] = C(0);

#pragma unroll
        for (int c = NCH - 1; c >= 0; --c) {
            if (c > 0) {
#pragma unroll
                for (int k = 0; k < GC; ++k) {
                    const int t = (c - 1) * GC + k;
                    if (t < T) gbuf[(c - 1) & 1][k] = load_pack<S, V>(g + static_cast<int64_t>(t) * N + col);
                }
            }
#pragma unroll
            for (int k = GC - 1; k >= 0; --k) {
                const int t = c * GC + k;
                if (t < T) {
                    Pack<S, V> out;
#pragma unroll
                    for (int j = 0; j < V; ++j) {
                        lif_reverse_step<C>(gu[j], u[t][j], Arith<S>::load(gbuf[c & 1][k].e[j]),
                                            alpha, thresh, beta, interval);
                        out.e[j] = Arith<S>::store(gu[j]);
                    }
                    store_pack<S, V>(gx + static_cast<int64_t>(t) * N + col, out);
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Streaming backward for long windows: the membrane potential comes from a workspace written by
// lif_forward_kernel<.., WRITE_U>.  Rows are consumed TC at a time from the end of the window.
// ---------------------------------------------------------------------------------------------
template <typename S, int V, int TC>
__global__ void __launch_bounds__(kBlock)
lif_backward_stream_kernel(const typename Arith<S>::type* __restrict__ mem,
                           const S* __restrict__ g, S* __restrict__ gx, int T, int64_t N,
                           int64_t nvec, typename Arith<S>::type alpha,
                           typename Arith<S>::type thresh, typename Arith<S>::type beta,
                           typename Arith<S>::type interval) {
    using C = typename Arith<S>::type;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlock;
    for (int64_t v = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x; v < nvec;
         v += stride) {
        const int64_t col = v * V;
        C gu[V];
#pragma unroll
        for (int j = 0; j < V; ++j) gu[j] = C(0);

        // Group c covers t in [c*TC, c*TC + TC); the last group may be partial.
        const int ngroups = (T + TC - 1) / TC;
        Pack<C, V> mcur[TC], mnxt[TC];
        Pack<S, V> gcur[TC], gnxt[TC];
#pragma unroll
        for (int k = 0; k < TC; ++k) {
            const int t = (ngroups - 1) * TC + k;
            if (t < T) {
                mcur[k] = load_pack<C, V>(mem + static_cast<int64_t>(t) * N + col);
                gcur[k] = load_pack<S, V>(g + static_cast<int64_t>(t) * N + col);
            }
        }
        for (int c = ngroups - 1; c >= 0; --c) {
            if (c > 0) {
#pragma unroll
                for (int k = 0; k < TC; ++k) {
                    const int64_t off = static_cast<int64_t>((c - 1) * TC + k) * N + col;
                    mnxt[k] = load_pack<C, V>(mem + off);
                    gnxt[k] = load_pack<S, V>(g + off);
                }
            }
#pragma unroll
            for (int k = TC - 1; k >= 0; --k) {
                const int t = c * TC + k;
                if (t < T) {
                    Pack<S, V> out;
#pragma unroll
                    for (int j = 0; j < V; ++j) {
                        lif_reverse_step<C>(gu[j], mcur[k].e[j], Arith<S>::load(gcur[k].e[j]),
                                            alpha, thresh, beta, interval);
                        out.e[j] = Arith<S>::store(gu[j]);
                    }
                    store_pack<S, V>(gx + static_cast<int64_t>(t) * N + col, out);
                }
            }
            if (c > 0) {
#pragma unroll
                for (int k = 0; k < TC; ++k) {
                    mcur[k] = mnxt[k];
                    gcur[k] = gnxt[k];
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Host side: argument checks, vector-width selection, launches.
// ---------------------------------------------------------------------------------------------

// Upper bound on blocks per launch; beyond it lanes take further columns in the grid-stride loop.
constexpr int64_t kMaxGrid = int64_t(1) << 24;

inline unsigned grid_for(int64_t nvec) {
    int64_t blocks = (nvec + kBlock - 1) / kBlock;
    if (blocks > kMaxGrid) blocks = kMaxGrid;
    if (blocks < 1) blocks = 1;
    return static_cast<unsigned>(blocks);
}

inline bool aligned_to(const void* p, size_t bytes) {
    return p == nullptr || (reinterpret_cast<uintptr_t>(p) % bytes) == 0;
}

// Largest power-of-two V <= maxv such that rows (N elements apart) and the bases of all given
// pointers stay aligned to V elements.  elem[i] is the element size behind ptrs[i].
inline int pick_vec(int maxv, int64_t N, const void* const* ptrs, const size_t* elem, int n) {
    int v = maxv;
    while (v > 1) {
        bool ok = (N % v) == 0;
        for (int i = 0; ok && i < n; ++i) ok = aligned_to(ptrs[i], elem[i] * v);
        if (ok) break;
        v >>= 1;
    }
    return v;
}

inline int shape_error(int64_t T, int64_t N) {
    if (T < 0 || N < 0) return SNNLIF_ERR_ARG;
    if (T > 0x7fffffff) return SNNLIF_ERR_ARG;
    if (T > 0 && N > (INT64_MAX / 16) / T) return SNNLIF_ERR_ARG;
    return SNNLIF_OK;
}

inline int launch_status() {
    return static_cast<int>(hipGetLastError());
}

template <typename S, typename M, int V, bool WRITE_U, bool WRITE_S>
int launch_forward_v(const S* x, M* mem, S* spike, int64_t T, int64_t N, float alpha, float thresh,
                     hipStream_t stream) {
    using C = typename Arith<S>::type;
    const int64_t nvec = N / V;
    const dim3 grid(grid_for(nvec)), block(kBlock);
    if (T <= 4) {
        hipLaunchKernelGGL((lif_forward_kernel<S, M, V, 4, WRITE_U, WRITE_S>), grid, block, 0, stream,
                           x, mem, spike, static_cast<int>(T), N, nvec, C(alpha), C(thresh));
    } else {
        hipLaunchKernelGGL((lif_forward_kernel<S, M, V, 8, WRITE_U, WRITE_S>), grid, block, 0, stream,
                           x, mem, spike, static_cast<int>(T), N, nvec, C(alpha), C(thresh));
    }
    return launch_status();
}

template <typename S, typename M, bool WRITE_U, bool WRITE_S>
int launch_forward(const S* x, M* mem, S* spike, int64_t T, int64_t N, float alpha, float thresh,
                   hipStream_t stream) {
    constexpr size_t widest = sizeof(S) > sizeof(M) ? sizeof(S) : sizeof(M);
    constexpr int maxv = static_cast<int>(16 / widest);
    const void* ptrs[3] = {x, WRITE_U ? mem : nullptr, WRITE_S ? spike : nullptr};
    const size_t elem[3] = {sizeof(S), sizeof(M), sizeof(S)};
    for (int i = 0; i < 3; ++i)
        if (!aligned_to(ptrs[i], elem[i])) return SNNLIF_ERR_ALIGN;
    const int v = pick_vec(maxv, N, ptrs, elem, 3);
    switch (v) {
        case 8:
            if constexpr (maxv >= 8)
                return launch_forward_v<S, M, 8, WRITE_U, WRITE_S>(x, mem, spike, T, N, alpha, thresh, stream);
            break;
        case 4:
            if constexpr (maxv >= 4)
                return launch_forward_v<S, M, 4, WRITE_U, WRITE_S>(x, mem, spike, T, N, alpha, thresh, stream);
            break;
        case 2:
            if constexpr (maxv >= 2)
                return launch_forward_v<S, M, 2, WRITE_U, WRITE_S>(x, mem, spike, T, N, alpha, thresh, stream);
            break;
        default:
            break;
    }
    return launch_forward_v<S, M, 1, WRITE_U, WRITE_S>(x, mem, spike, T, N, alpha, thresh, stream);
}

template <typename S>
int forward_dispatch(const void* x, void* mem, void* spike, int64_t T, int64_t N, float alpha,
                     float thresh, hipStream_t stream) {
    const S* xs = static_cast<const S*>(x);
    S* ms = static_cast<S*>(mem);
    S* ss = static_cast<S*>(spike);
    if (mem != nullptr && spike != nullptr)
        return launch_forward<S, S, true, true>(xs, ms, ss, T, N, alpha, thresh, stream);
    if (mem != nullptr)
        return launch_forward<S, S, true, false>(xs, ms, nullptr, T, N, alpha, thresh, stream);
    return launch_forward<S, S, false, true>(xs, nullptr, ss, T, N, alpha, thresh, stream);
}

template <typename S, int V, int TMAX>
int launch_backward_fused_vt(const S* x, const S* g, S* gx, int64_t T, int64_t N, float alpha,
                             float thresh, float beta, float interval, hipStream_t stream) {
    using C = typename Arith<S>::type;
    const int64_t nvec = N / V;
    hipLaunchKernelGGL((lif_backward_fused_kernel<S, V, TMAX>), dim3(grid_for(nvec)), dim3(kBlock),
                       0, stream, x, g, gx, static_cast<int>(T), N, nvec, C(alpha), C(thresh),
                       C(beta), C(interval));
    return launch_status();
}

// Register budget of the fused backward: TMAX*V arithmetic values for u plus two gradient
// buffers.  V is capped so that TMAX*V*sizeof(arithmetic)/4 stays within 128 VGPRs.
template <typename S, int TMAX>
constexpr int fused_max_vec() {
    using C = typename Arith<S>::type;
    constexpr int words = static_cast<int>(sizeof(C) / 4);
    constexpr int cap = 128 / (TMAX * words);
    constexpr int hw = Arith<S>::kMaxVec;
    return cap < 1 ? 1 : (cap < hw ? cap : hw);
}

template <typename S, int TMAX>
int launch_backward_fused_t(const S* x, const S* g, S* gx, int64_t T, int64_t N, float alpha,
                            float thresh, float beta, float interval, hipStream_t stream) {
    constexpr int maxv = fused_max_vec<S, TMAX>();
    const void* ptrs[3] = {x, g, gx};
    const size_t elem[3] = {sizeof(S), sizeof(S), sizeof(S)};
    const int v = pick_vec(maxv, N, ptrs, elem, 3);
    switch (v) {
        case 8:
            if constexpr (maxv >= 8)
                return launch_backward_fused_vt<S, 8, TMAX>(x, g, gx, T, N, alpha, thresh, beta, interval, stream);
            break;
        case 4:
            if constexpr (maxv >= 4)
                return launch_backward_fused_vt<S, 4, TMAX>(x, g, gx, T, N, alpha, thresh, beta, interval, stream);
            break;
        case 2:
            if constexpr (maxv >= 2)
                return launch_backward_fused_vt<S, 2, TMAX>(x, g, gx, T, N, alpha, thresh, beta, interval, stream);
            break;
        default:
            break;
    }
    return launch_backward_fused_vt<S, 1, TMAX>(x, g, gx, T, N, alpha, thresh, beta, interval, stream);
}

template <typename S, int V>
int launch_backward_stream_v(const typename Arith<S>::type* mem, const S* g, S* gx, int64_t T,
                             int64_t N, float alpha, float thresh, float beta, float interval,
                             hipStream_t stream) {
    using C = typename Arith<S>::type;
    const int64_t nvec = N / V;
    hipLaunchKernelGGL((lif_backward_stream_kernel<S, V, 8>), dim3(grid_for(nvec)), dim3(kBlock), 0,
                       stream, mem, g, gx, static_cast<int>(T), N, nvec, C(alpha), C(thresh),
                       C(beta), C(interval));
    return launch_status();
}

template <typename S>
int backward_dispatch(const void* x_, const void* g_, void* gx_, int64_t T, int64_t N, float alpha,
                      float thresh, float beta, float interval, void* workspace,
                      size_t workspace_bytes, hipStream_t stream) {
    using C = typename Arith<S>::type;
    const S* x = static_cast<const S*>(x_);
    const S* g = static_cast<const S*>(g_);
    S* gx = static_cast<S*>(gx_);
    if (!aligned_to(x, sizeof(S)) || !aligned_to(g, sizeof(S)) || !aligned_to(gx, sizeof(S)))
        return SNNLIF_ERR_ALIGN;

    if (T <= 4) return launch_backward_fused_t<S, 4>(x, g, gx, T, N, alpha, thresh, beta, interval, stream);
    if (T <= 8) return launch_backward_fused_t<S, 8>(x, g, gx, T, N, alpha, thresh, beta, interval, stream);
    if (T <= 16) return launch_backward_fused_t<S, 16>(x, g, gx, T, N, alpha, thresh, beta, interval, stream);
    if (T <= 32) return launch_backward_fused_t<S, 32>(x, g, gx, T, N, alpha, thresh, beta, interval, stream);
    static_assert(SNNLIF_BP_FUSED_MAX_T == 32, "dispatch above must cover the fused range");

    // Long window: u -> workspace (arithmetic type), then the streaming reverse sweep.
    const size_t need = static_cast<size_t>(T) * static_cast<size_t>(N) * sizeof(C);
    if (workspace == nullptr || workspace_bytes < need) return SNNLIF_ERR_WORKSPACE;
    if (!aligned_to(workspace, 16)) return SNNLIF_ERR_ALIGN;
    C* mem = static_cast<C*>(workspace);
    int rc = launch_forward<S, C, true, false>(x, mem, nullptr, T, N, alpha, thresh, stream);
    if (rc != SNNLIF_OK) return rc;

    constexpr size_t widest = sizeof(S) > sizeof(C) ? sizeof(S) : sizeof(C);
    constexpr int maxv = static_cast<int>(16 / widest);
    const void* ptrs[3] = {mem, g, gx};
    const size_t elem[3] = {sizeof(C), sizeof(S), sizeof(S)};
    const int v = pick_vec(maxv, N, ptrs, elem, 3);
    switch (v) {
        case 4:
            if constexpr (maxv >= 4)
                return launch_backward_stream_v<S, 4>(mem, g, gx, T, N, alpha, thresh, beta, interval, stream);
            break;
        case 2:
            if constexpr (maxv >= 2)
                return launch_backward_stream_v<S, 2>(mem, g, gx, T, N, alpha, thresh, beta, interval, stream);
            break;
        default:
            break;
    }
    return launch_backward_stream_v<S, 1>(mem, g, gx, T, N, alpha, thresh, beta, interval, stream);
}

inline size_t arith_size(int dtype) {
    switch (dtype) {
        case SNNLIF_DTYPE_F32: return sizeof(float);
        case SNNLIF_DTYPE_F64: return sizeof(double);
        case SNNLIF_DTYPE_BF16: return sizeof(float);
        default: return 0;
    }
}

}  // namespace

extern "C" {

int snnlif_abi_version(void) { return SNNLIF_ABI_VERSION; }

const char* snnlif_target_arch(void) { return "gfx950"; }

const char* snnlif_strerror(int code) {
    switch (code) {
        case SNNLIF_OK: return "success";
        case SNNLIF_ERR_ARG: return "snnlif: invalid argument (NULL tensor pointer, negative or overflowing T/N)";
        case SNNLIF_ERR_DTYPE: return "snnlif: unsupported dtype (expected SNNLIF_DTYPE_F32, _F64 or _BF16)";
        case SNNLIF_ERR_WORKSPACE: return "snnlif: workspace missing or smaller than snnlif_fire_bp_workspace_bytes()";
        case SNNLIF_ERR_ALIGN: return "snnlif: pointer not aligned to its element size (workspace: 16 bytes)";
        default: break;
    }
    if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
    return "snnlif: unknown error code";
}

int snnlif_fire_us_fp(const void* spatial, void* mem, void* spike, int dtype, int64_t T, int64_t N,
                      float alpha, float thresh, void* stream) {
    if (arith_size(dtype) == 0) return SNNLIF_ERR_DTYPE;
    const int se = shape_error(T, N);
    if (se != SNNLIF_OK) return se;
    if (T == 0 || N == 0) return SNNLIF_OK;
    if (spatial == nullptr || (mem == nullptr && spike == nullptr)) return SNNLIF_ERR_ARG;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case SNNLIF_DTYPE_F32: return forward_dispatch<float>(spatial, mem, spike, T, N, alpha, thresh, st);
        case SNNLIF_DTYPE_F64: return forward_dispatch<double>(spatial, mem, spike, T, N, alpha, thresh, st);
        default: return forward_dispatch<bf16_t>(spatial, mem, spike, T, N, alpha, thresh, st);
    }
}

int snnlif_fire_s_fp(const void* spatial, void* spike, int dtype, int64_t T, int64_t N,
                     float alpha, float thresh, void* stream) {
    if (arith_size(dtype) == 0) return SNNLIF_ERR_DTYPE;
    const int se = shape_error(T, N);
    if (se != SNNLIF_OK) return se;
    if (T == 0 || N == 0) return SNNLIF_OK;
    if (spike == nullptr) return SNNLIF_ERR_ARG;
    return snnlif_fire_us_fp(spatial, nullptr, spike, dtype, T, N, alpha, thresh, stream);
}

size_t snnlif_fire_bp_workspace_bytes(int dtype, int64_t T, int64_t N) {
    const size_t es = arith_size(dtype);
    if (es == 0 || shape_error(T, N) != SNNLIF_OK) return 0;
    if (T <= SNNLIF_BP_FUSED_MAX_T) return 0;
    return static_cast<size_t>(T) * static_cast<size_t>(N) * es;
}

int snnlif_fire_bp(const void* spatial, const void* grad_spike, void* grad_spatial, int dtype,
                   int64_t T, int64_t N, float alpha, float thresh, float beta, float interval,
                   void* workspace, size_t workspace_bytes, void* stream) {
    if (arith_size(dtype) == 0) return SNNLIF_ERR_DTYPE;
    const int se = shape_error(T, N);
    if (se != SNNLIF_OK) return se;
    if (T == 0 || N == 0) return SNNLIF_OK;
    if (spatial == nullptr || grad_spike == nullptr || grad_spatial == nullptr) return SNNLIF_ERR_ARG;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case SNNLIF_DTYPE_F32:
            return backward_dispatch<float>(spatial, grad_spike, grad_spatial, T, N, alpha, thresh, beta, interval, workspace, workspace_bytes, st);
        case SNNLIF_DTYPE_F64:
            return backward_dispatch<double>(spatial, grad_spike, grad_spatial, T, N, alpha, thresh, beta, interval, workspace, workspace_bytes, st);
        default:
            return backward_dispatch<bf16_t>(spatial, grad_spike, grad_spatial, T, N, alpha, thresh, beta, interval, workspace, workspace_bytes, st);
    }
}

}  // extern "C"
