// LIF "fire" forward / backward kernels for MI355X (gfx950, CDNA4): templates shared by the
// per-dtype translation units (lif_f32.hip, lif_f64.hip, lif_bf16.hip).
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
//   * A lane moves one dword per access (V = 1 float, 2 bf16; a double takes two dwords): a
//     64-lane wavefront touches 256 consecutive bytes per time step, and all T rows (which are
//     N*sizeof apart) are requested before the first value is consumed.  Measured on MI355X this
//     beats 16-byte lanes by 5-15 %: the narrow kernels need ~25 VGPRs, so every SIMD holds its full
//     8 waves, and the many small in-flight requests of one wave stay within a few DRAM pages per
//     row instead of spreading over sixteen.  It also removes every alignment constraint for fp32
//     and fp64 (element alignment is all a dword lane needs).  Windows of one or two steps are the
//     exception: too few rows per lane to fill the memory pipeline, so they take 16-byte lanes
//     when N and the base addresses allow it.
//   * The backward recomputes u[0..T-1] from x into registers (T <= 32) instead of writing a
//     membrane tensor to HBM and reading it back: 12 bytes per neuron-step instead of 20.
//     Gradient rows are streamed in reverse time order through a double-buffered register window.
//     The register-resident window needs compile-time row indices, so the kernel is instantiated
//     per window length (1-8, then multiples of 2, 4 and 8); every other length runs the multiple
//     of 8 below it as a straight-line body preceded by a head of up to 7 steps, the only rows
//     behind run-time tests (per-row control flow around the whole window costs the compiler
//     hundreds of VGPRs).
//   * The op is element-wise and HBM-bound: no LDS, no cross-lane traffic, no MFMA.
//   * Cache policy and launch shape follow what the caller says about the input current x
//     (template parameter KEEP of the kernels, SNNLIF_KEEP_SPATIAL of the C ABI):
//       - streamed (the default): x is read once per kernel from HBM, like every other tensor, with
//         the non-temporal hint.  This is the case of a network, where whole layers run between a
//         layer's forward and its backward.  Measured with nothing cached, the DRAM then prefers
//         fewer and larger streams in flight: 256-thread workgroups throughout and the backward
//         capped at 4-5 wavefronts per SIMD (+5-9 points of bandwidth over the shape below).
//       - kept: the caller will read x again soon (the backward straight after the forward, the same
//         x step after step).  x is then loaded with the default policy and may stay in the 256 MB
//         memory-side cache, spikes and gradients keep the non-temporal hint so they do not displace
//         it, the forward walks the neuron axis upwards and the backward downwards (whatever part of
//         x is still cached when the backward starts is what it asks for first), and small
//         workgroups with all 8 wavefronts per SIMD resident serve cache hits best.
//     Without a word from the caller tensors of at most 32 MiB are treated as kept (at that size a
//     launch is latency-bound and the tensor is likely to be cache-resident whatever lies between its
//     two readers) and larger ones as streamed.
//   * Built with -ffp-contract=off: each product and sum is rounded on its own, as PyTorch's
//     element-wise CPU/GPU ops do, which makes spikes, potentials and gradients bit-identical to
//     the per-op rounded reference arithmetic.
//
// Windows of up to 111 steps (71 with fp64 arithmetic; bf16 with a head up to 63) still run as one
// register window.  Other longer windows (up to 1024 steps) are cut into 32-step segments: one forward pass leaves the
// membrane potential at the segment boundaries in LDS, then each segment is recomputed into registers
// and swept in reverse, last segment first (x is read twice, nothing else changes).  Beyond that the
// forward kernel writes u to a caller-provided workspace and a streaming reverse kernel reads it back.
#ifndef SNNLIF_LIF_KERNELS_H
#define SNNLIF_LIF_KERNELS_H

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <cstddef>
#include <cstdint>
#include <tuple>
#include <type_traits>

#include "snnlib_lif.h"

// Bytes one lane moves per memory instruction (storage types narrower than this are packed).
#ifndef SNNLIF_LANE_BYTES
#define SNNLIF_LANE_BYTES 4
#endif
// Threads per workgroup of the forward / backward kernels.
#ifndef SNNLIF_FWD_BLOCK
#define SNNLIF_FWD_BLOCK 256
#endif
#ifndef SNNLIF_BWD_BLOCK
#define SNNLIF_BWD_BLOCK 256
#endif
// Largest tensor (bytes) for which the fused backward / the forward use their small workgroups.
#ifndef SNNLIF_SMALL_TENSOR_BYTES
#define SNNLIF_SMALL_TENSOR_BYTES (size_t(160) << 20)
#endif
#ifndef SNNLIF_SMALL_TENSOR_BYTES_FWD
#define SNNLIF_SMALL_TENSOR_BYTES_FWD (size_t(256) << 20)
#endif
// Windows of at most this many steps give a lane too few rows to keep enough bytes in flight with
// one dword per access; they use 16-byte lanes instead (4 fp32 / 2 fp64 / 8 bf16 neurons per lane).
#ifndef SNNLIF_WIDE_LANE_MAX_T
#define SNNLIF_WIDE_LANE_MAX_T 2
#endif
// VGPR budget (in 32-bit words) the fused backward may spend on the recomputed membrane potential.
#ifndef SNNLIF_FUSED_U_WORDS
#define SNNLIF_FUSED_U_WORDS 128
#endif
// Longest window run as one register window when its length is a multiple of 8 steps: with 4-byte
// arithmetic, and with 8-byte arithmetic (two VGPRs per potential).
#ifndef SNNLIF_BWD_WIDE_MAX_T
#define SNNLIF_BWD_WIDE_MAX_T 104
#endif
#ifndef SNNLIF_BWD_WIDE_MAX_T_F64
#define SNNLIF_BWD_WIDE_MAX_T_F64 64
#endif
// Column order of the fused backward: 1 = workgroups walk the neuron axis from its end, i.e.
// opposite to the forward (the cached tail of x is consumed before it can be displaced).
#ifndef SNNLIF_BWD_DESCENDING
#define SNNLIF_BWD_DESCENDING 1
#endif
// Tensors of at most this many bytes are handled as "kept" whatever the caller says (see above).
#ifndef SNNLIF_RESIDENT_TENSOR_BYTES
#define SNNLIF_RESIDENT_TENSOR_BYTES (size_t(32) << 20)
#endif
// Streamed policy: workgroup size of both kernels, wavefronts per SIMD of the backward for windows
// of at most 8 rows / longer ones, of the forward for windows of 9 to 16 rows / longer ones.
#ifndef SNNLIF_STREAM_BLOCK
#define SNNLIF_STREAM_BLOCK 256
#endif
#ifndef SNNLIF_STREAM_SMALL_BLOCK  // ... for tensors of at most SNNLIF_STREAM_SMALL_BYTES
#define SNNLIF_STREAM_SMALL_BLOCK 128
#endif
#ifndef SNNLIF_STREAM_SMALL_BYTES
#define SNNLIF_STREAM_SMALL_BYTES (size_t(128) << 20)
#endif
#ifndef SNNLIF_STREAM_BWD_WAVES_SHORT
#define SNNLIF_STREAM_BWD_WAVES_SHORT 5
#endif
#ifndef SNNLIF_STREAM_BWD_WAVES_LONG
#define SNNLIF_STREAM_BWD_WAVES_LONG 4
#endif
#ifndef SNNLIF_STREAM_BWD_WAVES_LONGER  // windows of 13 to 24 rows / 25 to 64 / beyond
#define SNNLIF_STREAM_BWD_WAVES_LONGER 3
#endif
#ifndef SNNLIF_STREAM_BWD_WAVES_LONGEST
#define SNNLIF_STREAM_BWD_WAVES_LONGEST 2
#endif
#ifndef SNNLIF_STREAM_BWD_WAVES_WIDE
#define SNNLIF_STREAM_BWD_WAVES_WIDE 2
#endif
#ifndef SNNLIF_STREAM_BWD_WAVES_3  // windows of exactly 3 / 4 rows
#define SNNLIF_STREAM_BWD_WAVES_3 8
#endif
#ifndef SNNLIF_STREAM_BWD_WAVES_4
#define SNNLIF_STREAM_BWD_WAVES_4 7
#endif
#ifndef SNNLIF_STREAM_FWD_WAVES_MID
#define SNNLIF_STREAM_FWD_WAVES_MID 4
#endif
#ifndef SNNLIF_STREAM_FWD_WAVES_LONG
#define SNNLIF_STREAM_FWD_WAVES_LONG 3
#endif
// Rows the streamed forward requests at once: windows of 9 rows up to the first run whole in that
// instantiation, windows up to halfway between the two in an instantiation of that many rows, longer
// ones up to the second in that one.
#ifndef SNNLIF_STREAM_FWD_ROWS_MID
#define SNNLIF_STREAM_FWD_ROWS_MID 16
#endif
#ifndef SNNLIF_STREAM_FWD_ROWS_LONG
#define SNNLIF_STREAM_FWD_ROWS_LONG 32
#endif
// Rows of x the forward requests before consuming the first (windows longer than this are
// streamed with the next group of rows in flight).
#ifndef SNNLIF_FWD_ROWS
#define SNNLIF_FWD_ROWS 8
#endif
// Backward windows longer than this fix their instruction schedule (see backward_window).
#ifndef SNNLIF_BWD_PIN_MIN_TW
#define SNNLIF_BWD_PIN_MIN_TW 32
#endif
// Rows of the gradient held in flight per buffer of the backward's reverse sweep.
#ifndef SNNLIF_BWD_GCHUNK
#define SNNLIF_BWD_GCHUNK 8
#endif

// Upper bound on resident wavefronts per SIMD of a kernel (the compiler spends the freed register
// budget; the hardware then cannot co-schedule more).
#define SNNLIF_WAVES_PER_SIMD(n) __attribute__((amdgpu_waves_per_eu(1, (n))))

namespace snnlif {

// Wavefronts per SIMD the backward kernels allow themselves for a register window of `rows` time
// steps.  A wavefront keeps 2*rows row requests in flight.
// Kept x (part of the traffic served by the memory-side cache): past roughly 100 requests per SIMD the
// streams of different wavefronts start to evict each other's DRAM pages (-4 % at 16 rows and -9 % at
// 32 rows with all 8 wavefronts resident; windows of up to 8 rows are best left uncapped).
// Streamed x (everything from HBM): fewer wavefronts already pay for windows of 5 to 8 rows (8 rows:
// 84 % of peak at 5 wavefronts against 78 % at 8), while windows of 3 and 4 rows need 8 and 7 to keep
// enough requests going (cold, 256 MiB tensors: 3 rows 71 -> 83 %, 4 rows 76 -> 84 % against 5
// wavefronts; 5 rows and more lose 1-6 points beyond 5); windows of 9-12 rows run 4, 13-24 rows 3 (16
// rows 80.0 -> 81.4 %, 20 rows 77.6 -> 78.8, 24 rows 77.8 -> 79.2 against 4), 25-64 rows 2 (32 rows
// 76.3 -> 77.5, 40 rows 75.4 -> 77.2, 64 rows 68.5 -> 70.7), and so do the windows beyond 64 rows (72
// rows 67.7 -> 69.1, 80 rows 72.8 -> 74.5, 96 rows 70.4 -> 73.4 against 3).  SNNLIF_BWD_MAX_WAVES
// overrides both.
constexpr int backward_waves(int rows, bool keep = true) {
#ifdef SNNLIF_BWD_MAX_WAVES
    return SNNLIF_BWD_MAX_WAVES;
#else
    if (!keep) {
        if (rows == 3) return SNNLIF_STREAM_BWD_WAVES_3;
        if (rows == 4) return SNNLIF_STREAM_BWD_WAVES_4;
        if (rows <= 8) return SNNLIF_STREAM_BWD_WAVES_SHORT;
        if (rows <= 12) return SNNLIF_STREAM_BWD_WAVES_LONG;
        if (rows <= 24) return SNNLIF_STREAM_BWD_WAVES_LONGER;
        return rows > 64 ? SNNLIF_STREAM_BWD_WAVES_WIDE : SNNLIF_STREAM_BWD_WAVES_LONGEST;
    }
    if (rows > 64) return 3;  // u alone takes `rows` VGPRs per lane
    return rows <= 8 ? 8 : (rows <= 12 ? 5 : 4);
#endif
}

// Streamed backward on tensors of at most SNNLIF_STREAM_SMALL_BYTES: windows of 4 to 16 steps run with
// fewer wavefronts still (0: no instantiation of its own).  Measured cold over 2-8 wavefronts, fp32, %
// of the HBM peak at this figure / at the one above: 4 steps on 128 MiB tensors 78.6 / 75.8, on 64 MiB
// 70.5 / 69.2; 6 steps on 96 MiB 73.7 / 71.2; 7 steps on 112 MiB 73.8 / 70.3; 8 steps on 128 MiB
// 72.8 / 68.8, on 64 MiB 73.4 / 70.1; 12 steps on 96 MiB 73.3 / 71.9; 16 steps on 128 MiB 73.4 / 71.5;
// bf16 8 steps on 128 MiB 72.8 / 68.5.  Larger tensors are best at the figures above (8 steps on
// 256 MiB: 84.6 % at 4 wavefronts, 83.1 at 5; on 512 MiB 82.6 / 83.3).
constexpr int stream_backward_small_waves(int rows) {
    return rows == 4 ? 5 : (rows >= 5 && rows <= 16) ? 3 : 0;
}

// The forward keeps `rows` (twice that when the window is streamed in groups) requests per wavefront
// in flight; long streamed windows gain from a cap.  `cap` > 0: the instantiation's own figure
// (streamed windows of up to 8 steps, see stream_forward_waves).
constexpr int forward_waves(int rows, bool keep, int cap = 0) {
#ifdef SNNLIF_FWD_MAX_WAVES
    return SNNLIF_FWD_MAX_WAVES;
#else
    if (cap > 0) return cap;
    if (!keep && rows > SNNLIF_STREAM_FWD_ROWS_MID) return SNNLIF_STREAM_FWD_WAVES_LONG;
    return (!keep && rows > 8) ? SNNLIF_STREAM_FWD_WAVES_MID : 8;  // groups of SNNLIF_STREAM_FWD_ROWS_MID too
#endif
}

// Wavefronts per SIMD of the straight-line instantiation of the streamed forward for a window of `rows`
// steps (one of those launch_forward_v lists).  Measured cold over 2-8 wavefronts, fp32, % of the HBM peak at the best / at
// 8 wavefronts: 8 steps 78 / 76 (256 MiB tensors, best at 5), 80 / 79 (512 MiB, 5), 69 / 62 (128 MiB, 3);
// 7 steps 77 / 76.5 (224 MiB, 5), 69 / 63.5 (112 MiB, 3); 6 steps 76 / 75 (192 MiB, 5), 68 / 64 (96 MiB,
// 4); 5 steps 75 / 72.5 (160 MiB, 5-7), 68 / 67 (80 MiB, 5); 4 and 3 steps are best at 7-8 at every size
// (3 steps: 72 % at 8, 63 % at 5); bf16 8 steps on 256 MiB tensors 81 / 76.5 (5).
// Longer windows: 10 steps 71 -> 78 % at 4 wavefronts against the 16-row instantiation with a test
// around each row; 12 steps at 3: 74 -> 77 % (256 MiB), 69.6 -> 71 (128 MiB); 16 steps gain only on
// tensors of at most 128 MiB, at 2 wavefronts (67 -> 72.7 %; 64 MiB 63 -> 66.5), and lose 2-6 points on
// larger ones; 20 / 24 / 28 steps at 2: 72 -> 77 % / 74 -> 79 / 73 -> 76 (256 MiB tensors) against the
// 24- and 32-row instantiations with tests, 32 steps 72.5 -> 73.8 against the rolling window.
// 0: no straight-line instantiation for this length and size.
inline int stream_forward_waves(int rows, size_t tensor_bytes) {
    const bool small = tensor_bytes <= static_cast<size_t>(SNNLIF_STREAM_SMALL_BYTES);
    if (rows == 20 || rows == 24 || rows == 28 || rows == 32) return 2;
    if (rows == 16) return small ? 2 : 0;
    if (rows == 12) return 3;
    if (rows == 10) return 4;
    if (rows > 8) return 0;
    if (rows >= 7) return small ? 3 : 5;
    if (rows == 6) return small ? 4 : 5;
    if (rows == 5) return 5;
    return 8;
}

constexpr int kLaneBytes = SNNLIF_LANE_BYTES;
constexpr int lane_vec(size_t elem_bytes) {
    return kLaneBytes / static_cast<int>(elem_bytes) < 1 ? 1 : kLaneBytes / static_cast<int>(elem_bytes);
}
constexpr int kFwdBlock = SNNLIF_FWD_BLOCK;
constexpr int kBwdBlock = SNNLIF_BWD_BLOCK;

// Workgroup size of the forward and the fused backward by the size of one tensor.  Tensors that
// the 256 MB memory-side cache can hold together with their outputs are served at fabric speed, and
// there small workgroups win (more, shorter-lived groups whose wavefronts are out of step with each
// other; measured +15-20 % forward, +5-10 % backward between 16 and 128 MiB); tensors streamed from
// HBM prefer the large workgroup, whose wavefronts walk neighbouring DRAM pages together (small
// groups lose 5-10 % from 512 MiB on).  Between the two (192-256 MiB) it makes no difference to
// the backward and to short forward windows, while forward windows of 24-32 steps still gain 5-10 %,
// so the forward switches later than the backward.
constexpr size_t kSmallTensorBytes = SNNLIF_SMALL_TENSOR_BYTES;
constexpr size_t kSmallTensorBytesFwd = SNNLIF_SMALL_TENSOR_BYTES_FWD;
constexpr size_t kResidentTensorBytes = SNNLIF_RESIDENT_TENSOR_BYTES;
// What the caller said about x: nothing, "will be read again soon" (SNNLIF_KEEP_SPATIAL) or "will not,
// however small it is" (SNNLIF_STREAM_SPATIAL).
enum class SpatialHint { none, keep, stream };

// Whether a launch uses the "kept" form of a kernel: the caller's word, else by size (a tensor small
// enough to be cache-resident anyway is kept).
inline bool keep_policy(SpatialHint hint, size_t tensor_bytes) {
    if (hint == SpatialHint::keep) return true;
    if (hint == SpatialHint::stream) return false;
    return tensor_bytes <= kResidentTensorBytes;
}
// Workgroup size of the streamed shape: 256 threads, 128 for tensors of at most
// SNNLIF_STREAM_SMALL_BYTES (cold, 64-128 MiB tensors: forward +1-15 points, backward 0-8; 256 MiB
// tensors lose 4-7 points with 128 threads, except at row pitches of 4 MiB).
inline int stream_block(size_t tensor_bytes, int limit) {
    const int block = tensor_bytes <= static_cast<size_t>(SNNLIF_STREAM_SMALL_BYTES)
                          ? SNNLIF_STREAM_SMALL_BLOCK
                          : SNNLIF_STREAM_BLOCK;
    return block < limit ? block : limit;
}
inline int forward_block(size_t tensor_bytes, bool keep = true) {
    if (!keep) return stream_block(tensor_bytes, kFwdBlock);
    return (tensor_bytes <= kSmallTensorBytesFwd && kFwdBlock > 128) ? 128 : kFwdBlock;
}
inline int backward_block(size_t tensor_bytes, int small = 64, bool keep = true) {
    if (!keep) return stream_block(tensor_bytes, kBwdBlock);
    return (tensor_bytes <= kSmallTensorBytes && kBwdBlock > small) ? small : kBwdBlock;
}

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
__device__ __forceinline__ Pack<S, V> zero_pack() {
    Pack<S, V> r;
    r.raw = typename Pack<S, V>::raw_t(0);
    return r;
}

// STREAM = true: single-use data, non-temporal hint.  STREAM = false: default policy (may be kept
// by the caches for a later reader).
template <typename S, int V, bool STREAM>
__device__ __forceinline__ Pack<S, V> load_pack(const S* p) {
    using raw_t = typename Pack<S, V>::raw_t;
    Pack<S, V> r;
    if (STREAM) {
        r.raw = __builtin_nontemporal_load(reinterpret_cast<const raw_t*>(p));
    } else {
        r.raw = *reinterpret_cast<const raw_t*>(p);
    }
    return r;
}

template <typename S, int V>
__device__ __forceinline__ void store_pack(S* p, const Pack<S, V>& v) {
    using raw_t = typename Pack<S, V>::raw_t;
    // outputs are not read again by this library: always the non-temporal hint (stores with the default
    // policy measured slower in every shape tried, rows that straddle 128-byte lines included)
    __builtin_nontemporal_store(v.raw, reinterpret_cast<raw_t*>(p));
}

// Storage type -> arithmetic type and conversions.
template <typename S> struct Arith;
template <> struct Arith<float> {
    using type = float;
    static constexpr int kMaxVec = lane_vec(sizeof(float));
    __device__ static __forceinline__ float load(float v) { return v; }
    __device__ static __forceinline__ float store(float v) { return v; }
};
template <> struct Arith<double> {
    using type = double;
    static constexpr int kMaxVec = lane_vec(sizeof(double));
    __device__ static __forceinline__ double load(double v) { return v; }
    __device__ static __forceinline__ double store(double v) { return v; }
};
template <> struct Arith<bf16_t> {
    using type = float;
    static constexpr int kMaxVec = lane_vec(sizeof(uint16_t));
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
// TC: rows requested before the first is consumed.  MULTI = false: the whole window fits in TC
// rows.  MULTI = true: the window is streamed TC rows at a time with the next TC rows already in
// flight while the current ones are processed.  KEEP: x is loaded with the default cache policy
// (see the file header); otherwise with the non-temporal hint.  CAP > 0: wavefronts per SIMD of this
// instantiation.  FULL: T == TC; no test around any row, requests go out in time order and each row is
// consumed and its result stored as soon as it has arrived.
// ---------------------------------------------------------------------------------------------
template <typename S, typename M, int V, int TC, bool MULTI, bool WRITE_U, bool WRITE_S, bool KEEP,
          int CAP = 0, bool FULL = false>
__global__ void __launch_bounds__(kFwdBlock) SNNLIF_WAVES_PER_SIMD(forward_waves(TC, KEEP, CAP))
lif_forward_kernel(const S* __restrict__ x, M* __restrict__ mem, S* __restrict__ spike, int T,
                   int64_t N, int64_t nvec, typename Arith<S>::type alpha,
                   typename Arith<S>::type thresh) {
    using C = typename Arith<S>::type;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t v = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; v < nvec;
         v += stride) {
        const int64_t col = v * V;
        C u[V], s[V];
#pragma unroll
        for (int j = 0; j < V; ++j) {
            u[j] = C(0);
            s[j] = C(0);
        }
        Pack<S, V> cur[TC];
        Pack<S, V> nxt[MULTI ? TC : 1];
#pragma unroll
        for (int k = 0; k < TC; ++k) {
            if (FULL || k < T)
                cur[k] = load_pack<S, V, !KEEP>(x + static_cast<int64_t>(k) * N + col);
            // requests go out in time order (left alone, the compiler issues the first row last but one)
            if (FULL) __builtin_amdgcn_sched_barrier(0);
        }
        for (int t0 = 0; t0 < T; t0 += TC) {
            if (MULTI && t0 + TC < T) {
#pragma unroll
                for (int k = 0; k < TC; ++k) {
                    const int t = t0 + TC + k;
                    if (t < T)
                        nxt[MULTI ? k : 0] = load_pack<S, V, !KEEP>(
                            x + static_cast<int64_t>(t) * N + col);
                }
            }
#pragma unroll
            for (int k = 0; k < TC; ++k) {
                const int t = t0 + k;
                if (FULL || t < T) {
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
                // a row is consumed and its result stored as soon as it has arrived, not after the
                // whole group has (left alone, the compiler gathers the stores behind the last wait)
                if (FULL) __builtin_amdgcn_sched_barrier(0);
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
// Forward with a rolling window of W rows in flight, for windows of a multiple of W steps: once a row
// has been consumed and its spike stored, the row W steps later is requested into the register it
// left.  A wavefront then keeps W loads outstanding from its first instruction to its last group and
// issues loads and stores alternately, instead of a burst of requests followed by a burst of stores.
// ---------------------------------------------------------------------------------------------
// RAGGED: the window is not a multiple of W steps; refills past its end are skipped and the last
// group is partial (tests that do not depend on the lane).
// Used for streamed windows from SNNLIF_FWD_ROLLING_MIN_T steps on.
// Measured cold on MI355X against the burst form (32 rows at once at 3 wavefronts per SIMD, groups of 16
// beyond), fp32, % of the HBM peak: 32 steps 71.9 -> 73.1 (256 MiB tensors), 63.4 -> 65.7 (128 MiB),
// 76.8 -> 77.8 (512 MiB); 64 steps 59.7 -> 67.0; 96 steps 66.2 -> 70.7.  16 rows at 2 wavefronts per SIMD
// is the best of 4 / 8 / 16 / 32 rows at 1-8 wavefronts (8 rows at 4: 66 % at 32 steps; 16 rows at 1: 64 %).
// Ragged windows against bursts of 16 rows: 40 steps 71.5 -> 75, 50 steps 67.5 -> 71, 100 steps 66 -> 70.5;
// below 32 steps the ragged form is no better than the bursts (20 steps 73 -> 71, 24 steps +1, 28 steps -1).
#ifndef SNNLIF_FWD_ROLLING_W
#define SNNLIF_FWD_ROLLING_W 16
#endif
#ifndef SNNLIF_FWD_ROLLING_MIN_T
#define SNNLIF_FWD_ROLLING_MIN_T 32
#endif
#ifndef SNNLIF_FWD_ROLLING_WAVES
#define SNNLIF_FWD_ROLLING_WAVES 2
#endif
template <typename S, typename M, int V, int W, bool WRITE_U, bool WRITE_S, bool KEEP, bool RAGGED = false>
__global__ void __launch_bounds__(kFwdBlock) SNNLIF_WAVES_PER_SIMD(SNNLIF_FWD_ROLLING_WAVES)
lif_forward_rolling_kernel(const S* __restrict__ x, M* __restrict__ mem, S* __restrict__ spike, int T,
                           int64_t N, int64_t nvec, typename Arith<S>::type alpha,
                           typename Arith<S>::type thresh) {
    using C = typename Arith<S>::type;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t v = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; v < nvec;
         v += stride) {
        const int64_t col = v * V;
        C u[V], s[V];
#pragma unroll
        for (int j = 0; j < V; ++j) {
            u[j] = C(0);
            s[j] = C(0);
        }
        Pack<S, V> buf[W];
#pragma unroll
        for (int k = 0; k < W; ++k) buf[k] = load_pack<S, V, !KEEP>(x + static_cast<int64_t>(k) * N + col);
        int t0 = 0;
        for (; t0 + W < T; t0 += W) {
#pragma unroll
            for (int k = 0; k < W; ++k) {
                Pack<M, V> mo;
                Pack<S, V> so;
#pragma unroll
                for (int j = 0; j < V; ++j) {
                    lif_step<C>(u[j], s[j], Arith<S>::load(buf[k].e[j]), alpha, thresh);
                    if (WRITE_U) mo.e[j] = Arith<M>::store(u[j]);
                    if (WRITE_S) so.e[j] = Arith<S>::store(s[j]);
                }
                const int64_t off = static_cast<int64_t>(t0 + k) * N + col;
                if (WRITE_U) store_pack<M, V>(mem + off, mo);
                if (WRITE_S) store_pack<S, V>(spike + off, so);
                if (!RAGGED || t0 + W + k < T)
                    buf[k] = load_pack<S, V, !KEEP>(x + static_cast<int64_t>(t0 + W + k) * N + col);
            }
        }
#pragma unroll
        for (int k = 0; k < W; ++k) {
            if (RAGGED && t0 + k >= T) break;
            Pack<M, V> mo;
            Pack<S, V> so;
#pragma unroll
            for (int j = 0; j < V; ++j) {
                lif_step<C>(u[j], s[j], Arith<S>::load(buf[k].e[j]), alpha, thresh);
                if (WRITE_U) mo.e[j] = Arith<M>::store(u[j]);
                if (WRITE_S) so.e[j] = Arith<S>::store(s[j]);
            }
            const int64_t off = static_cast<int64_t>(t0 + k) * N + col;
            if (WRITE_U) store_pack<M, V>(mem + off, mo);
            if (WRITE_S) store_pack<S, V>(spike + off, so);
        }
    }
}

// ---------------------------------------------------------------------------------------------
// One register-resident backward window of at most TW rows, for the neuron(s) at column `col`.
// Row pointers x, g, gx are those of the window's first row; rows of x and gx are N elements apart,
// rows of g GN elements (GN == N: a dense gradient; GN == 0: one row that stands for every step).  On entry uc / sc hold the membrane
// potential and spike of the step before the window (zeros at t = 0) and gu the gradient carried
// in from the step after it (zero at the end of time); on exit gu is the gradient of the window's
// first step, ready for the window before.
// EXACT = true: `rows` == TW, straight-line code.  EXACT = false: rows < TW; rows t >= `rows` are
// not fetched (zeros stand in for them), the recomputation runs over all TW rows (rows past the end
// only produce values nobody reads) and the reverse sweep skips them.
// Gradient rows are fetched in groups of at most GC, the newest time steps first; the fetch of the
// next (earlier) group is issued before the current group is consumed.
// KEEP: x is loaded with the default cache policy, otherwise with the non-temporal hint.
// GSHARED: the gradient is one row that stands for every step of the window (GN == 0): it is loaded
// once instead of once per step.
// HEAD > 0: the window is preceded by `head` (0 <= head <= HEAD, the same for all lanes) further rows,
// at rows -head .. -1 relative to the row pointers, which are part of the same register window: their
// loads are issued with the window's (behind run-time tests that do not depend on the lane, around a
// handful of registers only), their potentials are recomputed first and swept last.  A window of any
// length then runs as a straight-line body of a multiple of 8 steps plus a head of up to 7, and still
// reads every operand once.
// ---------------------------------------------------------------------------------------------
constexpr int kHeadMax = 7;

template <typename S, int V, int TW, bool EXACT, bool KEEP = true, bool GSHARED = false, int HEAD = 0>
__device__ __forceinline__ void backward_window(const S* __restrict__ x, const S* __restrict__ g,
                                                S* __restrict__ gx, int rows, int64_t N,
                                                int64_t GN, int64_t col,
                                                typename Arith<S>::type (&uc)[V],
                                                typename Arith<S>::type (&sc)[V],
                                                typename Arith<S>::type (&gu)[V],
                                                typename Arith<S>::type alpha,
                                                typename Arith<S>::type thresh,
                                                typename Arith<S>::type beta,
                                                typename Arith<S>::type interval, int head = 0) {
    using C = typename Arith<S>::type;
    constexpr int GC = (TW < SNNLIF_BWD_GCHUNK) ? TW : SNNLIF_BWD_GCHUNK;
    constexpr int NG = (TW + GC - 1) / GC;  // groups; group 0 holds the newest rows
    // group q covers rows [lo(q), hi(q)) with hi(q) = TW - q*GC and lo(q) = max(0, hi(q) - GC)
    constexpr int HS = HEAD > 0 ? HEAD : 1;
    // Windows with a head and all windows beyond SNNLIF_BWD_PIN_MIN_TW steps pin the order "requests of
    // the window, recomputation, then per group: requests of the next group, sweep and stores of this
    // one" with scheduling barriers.  Left to itself the compiler keeps that order for most window
    // lengths but falls back to one request at a time, each followed by a full wait, for some (fp32 40
    // steps; fp64 48 and 64; bf16 40 and 72-104 with one neuron per lane; every window with a head):
    // 33 % of the HBM peak instead of 75 % for the 40-step window.  Up to 32 steps no instantiation is
    // affected and the free schedule (all requests up front) measures 1-2 points better.
    constexpr bool kPinned = HEAD > 0 || (EXACT && TW > SNNLIF_BWD_PIN_MIN_TW);
    static_assert(HEAD == 0 || (EXACT && !GSHARED), "a head goes with a straight-line body");

    // slot k: row k - head, present when k < head.  Both operands of the head are requested here, ahead
    // of the body's rows, and its potentials are formed with selects: no branch lies between the body's
    // first load and its last store, so the body keeps the instruction order of the window without a head.
    Pack<S, V> xhead[HS], ghead[HS];
    if constexpr (HEAD > 0) {
#pragma unroll
        for (int k = 0; k < HEAD; ++k) {
            xhead[k] = zero_pack<S, V>();
            ghead[k] = zero_pack<S, V>();
            if (k < head) {
                xhead[k] = load_pack<S, V, !KEEP>(x + static_cast<int64_t>(k - head) * N + col);
                ghead[k] = load_pack<S, V, true>(g + static_cast<int64_t>(k - head) * GN + col);
            }
        }
    }
    Pack<S, V> xin[TW];
#pragma unroll
    for (int t = 0; t < TW; ++t) {
        if (EXACT) {
            xin[t] = load_pack<S, V, !KEEP>(x + static_cast<int64_t>(t) * N + col);
        } else {
            xin[t] = zero_pack<S, V>();
            if (t < rows)
                xin[t] = load_pack<S, V, !KEEP>(x + static_cast<int64_t>(t) * N + col);
        }
    }
    Pack<S, V> gbuf[2][GSHARED ? 1 : GC];
    if constexpr (GSHARED) gbuf[0][0] = load_pack<S, V, true>(g + col);
#pragma unroll
    for (int t = TW - 1; t >= ((TW - GC) > 0 ? (TW - GC) : 0); --t) {
        if constexpr (GSHARED) break;
        const int k = GSHARED ? 0 : t - ((TW - GC) > 0 ? (TW - GC) : 0);
        if (EXACT) {
            gbuf[0][k] = load_pack<S, V, true>(g + static_cast<int64_t>(t) * GN + col);
        } else {
            gbuf[0][k] = zero_pack<S, V>();
            if (t < rows) gbuf[0][k] = load_pack<S, V, true>(g + static_cast<int64_t>(t) * GN + col);
        }
    }

    if constexpr (HEAD == 0 && kPinned) __builtin_amdgcn_sched_barrier(0);
    C uhead[HS][V];
    if constexpr (HEAD > 0) {
        // everything requested so far stays ahead of the arithmetic (with the head's registers live
        // across the body the compiler otherwise falls back to one load at a time)
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int k = 0; k < HEAD; ++k) {
#pragma unroll
            for (int j = 0; j < V; ++j) {
                C un = uc[j], sn = sc[j];
                lif_step<C>(un, sn, Arith<S>::load(xhead[k].e[j]), alpha, thresh);
                uc[j] = k < head ? un : uc[j];
                sc[j] = k < head ? sn : sc[j];
                uhead[k][j] = uc[j];
            }
        }
    }
    C u[TW][V];
#pragma unroll
    for (int t = 0; t < TW; ++t) {
#pragma unroll
        for (int j = 0; j < V; ++j) {
            lif_step<C>(uc[j], sc[j], Arith<S>::load(xin[t].e[j]), alpha, thresh);
            u[t][j] = uc[j];
        }
    }

#pragma unroll
    for (int q = 0; q < NG; ++q) {
        const int hi = TW - q * GC;
        const int lo = (hi - GC) > 0 ? (hi - GC) : 0;
        if (!GSHARED && q + 1 < NG) {
            const int nhi = lo;
            const int nlo = (nhi - GC) > 0 ? (nhi - GC) : 0;
#pragma unroll
            for (int t = nhi - 1; t >= nlo; --t) {
                if (EXACT) {
                    gbuf[(q + 1) & 1][GSHARED ? 0 : t - nlo] =
                        load_pack<S, V, true>(g + static_cast<int64_t>(t) * GN + col);
                } else {
                    gbuf[(q + 1) & 1][GSHARED ? 0 : t - nlo] = zero_pack<S, V>();
                    if (t < rows)
                        gbuf[(q + 1) & 1][GSHARED ? 0 : t - nlo] =
                            load_pack<S, V, true>(g + static_cast<int64_t>(t) * GN + col);
                }
            }
        }
        // with a head: each group's requests stay ahead of the group before it being consumed
        if constexpr (kPinned) __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = hi - 1; t >= lo; --t) {
            if (EXACT || t < rows) {
                Pack<S, V> out;
#pragma unroll
                for (int j = 0; j < V; ++j) {
                    lif_reverse_step<C>(gu[j], u[t][j],
                                        Arith<S>::load(gbuf[GSHARED ? 0 : (q & 1)][GSHARED ? 0 : t - lo].e[j]),
                                        alpha, thresh, beta, interval);
                    out.e[j] = Arith<S>::store(gu[j]);
                }
                store_pack<S, V>(gx + static_cast<int64_t>(t) * N + col, out);
            }
        }
        if constexpr (kPinned) __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (HEAD > 0) {
#pragma unroll
        for (int k = HEAD - 1; k >= 0; --k) {
            if (k < head) {
                Pack<S, V> out;
#pragma unroll
                for (int j = 0; j < V; ++j) {
                    lif_reverse_step<C>(gu[j], uhead[k][j], Arith<S>::load(ghead[k].e[j]), alpha, thresh,
                                        beta, interval);
                    out.e[j] = Arith<S>::store(gu[j]);
                }
                store_pack<S, V>(gx + static_cast<int64_t>(k - head) * N + col, out);
            }
        }
    }
}

// Column a lane works on: the backward walks the neuron axis from its end (see the file header).
__device__ __forceinline__ int64_t backward_column(int64_t v, int64_t nvec, int V) {
#if SNNLIF_BWD_DESCENDING
    return (nvec - 1 - v) * V;
#else
    return v * V;
#endif
}

// ---------------------------------------------------------------------------------------------
// Fused backward for T <= TW: the whole time axis is one register window.  HEAD > 0: for
// TW < T <= TW + HEAD, the first T - TW steps being the window's head (see backward_window).
// ---------------------------------------------------------------------------------------------
template <typename S, int V, int TW, bool EXACT, bool KEEP, bool GSHARED = false, int HEAD = 0, int CAP = 0>
__global__ void __launch_bounds__(kBwdBlock)
    SNNLIF_WAVES_PER_SIMD(CAP > 0 ? CAP : backward_waves(TW + HEAD, KEEP))
lif_backward_fused_kernel(const S* __restrict__ x, const S* __restrict__ g, S* __restrict__ gx,
                          int T, int64_t N, int64_t GN, int64_t nvec,
                          typename Arith<S>::type alpha, typename Arith<S>::type thresh,
                          typename Arith<S>::type beta, typename Arith<S>::type interval) {
    using C = typename Arith<S>::type;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t v = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; v < nvec;
         v += stride) {
        const int64_t col = backward_column(v, nvec, V);
        C uc[V], sc[V], gu[V];
#pragma unroll
        for (int j = 0; j < V; ++j) {
            uc[j] = C(0);
            sc[j] = C(0);
            gu[j] = C(0);
        }
        const int head = HEAD > 0 ? T - TW : 0;
        backward_window<S, V, TW, EXACT, KEEP, GSHARED, HEAD>(
            x + static_cast<int64_t>(head) * N, g + static_cast<int64_t>(head) * GN,
            gx + static_cast<int64_t>(head) * N, T - head, N, GN, col, uc, sc, gu, alpha, thresh, beta,
            interval, head);
    }
}

// ---------------------------------------------------------------------------------------------
// Segmented backward for windows longer than the register-window forms take.  Two phases per
// lane, no scratch memory in HBM:
//   1. run the recurrence forward over all but the last segment and keep the membrane potential at
//      every segment boundary in LDS (one value per neuron and segment, in a slot only this lane
//      touches: no synchronisation; the spike flag at a boundary is u > thresh);
//   2. from the last segment to the first, recompute that segment's u into registers from its
//      boundary value and sweep it in reverse, carrying the gradient across segments.
// x is read twice (12 + 4 = 16 bytes per neuron-step in fp32); the second read of the last
// segments usually still hits the caches.  Dynamic LDS: ceil(T/kSegment) * blockDim.x * V values.
// ---------------------------------------------------------------------------------------------
constexpr int kSegment = 32;

// TAIL > 0: the end of the window is not a (partial) 32-step segment but one register window of
// 64 + T mod 32 steps -- a straight-line body of TAIL steps (the multiple of 8 below that) with a head --
// so that two to three segments fewer are read twice: 12 + 4 * (T - 64 - T mod 32) / T bytes per
// neuron-step instead of 12 + 4 * (T - T mod 32) / T (120 steps: 13.1 instead of 15.1).
template <typename S, int V, int TAIL = 0>
__global__ void __launch_bounds__(kBwdBlock)
    SNNLIF_WAVES_PER_SIMD(backward_waves(TAIL > 0 ? TAIL + kHeadMax : kSegment))
lif_backward_segmented_kernel(const S* __restrict__ x, const S* __restrict__ g,
                              S* __restrict__ gx, int T, int64_t N, int64_t GN, int64_t nvec,
                              typename Arith<S>::type alpha, typename Arith<S>::type thresh,
                              typename Arith<S>::type beta, typename Arith<S>::type interval) {
    using C = typename Arith<S>::type;
    extern __shared__ __align__(16) unsigned char lds_raw[];
    C* boundary = reinterpret_cast<C*>(lds_raw);  // [segment][lane][V]
    // segments in all, the last one being the partial segment or the long tail window
    const int tail = 2 * kSegment + T % kSegment;
    const int nseg = TAIL > 0 ? (T - tail) / kSegment + 1 : (T + kSegment - 1) / kSegment;
    constexpr int ROWS = 8;  // rows requested at a time in phase 1
    static_assert(kSegment % ROWS == 0, "a segment is a whole number of phase-1 groups");

    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t v = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; v < nvec;
         v += stride) {
        const int64_t col = backward_column(v, nvec, V);
        C uc[V], sc[V], gu[V];
#pragma unroll
        for (int j = 0; j < V; ++j) {
            uc[j] = C(0);
            sc[j] = C(0);
            gu[j] = C(0);
        }

        // phase 1: all full segments before the last one
        for (int seg = 0; seg + 1 < nseg; ++seg) {
            for (int t0 = seg * kSegment; t0 < (seg + 1) * kSegment; t0 += ROWS) {
                Pack<S, V> rows[ROWS];
#pragma unroll
                for (int k = 0; k < ROWS; ++k)
                    rows[k] = load_pack<S, V, false>(x + static_cast<int64_t>(t0 + k) * N + col);
#pragma unroll
                for (int k = 0; k < ROWS; ++k) {
#pragma unroll
                    for (int j = 0; j < V; ++j)
                        lif_step<C>(uc[j], sc[j], Arith<S>::load(rows[k].e[j]), alpha, thresh);
                }
            }
#pragma unroll
            for (int j = 0; j < V; ++j)
                boundary[(static_cast<int64_t>(seg + 1) * blockDim.x + threadIdx.x) * V + j] = uc[j];
        }

        // phase 2: the last (possibly partial) segment or the tail window first; uc / sc already hold
        // its boundary
        if constexpr (TAIL > 0) {
            const int head = tail - TAIL;
            const int t0 = (nseg - 1) * kSegment + head;  // first row of the tail's body
            const int64_t off = static_cast<int64_t>(t0) * N;
            backward_window<S, V, TAIL, true, true, false, kHeadMax>(
                x + off, g + static_cast<int64_t>(t0) * GN, gx + off, TAIL, N, GN, col, uc, sc, gu, alpha,
                thresh, beta, interval, head);
        } else {
            const int t0 = (nseg - 1) * kSegment;
            const int64_t off = static_cast<int64_t>(t0) * N;
            backward_window<S, V, kSegment, false>(x + off, g + static_cast<int64_t>(t0) * GN, gx + off,
                                                   T - t0, N, GN, col, uc, sc, gu, alpha, thresh,
                                                   beta, interval);
        }
        for (int seg = nseg - 2; seg >= 0; --seg) {
#pragma unroll
            for (int j = 0; j < V; ++j) {
                uc[j] = seg == 0 ? C(0)
                                 : boundary[(static_cast<int64_t>(seg) * blockDim.x + threadIdx.x) * V + j];
                sc[j] = (seg != 0 && uc[j] > thresh) ? C(1) : C(0);
            }
            const int64_t off = static_cast<int64_t>(seg) * kSegment * N;
            backward_window<S, V, kSegment, true>(x + off, g + static_cast<int64_t>(seg) * kSegment * GN,
                                                  gx + off, kSegment, N, GN, col, uc, sc, gu, alpha,
                                                  thresh, beta, interval);
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Streaming backward for long windows: the membrane potential comes from a workspace written by
// lif_forward_kernel<.., WRITE_U>.  Rows are consumed TC at a time from the end of the window.
// ---------------------------------------------------------------------------------------------
template <typename S, int V, int TC>
__global__ void __launch_bounds__(kBwdBlock)
lif_backward_stream_kernel(const typename Arith<S>::type* __restrict__ mem,
                           const S* __restrict__ g, S* __restrict__ gx, int T, int64_t N,
                           int64_t GN, int64_t nvec, typename Arith<S>::type alpha,
                           typename Arith<S>::type thresh, typename Arith<S>::type beta,
                           typename Arith<S>::type interval) {
    using C = typename Arith<S>::type;
    const int64_t stride = static_cast<int64_t>(gridDim.x) * kBwdBlock;
    for (int64_t v = static_cast<int64_t>(blockIdx.x) * kBwdBlock + threadIdx.x; v < nvec;
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
        for (int k = TC - 1; k >= 0; --k) {
            const int t = (ngroups - 1) * TC + k;
            mcur[k] = zero_pack<C, V>();
            gcur[k] = zero_pack<S, V>();
            if (t < T) {
                mcur[k] = load_pack<C, V, true>(mem + static_cast<int64_t>(t) * N + col);
                gcur[k] = load_pack<S, V, true>(g + static_cast<int64_t>(t) * GN + col);
            }
        }
        for (int c = ngroups - 1; c >= 0; --c) {
            if (c > 0) {
#pragma unroll
                for (int k = TC - 1; k >= 0; --k) {
                    const int64_t row = static_cast<int64_t>((c - 1) * TC + k);
                    mnxt[k] = load_pack<C, V, true>(mem + row * N + col);
                    gnxt[k] = load_pack<S, V, true>(g + row * GN + col);
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
// Host side: vector-width selection and launches.
// ---------------------------------------------------------------------------------------------

// Events a caller armed with snnlif_time_next_kernel() for this thread: the next kernel launched
// from this thread gets them attached to its dispatch (start = the kernel begins, stop = it has
// finished), which times the kernel itself rather than the interval between two stream markers.
struct KernelTimer {
    hipEvent_t start = nullptr;
    hipEvent_t stop = nullptr;
};
extern thread_local KernelTimer tl_kernel_timer;  // defined in lif_abi.hip

// Status of the most recent launch_kernel() of this thread (what the launch call itself returned,
// not the runtime's sticky last-error slot, which an unrelated earlier call may have filled).
extern thread_local hipError_t tl_launch_error;  // defined in lif_abi.hip

// Launches `kernel` with `args` converted to its parameter types; a pending KernelTimer of this
// thread is attached to the dispatch and consumed.
template <typename... Params, typename... Args>
inline void launch_kernel(void (*kernel)(Params...), dim3 grid, dim3 block, size_t lds_bytes,
                          hipStream_t stream, Args... args) {
    static_assert(sizeof...(Params) == sizeof...(Args), "one argument per kernel parameter");
    std::tuple<Params...> converted{static_cast<Params>(args)...};
    void* slots[sizeof...(Params) > 0 ? sizeof...(Params) : 1];
    std::apply([&](auto&... a) { int i = 0; ((slots[i++] = static_cast<void*>(&a)), ...); }, converted);
    const KernelTimer timer = tl_kernel_timer;
    if (timer.start != nullptr || timer.stop != nullptr) {
        tl_kernel_timer = KernelTimer{};
        tl_launch_error = hipExtLaunchKernel(reinterpret_cast<const void*>(kernel), grid, block, slots,
                                             lds_bytes, stream, timer.start, timer.stop, 0);
    } else {
        tl_launch_error = hipLaunchKernel(reinterpret_cast<const void*>(kernel), grid, block, slots,
                                          lds_bytes, stream);
    }
}

// Upper bound on blocks per launch; beyond it lanes take further columns in the grid-stride loop.
constexpr int64_t kMaxGrid = int64_t(1) << 24;

inline unsigned grid_for(int64_t nvec, int block) {
    int64_t blocks = (nvec + block - 1) / block;
    if (blocks > kMaxGrid) blocks = kMaxGrid;
    if (blocks < 1) blocks = 1;
    return static_cast<unsigned>(blocks);
}

inline bool aligned_to(const void* p, size_t bytes) {
    return p == nullptr || (reinterpret_cast<uintptr_t>(p) % bytes) == 0;
}

// Largest power-of-two V <= maxv such that rows (N elements apart, and GN for a tensor with a row
// pitch of its own) and the bases of all given pointers stay aligned to V elements.  elem[i] is the
// element size behind ptrs[i].
inline int pick_vec(int maxv, int64_t N, const void* const* ptrs, const size_t* elem, int n,
                    int64_t GN = 0) {
    int v = maxv;
    while (v > 1) {
        bool ok = (N % v) == 0 && (GN % v) == 0;
        for (int i = 0; ok && i < n; ++i) ok = aligned_to(ptrs[i], elem[i] * v);
        if (ok) break;
        v >>= 1;
    }
    return v;
}

inline int launch_status() {
    return static_cast<int>(tl_launch_error);
}

// Calls f(std::integral_constant<int, v>) for the runtime vector width v in {MAXV, MAXV/2, .., 1}.
template <int MAXV, typename F>
inline int with_vec(int v, F&& f) {
    if constexpr (MAXV >= 8) {
        if (v == 8) return f(std::integral_constant<int, 8>());
    }
    if constexpr (MAXV >= 4) {
        if (v == 4) return f(std::integral_constant<int, 4>());
    }
    if constexpr (MAXV >= 2) {
        if (v == 2) return f(std::integral_constant<int, 2>());
    }
    return f(std::integral_constant<int, 1>());
}

// One forward launch with TC rows per group.
template <typename S, typename M, int V, int TC, bool MULTI, bool WRITE_U, bool WRITE_S, bool KEEP,
          int CAP = 0>
int launch_forward_rows(const S* x, M* mem, S* spike, int64_t T, int64_t N, float alpha, float thresh,
                        int threads, hipStream_t stream) {
    using C = typename Arith<S>::type;
    const int64_t nvec = N / V;
    // A window that fills the instantiation can run without the tests around each row.  fp64 windows
    // of 8 / 16 steps: 62 -> 71 % / 51 -> 65.5 % of the HBM peak, cold (behind the tests the compiler waits
    // for each 8-byte load before it issues the next); the streamed fp32 / bf16 windows of up to 8 steps
    // have an instantiation per length (CAP > 0), and 4 steps gain a point in the kept form as well.
    constexpr bool can_fill = !MULTI && (sizeof(S) == 8 || CAP > 0 || (sizeof(S) == 4 && TC == 4));
    if constexpr (can_fill) {
        if (T == TC) {
            launch_kernel(lif_forward_kernel<S, M, V, TC, false, WRITE_U, WRITE_S, KEEP, CAP, true>,
                          dim3(grid_for(nvec, threads)), dim3(threads), 0, stream, x, mem, spike,
                          static_cast<int>(T), N, nvec, C(alpha), C(thresh));
            return launch_status();
        }
    }
    if constexpr (CAP > 0) {
        return SNNLIF_ERR_ARG;  // the capped instantiations exist for T == TC only
    } else {
        launch_kernel(lif_forward_kernel<S, M, V, TC, MULTI, WRITE_U, WRITE_S, KEEP, CAP>,
                      dim3(grid_for(nvec, threads)), dim3(threads), 0, stream, x, mem, spike,
                      static_cast<int>(T), N, nvec, C(alpha), C(thresh));
        return launch_status();
    }
}

// Rows per group by window length.  Kept x: the whole window up to SNNLIF_FWD_ROWS rows, longer ones
// streamed in groups of that many.  Streamed x: windows of up to 16 rows are requested whole (a
// window of 9-16 rows as one group measures +5-8 points over two groups of 8), windows of 17-24 rows
// whole in a 24-row instantiation and windows of 25-31 rows in a 32-row one, both at 3 wavefronts per
// SIMD (against a group of 16 followed by the rest, cold, rows 8 MiB apart: 17 rows 48 -> 55 % of the HBM
// peak, 20 rows 59 -> 64, 23 rows 63 -> 66; 24 rows in their own instantiation +2 over the 32-row one;
// 32 rows at once +3-5 points over two groups of 16).  From 32 rows on every window runs the
// rolling-window kernel.
template <typename S, typename M, int V, bool WRITE_U, bool WRITE_S, bool KEEP>
int launch_forward_v(const S* x, M* mem, S* spike, int64_t T, int64_t N, float alpha, float thresh,
                     hipStream_t stream) {
    const int threads =
        forward_block(static_cast<size_t>(T) * static_cast<size_t>(N) * sizeof(S), KEEP);
    constexpr int TC = SNNLIF_FWD_ROWS;
    constexpr int TM = KEEP ? TC : SNNLIF_STREAM_FWD_ROWS_MID;  // rows per group of the long-window form
    constexpr int TL = SNNLIF_STREAM_FWD_ROWS_LONG;
#define SNNLIF_FWD_LAUNCH(ROWS, MULTI)                                                           \
    launch_forward_rows<S, M, V, ROWS, MULTI, WRITE_U, WRITE_S, KEEP>(x, mem, spike, T, N, alpha,  \
                                                                      thresh, threads, stream)
    if constexpr (!KEEP) {
        // streamed windows of up to 8 steps and of 10, 12, 16 (small tensors), 20, 24, 28, 32: a
        // straight-line instantiation per length and number of wavefronts per SIMD
        const size_t tensor_bytes = static_cast<size_t>(T) * static_cast<size_t>(N) * sizeof(S);
        const int waves = stream_forward_waves(static_cast<int>(T), tensor_bytes);
#define SNNLIF_FWD_EXACT(ROWS, WAVES)                                                              \
    if (T == ROWS && waves == WAVES)                                                               \
        return launch_forward_rows<S, M, V, ROWS, false, WRITE_U, WRITE_S, KEEP, WAVES>(            \
            x, mem, spike, T, N, alpha, thresh, threads, stream);
        SNNLIF_FWD_EXACT(3, 8)  // (one and two steps: launch_forward_short)
        SNNLIF_FWD_EXACT(4, 8)
        SNNLIF_FWD_EXACT(5, 5)
        SNNLIF_FWD_EXACT(6, 5)
        SNNLIF_FWD_EXACT(6, 4)
        SNNLIF_FWD_EXACT(7, 5)
        SNNLIF_FWD_EXACT(7, 3)
        SNNLIF_FWD_EXACT(8, 5)
        SNNLIF_FWD_EXACT(8, 3)
        SNNLIF_FWD_EXACT(10, 4)
        SNNLIF_FWD_EXACT(12, 3)
        SNNLIF_FWD_EXACT(16, 2)
        SNNLIF_FWD_EXACT(20, 2)
        SNNLIF_FWD_EXACT(24, 2)
        SNNLIF_FWD_EXACT(28, 2)
        SNNLIF_FWD_EXACT(32, 2)
#undef SNNLIF_FWD_EXACT
    }
    if (T <= 4 && TC > 4) return SNNLIF_FWD_LAUNCH(4, false);
    if (T <= TC) return SNNLIF_FWD_LAUNCH(TC, false);
    if constexpr (!KEEP && SNNLIF_FWD_ROLLING_W > 0) {
        constexpr int W = SNNLIF_FWD_ROLLING_W > 0 ? SNNLIF_FWD_ROLLING_W : 1;
        if (T >= SNNLIF_FWD_ROLLING_MIN_T && T > W) {
            using C = typename Arith<S>::type;
            const int64_t nvec = N / V;
            const dim3 grid(grid_for(nvec, threads)), block(threads);
            if (T % W == 0)
                launch_kernel(lif_forward_rolling_kernel<S, M, V, W, WRITE_U, WRITE_S, KEEP, false>, grid,
                              block, 0, stream, x, mem, spike, static_cast<int>(T), N, nvec, C(alpha),
                              C(thresh));
            else
                launch_kernel(lif_forward_rolling_kernel<S, M, V, W, WRITE_U, WRITE_S, KEEP, true>, grid,
                              block, 0, stream, x, mem, spike, static_cast<int>(T), N, nvec, C(alpha),
                              C(thresh));
            return launch_status();
        }
    }
    if constexpr (!KEEP) {
        if (T <= TM) return SNNLIF_FWD_LAUNCH(TM, false);
        if (T <= (TM + TL) / 2) return SNNLIF_FWD_LAUNCH((TM + TL) / 2, false);
        if (T <= TL) return SNNLIF_FWD_LAUNCH(TL, false);
    }
    return SNNLIF_FWD_LAUNCH(TM, true);  // kept x only: streamed windows of this length have returned above
#undef SNNLIF_FWD_LAUNCH
}

// Windows of at most SNNLIF_WIDE_LANE_MAX_T (<= 4) steps: only the 4-row instantiation is needed.
template <typename S, typename M, int V, bool WRITE_U, bool WRITE_S, bool KEEP>
int launch_forward_short(const S* x, M* mem, S* spike, int64_t T, int64_t N, float alpha,
                         float thresh, hipStream_t stream) {
    static_assert(SNNLIF_WIDE_LANE_MAX_T <= 4, "the short-window forward holds 4 rows");
    const int threads =
        forward_block(static_cast<size_t>(T) * static_cast<size_t>(N) * sizeof(S), KEEP);
    return launch_forward_rows<S, M, V, 4, false, WRITE_U, WRITE_S, KEEP>(x, mem, spike, T, N, alpha,
                                                                          thresh, threads, stream);
}

template <typename S, typename M, bool WRITE_U, bool WRITE_S, bool KEEP>
int launch_forward_policy(const S* x, M* mem, S* spike, int64_t T, int64_t N, float alpha,
                          float thresh, hipStream_t stream) {
    // lanes are sized by the narrower of the two element types; the wider one (the fp32 workspace
    // behind bf16 storage) then moves V of its elements, at most 16 bytes
    constexpr size_t narrowest = sizeof(S) < sizeof(M) ? sizeof(S) : sizeof(M);
    constexpr size_t widest = sizeof(S) > sizeof(M) ? sizeof(S) : sizeof(M);
    constexpr int maxv = lane_vec(narrowest) < static_cast<int>(16 / widest)
                             ? lane_vec(narrowest)
                             : static_cast<int>(16 / widest);
    const void* ptrs[3] = {x, WRITE_U ? mem : nullptr, WRITE_S ? spike : nullptr};
    const size_t elem[3] = {sizeof(S), sizeof(M), sizeof(S)};
    for (int i = 0; i < 3; ++i)
        if (!aligned_to(ptrs[i], elem[i])) return SNNLIF_ERR_ALIGN;
    if (T <= SNNLIF_WIDE_LANE_MAX_T) {
        constexpr int widev = static_cast<int>(16 / widest);
        const int wv = pick_vec(widev, N, ptrs, elem, 3);
        return with_vec<widev>(wv, [&](auto vc) {
            constexpr int V = decltype(vc)::value;
            return launch_forward_short<S, M, V, WRITE_U, WRITE_S, KEEP>(x, mem, spike, T, N, alpha,
                                                                         thresh, stream);
        });
    }
    const int v = pick_vec(maxv, N, ptrs, elem, 3);
    return with_vec<maxv>(v, [&](auto vc) {
        constexpr int V = decltype(vc)::value;
        return launch_forward_v<S, M, V, WRITE_U, WRITE_S, KEEP>(x, mem, spike, T, N, alpha, thresh,
                                                                 stream);
    });
}

// keep_x: what the caller said about x (see the file header); small tensors are always kept.
template <typename S, typename M, bool WRITE_U, bool WRITE_S>
int launch_forward(const S* x, M* mem, S* spike, int64_t T, int64_t N, float alpha, float thresh,
                   SpatialHint keep_x, hipStream_t stream) {
    if (keep_policy(keep_x, static_cast<size_t>(T) * static_cast<size_t>(N) * sizeof(S)))
        return launch_forward_policy<S, M, WRITE_U, WRITE_S, true>(x, mem, spike, T, N, alpha, thresh,
                                                                   stream);
    return launch_forward_policy<S, M, WRITE_U, WRITE_S, false>(x, mem, spike, T, N, alpha, thresh,
                                                                stream);
}

template <typename S>
int forward_dispatch(const void* x, void* mem, void* spike, int64_t T, int64_t N, float alpha,
                     float thresh, SpatialHint keep_x, hipStream_t stream) {
    const S* xs = static_cast<const S*>(x);
    S* ms = static_cast<S*>(mem);
    S* ss = static_cast<S*>(spike);
    if (mem != nullptr && spike != nullptr)
        return launch_forward<S, S, true, true>(xs, ms, ss, T, N, alpha, thresh, keep_x, stream);
    if (mem != nullptr)
        return launch_forward<S, S, true, false>(xs, ms, nullptr, T, N, alpha, thresh, keep_x, stream);
    return launch_forward<S, S, false, true>(xs, nullptr, ss, T, N, alpha, thresh, keep_x, stream);
}

// Register budget of the fused backward: TW*V arithmetic values for u plus two gradient
// buffers.  V is capped so that u stays within SNNLIF_FUSED_U_WORDS VGPRs.
template <typename S, int TW>
constexpr int fused_max_vec() {
    using C = typename Arith<S>::type;
    constexpr int words = static_cast<int>(sizeof(C) / 4);
    constexpr int cap = SNNLIF_FUSED_U_WORDS / (TW * words);
    constexpr int hw = TW <= SNNLIF_WIDE_LANE_MAX_T ? static_cast<int>(16 / sizeof(S))
                                                    : Arith<S>::kMaxVec;
    return cap < 1 ? 1 : (cap < hw ? cap : hw);
}

template <typename S, int TW, bool KEEP>
int launch_backward_fused_policy(const S* x, const S* g, S* gx, int64_t T, int64_t N, int64_t GN,
                                 float alpha, float thresh, float beta, float interval,
                                 hipStream_t stream) {
    using C = typename Arith<S>::type;
    constexpr int maxv = fused_max_vec<S, TW>();
    const void* ptrs[3] = {x, g, gx};
    const size_t elem[3] = {sizeof(S), sizeof(S), sizeof(S)};
    const int v = pick_vec(maxv, N, ptrs, elem, 3, GN);
    // always entered with T == TW: every other length takes the form with a head
    return with_vec<maxv>(v, [&](auto vc) {
        constexpr int V = decltype(vc)::value;
        const int64_t nvec = N / V;
        const int threads =
            backward_block(static_cast<size_t>(T) * static_cast<size_t>(N) * sizeof(S), 64, KEEP);
        const dim3 grid(grid_for(nvec, threads)), block(threads);
        const int Ti = static_cast<int>(T);
        // one gradient row for all steps: the form that loads the row once (windows with a head and
        // the long ones read it in place once per step)
        constexpr bool has_shared = TW >= 2 && TW <= SNNLIF_BP_FUSED_MAX_T;
        if (GN == 0 && has_shared) {
            if constexpr (has_shared)
                launch_kernel(lif_backward_fused_kernel<S, V, TW, true, KEEP, true>, grid, block, 0,
                              stream, x, g, gx, Ti, N, GN, nvec, C(alpha), C(thresh), C(beta),
                              C(interval));
        } else {
            if constexpr (!KEEP && stream_backward_small_waves(TW) > 0) {
                if (static_cast<size_t>(T) * static_cast<size_t>(N) * sizeof(S) <=
                    static_cast<size_t>(SNNLIF_STREAM_SMALL_BYTES)) {
                    launch_kernel(lif_backward_fused_kernel<S, V, TW, true, KEEP, false, 0,
                                                            stream_backward_small_waves(TW)>,
                                  grid, block, 0, stream, x, g, gx, Ti, N, GN, nvec, C(alpha), C(thresh),
                                  C(beta), C(interval));
                    return launch_status();
                }
            }
            launch_kernel(lif_backward_fused_kernel<S, V, TW, true, KEEP>, grid, block, 0, stream,
                               x, g, gx, Ti, N, GN, nvec, C(alpha), C(thresh), C(beta), C(interval));
        }
        return launch_status();
    });
}

template <typename S, int TW>
int launch_backward_fused(const S* x, const S* g, S* gx, int64_t T, int64_t N, int64_t GN,
                          float alpha, float thresh, float beta, float interval, SpatialHint keep_x,
                          hipStream_t stream) {
    if (keep_policy(keep_x, static_cast<size_t>(T) * static_cast<size_t>(N) * sizeof(S)))
        return launch_backward_fused_policy<S, TW, true>(x, g, gx, T, N, GN, alpha, thresh, beta,
                                                         interval, stream);
    return launch_backward_fused_policy<S, TW, false>(x, g, gx, T, N, GN, alpha, thresh, beta,
                                                      interval, stream);
}

// Windows of TB + 1 .. TB + kHeadMax steps, TB a multiple of 8: straight-line body with a head.
template <typename S, int TB>
int launch_backward_headed(const S* x, const S* g, S* gx, int64_t T, int64_t N, int64_t GN,
                           float alpha, float thresh, float beta, float interval, SpatialHint keep_x,
                           hipStream_t stream) {
    using C = typename Arith<S>::type;
    constexpr int maxv = fused_max_vec<S, TB + kHeadMax>();
    const void* ptrs[3] = {x, g, gx};
    const size_t elem[3] = {sizeof(S), sizeof(S), sizeof(S)};
    const int v = pick_vec(maxv, N, ptrs, elem, 3, GN);
    const size_t bytes = static_cast<size_t>(T) * static_cast<size_t>(N) * sizeof(S);
    const bool keep = keep_policy(keep_x, bytes);
    return with_vec<maxv>(v, [&](auto vc) {
        constexpr int V = decltype(vc)::value;
        const int64_t nvec = N / V;
        const int threads = backward_block(bytes, 64, keep);
        const dim3 grid(grid_for(nvec, threads)), block(threads);
        const int Ti = static_cast<int>(T);
        constexpr int small_waves = stream_backward_small_waves(TB + kHeadMax);
        if (keep) {
            launch_kernel(lif_backward_fused_kernel<S, V, TB, true, true, false, kHeadMax>, grid, block,
                          0, stream, x, g, gx, Ti, N, GN, nvec, C(alpha), C(thresh), C(beta), C(interval));
        } else if (small_waves > 0 && bytes <= static_cast<size_t>(SNNLIF_STREAM_SMALL_BYTES)) {
            if constexpr (small_waves > 0)
                launch_kernel(lif_backward_fused_kernel<S, V, TB, true, false, false, kHeadMax, small_waves>,
                              grid, block, 0, stream, x, g, gx, Ti, N, GN, nvec, C(alpha), C(thresh),
                              C(beta), C(interval));
        } else {
            launch_kernel(lif_backward_fused_kernel<S, V, TB, true, false, false, kHeadMax>, grid, block,
                          0, stream, x, g, gx, Ti, N, GN, nvec, C(alpha), C(thresh), C(beta), C(interval));
        }
        return launch_status();
    });
}

template <typename S, int V>
int launch_backward_stream_v(const typename Arith<S>::type* mem, const S* g, S* gx, int64_t T,
                             int64_t N, int64_t GN, float alpha, float thresh, float beta,
                             float interval, hipStream_t stream) {
    using C = typename Arith<S>::type;
    const int64_t nvec = N / V;
    launch_kernel(lif_backward_stream_kernel<S, V, 8>, dim3(grid_for(nvec, kBwdBlock)),
                       dim3(kBwdBlock), 0, stream, mem, g, gx, static_cast<int>(T), N, GN, nvec,
                       C(alpha), C(thresh), C(beta), C(interval));
    return launch_status();
}

template <typename S>
int backward_dispatch(const void* x_, const void* g_, void* gx_, int64_t T, int64_t N, int64_t GN,
                      float alpha, float thresh, float beta, float interval, SpatialHint keep_x,
                      void* workspace, size_t workspace_bytes, hipStream_t stream) {
    using C = typename Arith<S>::type;
    const S* x = static_cast<const S*>(x_);
    const S* g = static_cast<const S*>(g_);
    S* gx = static_cast<S*>(gx_);
    if (!aligned_to(x, sizeof(S)) || !aligned_to(g, sizeof(S)) || !aligned_to(gx, sizeof(S)))
        return SNNLIF_ERR_ALIGN;

    // Window lengths with a straight-line instantiation of their own (T == TW) ...
#define SNNLIF_BWD_WINDOW(TW)                                                                    \
    if (T == TW)                                                                                 \
        return launch_backward_fused<S, TW>(x, g, gx, T, N, GN, alpha, thresh, beta, interval,     \
                                            keep_x, stream);
    // ... and every length between them: the multiple of 8 below it as a straight-line body, the
    // first T % 8 steps as its head (see backward_window).  Against the next larger window with the
    // absent rows replaced by zeros, which this form replaced, cold at 64 Mi elements, % of the HBM
    // peak: fp32 18 steps 71 -> 76, 22 steps 69 -> 73.5, 26 steps 57 -> 73, 30 steps 66 -> 72 (9-15
    // steps unchanged within a point); bf16 13 steps 61 -> 70, 26 steps 30 -> 70.
#define SNNLIF_BWD_HEADED_WINDOW(TB)                                                             \
    if constexpr (fused_max_vec<S, TB + kHeadMax>() >= Arith<S>::kMaxVec) {                       \
        if (TB <= wide_max && T > TB && T <= TB + kHeadMax)                                      \
            return launch_backward_headed<S, TB>(x, g, gx, T, N, GN, alpha, thresh, beta,         \
                                                 interval, keep_x, stream);                      \
    }
    constexpr int64_t wide_max =
        sizeof(C) == 4 ? SNNLIF_BWD_WIDE_MAX_T : SNNLIF_BWD_WIDE_MAX_T_F64;
    SNNLIF_BWD_WINDOW(1)
    SNNLIF_BWD_WINDOW(2)
    SNNLIF_BWD_WINDOW(3)
    SNNLIF_BWD_WINDOW(4)
    SNNLIF_BWD_WINDOW(5)
    SNNLIF_BWD_WINDOW(6)
    SNNLIF_BWD_WINDOW(7)
    SNNLIF_BWD_WINDOW(8)
    SNNLIF_BWD_WINDOW(10)
    SNNLIF_BWD_WINDOW(12)
    SNNLIF_BWD_WINDOW(16)
    SNNLIF_BWD_WINDOW(20)
    SNNLIF_BWD_WINDOW(24)
    SNNLIF_BWD_WINDOW(28)
    SNNLIF_BWD_WINDOW(32)
#undef SNNLIF_BWD_WINDOW
    SNNLIF_BWD_HEADED_WINDOW(8)
    SNNLIF_BWD_HEADED_WINDOW(16)
    SNNLIF_BWD_HEADED_WINDOW(24)
    static_assert(SNNLIF_BP_FUSED_MAX_T == 32, "windows above must cover the fused range");

    // Windows of a multiple of 8 steps still fit the register file whole a good way further (u alone
    // takes T VGPRs per lane with 4-byte arithmetic: 4 wavefronts per SIMD up to 64 steps, 3 up to
    // 104; at 128 steps a single wavefront is left and the kernel collapses to a fifth of the
    // segmented kernel's rate).  They move 12 bytes per neuron-step where the segmented kernel
    // re-reads x; cold-cache backward at 64 Mi elements, fp32: 67-72 % of the HBM peak against
    // 54-65 %.  Only the exact length qualifies: the zero-filled form of these wide windows runs at
    // 40-58 %, below the segmented kernel.
#define SNNLIF_BWD_WIDE_WINDOW(TW)                                                               \
    if (TW <= wide_max && T == TW)                                                               \
        return launch_backward_fused<S, TW>(x, g, gx, T, N, GN, alpha, thresh, beta, interval,     \
                                            keep_x, stream);
    SNNLIF_BWD_WIDE_WINDOW(40)
    SNNLIF_BWD_WIDE_WINDOW(48)
    SNNLIF_BWD_WIDE_WINDOW(56)
    SNNLIF_BWD_WIDE_WINDOW(64)
    if constexpr (sizeof(C) == 4) {
        SNNLIF_BWD_WIDE_WINDOW(72)
        SNNLIF_BWD_WIDE_WINDOW(80)
        SNNLIF_BWD_WIDE_WINDOW(88)
        SNNLIF_BWD_WIDE_WINDOW(96)
        SNNLIF_BWD_WIDE_WINDOW(104)
    }
#undef SNNLIF_BWD_WIDE_WINDOW

    // Every other length up to 7 steps past the longest of these, again as body + head.  Still 12
    // bytes per neuron-step, where the segmented kernel below reads x twice.  Cold-cache backward at
    // 64 Mi elements, % of the HBM peak of 12 bytes per neuron-step, segmented -> with a head: fp32
    // 33 steps 66 -> 74, 39 steps 62 -> 68, 50 steps 62 -> 70, 60 steps 65 -> 71, 84 steps 62 -> 70,
    // 100 steps 62 -> 68.5, 111 steps 56 -> 59; bf16 39 steps 54 -> 66, 47 steps 53 -> 64, 60 steps
    // 57 -> 67.  Only while the register budget still allows full dword lanes: bf16 bodies from 64
    // steps on would be down to one neuron per lane and lose to the segmented kernel (71 steps
    // 50 -> 46, 100 steps 53 -> 50).
    SNNLIF_BWD_HEADED_WINDOW(32)
    SNNLIF_BWD_HEADED_WINDOW(40)
    SNNLIF_BWD_HEADED_WINDOW(48)
    SNNLIF_BWD_HEADED_WINDOW(56)
    SNNLIF_BWD_HEADED_WINDOW(64)
    if constexpr (sizeof(C) == 4) {
        SNNLIF_BWD_HEADED_WINDOW(72)
        SNNLIF_BWD_HEADED_WINDOW(80)
        SNNLIF_BWD_HEADED_WINDOW(88)
        SNNLIF_BWD_HEADED_WINDOW(96)
        SNNLIF_BWD_HEADED_WINDOW(104)
    }
#undef SNNLIF_BWD_HEADED_WINDOW

    // Longer windows, up to what the boundary values of a workgroup fit into 64 KiB of LDS for
    // every storage type: segmented kernel, still no scratch memory in HBM.
    if (T <= SNNLIF_BP_NO_WORKSPACE_MAX_T) {
        constexpr int maxv = fused_max_vec<S, kSegment>();
        const void* ptrs[3] = {x, g, gx};
        const size_t elem[3] = {sizeof(S), sizeof(S), sizeof(S)};
        const int v = pick_vec(maxv, N, ptrs, elem, 3, GN);
        return with_vec<maxv>(v, [&](auto vc) {
            constexpr int V = decltype(vc)::value;
            const int64_t nvec = N / V;
            const int nseg = static_cast<int>((T + kSegment - 1) / kSegment);
            // small tensors: 128-thread workgroups (+3-20 % measured; 64 is no better and costs bf16)
            const int threads =
                backward_block(static_cast<size_t>(T) * static_cast<size_t>(N) * sizeof(S), 128);
            const size_t lds = static_cast<size_t>(nseg) * threads * V * sizeof(C);
            const dim3 grid(grid_for(nvec, threads)), block(threads);
            const int Ti = static_cast<int>(T);
            // fp32: the window ends in a long register window instead of a partial segment (see the
            // kernel).  Cold, 64 Mi elements, % of the HBM peak of 12 bytes per neuron-step: 112 steps
            // 53 -> 57, 120 steps 62 -> 68, 140 steps 61 -> 66, 250 steps 56 -> 63, 500 steps 54 -> 55.
            // (bf16 and fp64 would not keep full lanes / enough wavefronts for it.)
            if constexpr (std::is_same<S, float>::value) {
                const int body = (2 * kSegment + static_cast<int>(T % kSegment)) / 8 * 8;
#define SNNLIF_BWD_TAIL(TB)                                                                        \
    if (body == TB) {                                                                              \
        launch_kernel(lif_backward_segmented_kernel<S, V, TB>, grid, block, lds, stream, x, g, gx, \
                      Ti, N, GN, nvec, C(alpha), C(thresh), C(beta), C(interval));                 \
        return launch_status();                                                                    \
    }
                SNNLIF_BWD_TAIL(64) SNNLIF_BWD_TAIL(72) SNNLIF_BWD_TAIL(80) SNNLIF_BWD_TAIL(88)
#undef SNNLIF_BWD_TAIL
            }
            launch_kernel(lif_backward_segmented_kernel<S, V>, grid, block, lds, stream, x, g, gx, Ti, N,
                          GN, nvec, C(alpha), C(thresh), C(beta), C(interval));
            return launch_status();
        });
    }

    // Very long window: u -> workspace (arithmetic type), then the streaming reverse sweep.
    const size_t need = static_cast<size_t>(T) * static_cast<size_t>(N) * sizeof(C);
    if (workspace == nullptr || workspace_bytes < need) return SNNLIF_ERR_WORKSPACE;
    if (!aligned_to(workspace, 16)) return SNNLIF_ERR_ALIGN;
    C* mem = static_cast<C*>(workspace);
    int rc = launch_forward<S, C, true, false>(x, mem, nullptr, T, N, alpha, thresh, keep_x, stream);
    if (rc != SNNLIF_OK) return rc;

    constexpr int maxv = Arith<S>::kMaxVec < static_cast<int>(16 / sizeof(C))
                             ? Arith<S>::kMaxVec
                             : static_cast<int>(16 / sizeof(C));
    const void* ptrs[3] = {mem, g, gx};
    const size_t elem[3] = {sizeof(C), sizeof(S), sizeof(S)};
    const int v = pick_vec(maxv, N, ptrs, elem, 3, GN);
    return with_vec<maxv>(v, [&](auto vc) {
        constexpr int V = decltype(vc)::value;
        return launch_backward_stream_v<S, V>(mem, g, gx, T, N, GN, alpha, thresh, beta, interval,
                                              stream);
    });
}

// Entry points of the per-dtype translation units (defined in lif_f32.hip, lif_f64.hip,
// lif_bf16.hip; called from lif_abi.hip).
#define SNNLIF_DECLARE_DTYPE(NAME)                                                                  \
    int forward_##NAME(const void* x, void* mem, void* spike, int64_t T, int64_t N, float alpha,    \
                       float thresh, SpatialHint keep_x, hipStream_t stream);                              \
    int backward_##NAME(const void* x, const void* g, void* gx, int64_t T, int64_t N, int64_t GN,   \
                        float alpha, float thresh, float beta, float interval, SpatialHint keep_x,  \
                        void* workspace, size_t workspace_bytes, hipStream_t stream);
SNNLIF_DECLARE_DTYPE(f32)
SNNLIF_DECLARE_DTYPE(f64)
SNNLIF_DECLARE_DTYPE(bf16)
#undef SNNLIF_DECLARE_DTYPE

#define SNNLIF_DEFINE_DTYPE(NAME, S)                                                                \
    int forward_##NAME(const void* x, void* mem, void* spike, int64_t T, int64_t N, float alpha,    \
                       float thresh, SpatialHint keep_x, hipStream_t stream) {                             \
        return forward_dispatch<S>(x, mem, spike, T, N, alpha, thresh, keep_x, stream);             \
    }                                                                                               \
    int backward_##NAME(const void* x, const void* g, void* gx, int64_t T, int64_t N, int64_t GN,   \
                        float alpha, float thresh, float beta, float interval, SpatialHint keep_x,  \
                        void* workspace, size_t workspace_bytes, hipStream_t stream) {              \
        return backward_dispatch<S>(x, g, gx, T, N, GN, alpha, thresh, beta, interval, keep_x,      \
                                    workspace, workspace_bytes, stream);                            \
    }

}  // namespace snnlif

#endif  // SNNLIF_LIF_KERNELS_H
