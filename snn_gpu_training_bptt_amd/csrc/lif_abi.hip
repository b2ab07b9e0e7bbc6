// C ABI of libsnnlif_gfx950.so (include/snnlib_lif.h): argument checks and dtype dispatch in front
// of the per-dtype kernel launchers.  No kernel lives in this file; the only device-side object is
// the fixed scratch array behind snnlif_bn_fire_bp_static.
#include <atomic>

#include "lif_bn.h"
#include "lif_kernels.h"

// Device memory of the one entry point that may not take a workspace from its caller
// (snnlif_bn_fire_bp_static).  Every GPU the library runs on holds its own copy of this array, at its
// own address, until the process ends.  In host code the name below is only a handle for
// hipGetSymbolAddress: it is never passed to a kernel or to a memory routine; static_scratch() hands
// out the device address instead.
static __device__ __align__(256) unsigned char scratch[SNNLIF_STATIC_SCRATCH_BYTES];

namespace snnlif {
thread_local KernelTimer tl_kernel_timer;
thread_local hipError_t tl_launch_error = hipSuccess;
}  // namespace snnlif

namespace {

// `dtype` arguments carry the storage type in their low byte and the cache hints above it.
constexpr int kHintBits = SNNLIF_KEEP_SPATIAL | SNNLIF_STREAM_SPATIAL;
inline int storage_of(int dtype) { return dtype & 0xff; }
inline snnlif::SpatialHint hint_of(int dtype) {
    if (dtype & SNNLIF_KEEP_SPATIAL) return snnlif::SpatialHint::keep;
    if (dtype & SNNLIF_STREAM_SPATIAL) return snnlif::SpatialHint::stream;
    return snnlif::SpatialHint::none;
}

// Size of the arithmetic type; 0 for an unknown storage type, unknown flag bits or both hints at once.
inline size_t arith_size(int dtype) {
    if (dtype < 0 || (dtype & ~(0xff | kHintBits)) != 0 || (dtype & kHintBits) == kHintBits) return 0;
    switch (storage_of(dtype)) {
        case SNNLIF_DTYPE_F32: return sizeof(float);
        case SNNLIF_DTYPE_F64: return sizeof(double);
        case SNNLIF_DTYPE_BF16: return sizeof(float);
        default: return 0;
    }
}

// Device address of `scratch` on the current device, resolved on the first call made with that
// device current and kept per device.  Returns SNNLIF_OK, SNNLIF_ERR_ARG for a device ordinal beyond
// the table, or the hipError_t of the failing runtime call.
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_address[kMaxDevices];

int static_scratch(void** out) {
    int device = -1;
    hipError_t err = hipGetDevice(&device);
    if (err != hipSuccess) return static_cast<int>(err);
    if (device < 0 || device >= kMaxDevices) return SNNLIF_ERR_ARG;
    void* address = g_scratch_address[device].load(std::memory_order_acquire);
    if (address == nullptr) {
        // two threads racing here resolve the same address; the second store is harmless
        err = hipGetSymbolAddress(&address, HIP_SYMBOL(scratch));
        if (err != hipSuccess) return static_cast<int>(err);
        if (address == nullptr) return static_cast<int>(hipErrorInvalidSymbol);
        g_scratch_address[device].store(address, std::memory_order_release);
    }
    *out = address;
    return SNNLIF_OK;
}

// Every entry point that can launch holds one of these: whatever way it returns (argument error,
// empty shape, launch), a timer armed with snnlif_time_next_kernel() does not outlive the call and
// cannot end up on a later, unrelated launch.
struct TimerScope {
    ~TimerScope() { snnlif::tl_kernel_timer = snnlif::KernelTimer{}; }
};

// For entry points that launch several kernels: the armed events bracket the whole operation
// (start recorded on the stream before the first kernel, stop after the last, dispatch gaps
// included) instead of riding on the first dispatch alone.
struct OperationTimer {
    snnlif::KernelTimer timer;
    hipStream_t stream;
    // active = false: a single-kernel case of the same entry point; the timer stays armed for the
    // dispatch itself
    explicit OperationTimer(hipStream_t st, bool active = true) : stream(st) {
        if (!active) return;
        timer = snnlif::tl_kernel_timer;
        snnlif::tl_kernel_timer = snnlif::KernelTimer{};
        if (timer.start != nullptr) (void)hipEventRecord(timer.start, stream);
    }
    ~OperationTimer() {
        if (timer.stop != nullptr) (void)hipEventRecord(timer.stop, stream);
    }
};

inline int shape_error(int64_t T, int64_t N) {
    if (T < 0 || N < 0) return SNNLIF_ERR_ARG;
    if (T > 0x7fffffff) return SNNLIF_ERR_ARG;
    if (T > 0 && N > (INT64_MAX / 16) / T) return SNNLIF_ERR_ARG;
    return SNNLIF_OK;
}

}  // namespace

extern "C" {

int snnlif_abi_version(void) { return SNNLIF_ABI_VERSION; }

const char* snnlif_target_arch(void) { return "gfx950"; }

int snnlif_time_next_kernel(void* start_event, void* stop_event) {
    snnlif::tl_kernel_timer.start = static_cast<hipEvent_t>(start_event);
    snnlif::tl_kernel_timer.stop = static_cast<hipEvent_t>(stop_event);
    return SNNLIF_OK;
}

const char* snnlif_strerror(int code) {
    switch (code) {
        case SNNLIF_OK: return "success";
        case SNNLIF_ERR_ARG: return "snnlif: invalid argument (NULL tensor pointer, negative or overflowing T/N)";
        case SNNLIF_ERR_DTYPE: return "snnlif: unsupported dtype (expected SNNLIF_DTYPE_F32, _F64 or _BF16, optionally or-ed with SNNLIF_KEEP_SPATIAL or SNNLIF_STREAM_SPATIAL)";
        case SNNLIF_ERR_WORKSPACE: return "snnlif: workspace missing or smaller than snnlif_fire_bp_workspace_bytes()";
        case SNNLIF_ERR_ALIGN: return "snnlif: pointer not aligned to its element size (workspace: 16 bytes)";
        case SNNLIF_ERR_SCRATCH: return "snnlif: this shape needs more scratch memory than the library's fixed array holds (SNNLIF_STATIC_SCRATCH_BYTES); call snnlif_bn_fire_bp with a workspace instead";
        case SNNLIF_ERR_UNSUPPORTED: return "snnlif: not implemented for these arguments (batch-norm entry points take fp32 / fp64 only)";
        default: break;
    }
    if (code > 0) return hipGetErrorString(static_cast<hipError_t>(code));
    return "snnlif: unknown error code";
}

int snnlif_fire_us_fp(const void* spatial, void* mem, void* spike, int dtype, int64_t T, int64_t N,
                      float alpha, float thresh, void* stream) {
    const TimerScope timer_scope;
    if (arith_size(dtype) == 0) return SNNLIF_ERR_DTYPE;
    const int se = shape_error(T, N);
    if (se != SNNLIF_OK) return se;
    if (T == 0 || N == 0) return SNNLIF_OK;
    if (spatial == nullptr || (mem == nullptr && spike == nullptr)) return SNNLIF_ERR_ARG;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const snnlif::SpatialHint keep = hint_of(dtype);
    switch (storage_of(dtype)) {
        case SNNLIF_DTYPE_F32: return snnlif::forward_f32(spatial, mem, spike, T, N, alpha, thresh, keep, st);
        case SNNLIF_DTYPE_F64: return snnlif::forward_f64(spatial, mem, spike, T, N, alpha, thresh, keep, st);
        default: return snnlif::forward_bf16(spatial, mem, spike, T, N, alpha, thresh, keep, st);
    }
}

int snnlif_fire_s_fp(const void* spatial, void* spike, int dtype, int64_t T, int64_t N,
                     float alpha, float thresh, void* stream) {
    const TimerScope timer_scope;
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
    if (T <= SNNLIF_BP_NO_WORKSPACE_MAX_T) return 0;
    return static_cast<size_t>(T) * static_cast<size_t>(N) * es;
}

int snnlif_fire_bp(const void* spatial, const void* grad_spike, void* grad_spatial, int dtype,
                   int64_t T, int64_t N, float alpha, float thresh, float beta, float interval,
                   void* workspace, size_t workspace_bytes, void* stream) {
    return snnlif_fire_bp_strided(spatial, grad_spike, grad_spatial, dtype, T, N, N, alpha, thresh, beta,
                                  interval, workspace, workspace_bytes, stream);
}

int snnlif_fire_bp_strided(const void* spatial, const void* grad_spike, void* grad_spatial, int dtype,
                           int64_t T, int64_t N, int64_t grad_row_stride, float alpha, float thresh,
                           float beta, float interval, void* workspace, size_t workspace_bytes,
                           void* stream) {
    const TimerScope timer_scope;
    if (arith_size(dtype) == 0) return SNNLIF_ERR_DTYPE;
    const int se = shape_error(T, N);
    if (se != SNNLIF_OK) return se;
    const int64_t GN = grad_row_stride;
    if (GN < 0 || (GN != 0 && GN < N)) return SNNLIF_ERR_ARG;
    if (T == 0 || N == 0) return SNNLIF_OK;
    if (GN > 0 && (T - 1) > (INT64_MAX / 16 - N) / GN) return SNNLIF_ERR_ARG;  // byte offsets stay in int64
    if (spatial == nullptr || grad_spike == nullptr || grad_spatial == nullptr) return SNNLIF_ERR_ARG;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const snnlif::SpatialHint keep = hint_of(dtype);
    // one kernel up to SNNLIF_BP_NO_WORKSPACE_MAX_T steps; beyond, a recompute kernel and a reverse kernel
    const bool two_kernels = T > SNNLIF_BP_NO_WORKSPACE_MAX_T;
    const OperationTimer whole_operation(st, two_kernels);
    switch (storage_of(dtype)) {
        case SNNLIF_DTYPE_F32:
            return snnlif::backward_f32(spatial, grad_spike, grad_spatial, T, N, GN, alpha, thresh, beta, interval, keep, workspace, workspace_bytes, st);
        case SNNLIF_DTYPE_F64:
            return snnlif::backward_f64(spatial, grad_spike, grad_spatial, T, N, GN, alpha, thresh, beta, interval, keep, workspace, workspace_bytes, st);
        default:
            return snnlif::backward_bf16(spatial, grad_spike, grad_spatial, T, N, GN, alpha, thresh, beta, interval, keep, workspace, workspace_bytes, st);
    }
}

namespace {

inline int bn_shape_error(int64_t T, int64_t B, int64_t C, int64_t HW) {
    if (T < 0 || B < 0 || C < 0 || HW < 0) return SNNLIF_ERR_ARG;
    if (C > 0x7fffffff) return SNNLIF_ERR_ARG;
    const int64_t lim = INT64_MAX / 64;
    if (C > 0 && HW > lim / C) return SNNLIF_ERR_ARG;
    if (B > 0 && C * HW > 0 && B > lim / (C * HW)) return SNNLIF_ERR_ARG;
    return shape_error(T, B * C * HW);
}

}  // namespace

// The batch-norm entry points take float or double storage (bf16: SNNLIF_ERR_UNSUPPORTED).
// Returns the element size, or 0 with *rc set to the error.
static size_t bn_element_size(int dtype, int* rc) {
    if (arith_size(dtype) == 0) {
        *rc = SNNLIF_ERR_DTYPE;
        return 0;
    }
    // the cache hints steer the forward kernels only: both sweeps of the backward read x anyway
    if (storage_of(dtype) == SNNLIF_DTYPE_F32) return sizeof(float);
    if (storage_of(dtype) == SNNLIF_DTYPE_F64) return sizeof(double);
    *rc = SNNLIF_ERR_UNSUPPORTED;
    return 0;
}

static bool all_aligned(const void* const* ptrs, int n, size_t bytes) {
    for (int i = 0; i < n; ++i)
        if (!snnlif::aligned_to(ptrs[i], bytes)) return false;
    return true;
}

// Calls the f32 or the f64 instantiation of a launcher with typed pointers.
#define SNNLIF_BN_DISPATCH(es, CALL_F32, CALL_F64) ((es) == sizeof(float) ? (CALL_F32) : (CALL_F64))
#define CF(p) static_cast<const float*>(p)
#define MF(p) static_cast<float*>(p)
#define CD(p) static_cast<const double*>(p)
#define MD(p) static_cast<double*>(p)

int snnlif_bn_fire_s_fp(const void* spatial, const void* weight, const void* bias, const void* var,
                        const void* mean, void* ivar, void* spike, int dtype, int64_t T, int64_t B,
                        int64_t C, int64_t HW, float eps, float alpha, float thresh, void* stream) {
    const TimerScope timer_scope;
    int rc = SNNLIF_OK;
    const size_t es = bn_element_size(dtype, &rc);
    if (es == 0) return rc;
    const int se = bn_shape_error(T, B, C, HW);
    if (se != SNNLIF_OK) return se;
    if (T == 0 || B * C * HW == 0) return SNNLIF_OK;
    if (!spatial || !weight || !bias || !var || !mean || !ivar || !spike) return SNNLIF_ERR_ARG;
    const void* ptrs[7] = {spatial, weight, bias, var, mean, ivar, spike};
    if (!all_aligned(ptrs, 7, es)) return SNNLIF_ERR_ALIGN;
    hipStream_t st = static_cast<hipStream_t>(stream);
    return SNNLIF_BN_DISPATCH(
        es,
        snnlif::bn_forward_f32(CF(spatial), CF(weight), CF(bias), CF(var), CF(mean), MF(ivar),
                               MF(spike), /*from_ivar=*/false, T, B, C, HW, eps, alpha, thresh, hint_of(dtype), st),
        snnlif::bn_forward_f64(CD(spatial), CD(weight), CD(bias), CD(var), CD(mean), MD(ivar),
                               MD(spike), /*from_ivar=*/false, T, B, C, HW, eps, alpha, thresh, hint_of(dtype), st));
}

int snnlif_bn_fire_s_recompute(const void* spatial, const void* weight, const void* bias,
                               const void* ivar, const void* mean, void* spike, int dtype, int64_t T,
                               int64_t B, int64_t C, int64_t HW, float alpha, float thresh,
                               void* stream) {
    const TimerScope timer_scope;
    int rc = SNNLIF_OK;
    const size_t es = bn_element_size(dtype, &rc);
    if (es == 0) return rc;
    const int se = bn_shape_error(T, B, C, HW);
    if (se != SNNLIF_OK) return se;
    if (T == 0 || B * C * HW == 0) return SNNLIF_OK;
    if (!spatial || !weight || !bias || !ivar || !mean || !spike) return SNNLIF_ERR_ARG;
    const void* ptrs[6] = {spatial, weight, bias, ivar, mean, spike};
    if (!all_aligned(ptrs, 6, es)) return SNNLIF_ERR_ALIGN;
    hipStream_t st = static_cast<hipStream_t>(stream);
    return SNNLIF_BN_DISPATCH(
        es,
        snnlif::bn_forward_f32(CF(spatial), CF(weight), CF(bias), CF(ivar), CF(mean), nullptr,
                               MF(spike), /*from_ivar=*/true, T, B, C, HW, 0.f, alpha, thresh, hint_of(dtype), st),
        snnlif::bn_forward_f64(CD(spatial), CD(weight), CD(bias), CD(ivar), CD(mean), nullptr,
                               MD(spike), /*from_ivar=*/true, T, B, C, HW, 0.f, alpha, thresh, hint_of(dtype), st));
}

size_t snnlif_bn_stats_workspace_bytes(int dtype, int64_t T, int64_t B, int64_t C, int64_t HW) {
    int rc = SNNLIF_OK;
    const size_t es = bn_element_size(dtype, &rc);
    if (es == 0 || bn_shape_error(T, B, C, HW) != SNNLIF_OK) return 0;
    if (T == 0 || B * C * HW == 0) return 0;
    return snnlif::bn_stats_workspace_elems(T, B, C, HW) * sizeof(double);
}

int snnlif_bn_stats(const void* spatial, void* mean, void* var, int dtype, int64_t T, int64_t B,
                    int64_t C, int64_t HW, int raw_moments, void* workspace, size_t workspace_bytes,
                    void* stream) {
    const TimerScope timer_scope;
    int rc = SNNLIF_OK;
    const size_t es = bn_element_size(dtype, &rc);
    if (es == 0) return rc;
    const int se = bn_shape_error(T, B, C, HW);
    if (se != SNNLIF_OK) return se;
    if (C == 0) return SNNLIF_OK;
    // a channel without elements has no statistics: refuse rather than divide by zero
    if (T == 0 || B == 0 || HW == 0) return SNNLIF_ERR_ARG;
    if (!spatial || !mean || !var) return SNNLIF_ERR_ARG;
    const void* ptrs[3] = {spatial, mean, var};
    if (!all_aligned(ptrs, 3, es)) return SNNLIF_ERR_ALIGN;
    const size_t need = snnlif::bn_stats_workspace_elems(T, B, C, HW) * sizeof(double);
    if (workspace == nullptr || workspace_bytes < need) return SNNLIF_ERR_WORKSPACE;
    if (!snnlif::aligned_to(workspace, 16)) return SNNLIF_ERR_ALIGN;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const OperationTimer whole_operation(st);
    const int stats_mode = raw_moments != 0 ? snnlif::kStatsMoments : snnlif::kStatsVariance;
    return SNNLIF_BN_DISPATCH(
        es,
        snnlif::bn_stats_f32(CF(spatial), MF(mean), MF(var), stats_mode, T, B, C, HW,
                             MD(workspace), st),
        snnlif::bn_stats_f64(CD(spatial), MD(mean), MD(var), stats_mode, T, B, C, HW,
                             MD(workspace), st));
}

}  // extern "C"

template <typename F>
static snnlif::RunningUpdate<F> running_update(const void* running_mean, const void* running_var,
                                               void* new_running_mean, void* new_running_var,
                                               double keep, double gain_mean, double gain_var) {
    // the factors are rounded to the storage type once, as the framework rounds a Python scalar
    return snnlif::RunningUpdate<F>{static_cast<const F*>(running_mean), static_cast<const F*>(running_var),
                                    static_cast<F*>(new_running_mean), static_cast<F*>(new_running_var),
                                    static_cast<F>(keep), static_cast<F>(gain_mean), static_cast<F>(gain_var)};
}

extern "C" {

int snnlif_bn_stats_running(const void* spatial, void* mean, void* var, const void* running_mean,
                            const void* running_var, void* new_running_mean, void* new_running_var,
                            double keep, double gain_mean, double gain_var, int dtype, int64_t T,
                            int64_t B, int64_t C, int64_t HW, void* workspace, size_t workspace_bytes,
                            void* stream) {
    const TimerScope timer_scope;
    int rc = SNNLIF_OK;
    const size_t es = bn_element_size(dtype, &rc);
    if (es == 0) return rc;
    const int se = bn_shape_error(T, B, C, HW);
    if (se != SNNLIF_OK) return se;
    if (C == 0) return SNNLIF_OK;
    if (T == 0 || B == 0 || HW == 0) return SNNLIF_ERR_ARG;
    if (!spatial || !mean || !var || !running_mean || !running_var || !new_running_mean ||
        !new_running_var)
        return SNNLIF_ERR_ARG;
    const void* ptrs[7] = {spatial, mean, var, running_mean, running_var, new_running_mean, new_running_var};
    if (!all_aligned(ptrs, 7, es)) return SNNLIF_ERR_ALIGN;
    const size_t need = snnlif::bn_stats_workspace_elems(T, B, C, HW) * sizeof(double);
    if (workspace == nullptr || workspace_bytes < need) return SNNLIF_ERR_WORKSPACE;
    if (!snnlif::aligned_to(workspace, 16)) return SNNLIF_ERR_ALIGN;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const OperationTimer whole_operation(st);
    return SNNLIF_BN_DISPATCH(
        es,
        snnlif::bn_stats_f32(CF(spatial), MF(mean), MF(var), snnlif::kStatsVariance, T, B, C, HW,
                             MD(workspace), st,
                             running_update<float>(running_mean, running_var, new_running_mean,
                                                   new_running_var, keep, gain_mean, gain_var)),
        snnlif::bn_stats_f64(CD(spatial), MD(mean), MD(var), snnlif::kStatsVariance, T, B, C, HW,
                             MD(workspace), st,
                             running_update<double>(running_mean, running_var, new_running_mean,
                                                    new_running_var, keep, gain_mean, gain_var)));
}

int snnlif_bn_moments_finish(const void* first, const void* second, void* mean, void* var,
                             const void* running_mean, const void* running_var,
                             void* new_running_mean, void* new_running_var, double world_size,
                             double keep, double gain_mean, double gain_var, int dtype, int64_t C,
                             void* stream) {
    const TimerScope timer_scope;
    int rc = SNNLIF_OK;
    const size_t es = bn_element_size(dtype, &rc);
    if (es == 0) return rc;
    if (C < 0 || !(world_size >= 1.0)) return SNNLIF_ERR_ARG;
    if (C == 0) return SNNLIF_OK;
    if (!first || !second || !mean || !var) return SNNLIF_ERR_ARG;
    // the running pair is optional, but all four of its pointers go together
    const int given = (running_mean != nullptr) + (running_var != nullptr) +
                      (new_running_mean != nullptr) + (new_running_var != nullptr);
    if (given != 0 && given != 4) return SNNLIF_ERR_ARG;
    const void* ptrs[8] = {first, second, mean, var, running_mean, running_var, new_running_mean, new_running_var};
    if (!all_aligned(ptrs, given ? 8 : 4, es)) return SNNLIF_ERR_ALIGN;
    hipStream_t st = static_cast<hipStream_t>(stream);
    // 1 / world in the storage type: the framework divides by a scalar as a product with its reciprocal
    return SNNLIF_BN_DISPATCH(
        es,
        snnlif::bn_moments_finish_f32(CF(first), CF(second), MF(mean), MF(var),
                                      1.0f / static_cast<float>(world_size),
                                      running_update<float>(running_mean, running_var, new_running_mean,
                                                            new_running_var, keep, gain_mean, gain_var),
                                      C, st),
        snnlif::bn_moments_finish_f64(CD(first), CD(second), MD(mean), MD(var), 1.0 / world_size,
                                      running_update<double>(running_mean, running_var, new_running_mean,
                                                             new_running_var, keep, gain_mean, gain_var),
                                      C, st));
}

int snnlif_channel_sum(const void* grad, void* sum, int dtype, int64_t T, int64_t B, int64_t C,
                       int64_t HW, void* workspace, size_t workspace_bytes, void* stream) {
    const TimerScope timer_scope;
    int rc = SNNLIF_OK;
    const size_t es = bn_element_size(dtype, &rc);
    if (es == 0) return rc;
    const int se = bn_shape_error(T, B, C, HW);
    if (se != SNNLIF_OK) return se;
    if (C == 0) return SNNLIF_OK;
    // the kernels read a channel's first element: nothing to read in an empty channel
    if (T == 0 || B == 0 || HW == 0) return SNNLIF_ERR_ARG;
    if (!grad || !sum) return SNNLIF_ERR_ARG;
    const void* ptrs[2] = {grad, sum};
    if (!all_aligned(ptrs, 2, es)) return SNNLIF_ERR_ALIGN;
    const size_t need = snnlif::bn_stats_workspace_elems(T, B, C, HW) * sizeof(double);
    if (workspace == nullptr || workspace_bytes < need) return SNNLIF_ERR_WORKSPACE;
    if (!snnlif::aligned_to(workspace, 16)) return SNNLIF_ERR_ALIGN;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const OperationTimer whole_operation(st);
    return SNNLIF_BN_DISPATCH(
        es,
        snnlif::bn_stats_f32(CF(grad), MF(sum), nullptr, snnlif::kStatsSums, T, B, C, HW,
                             MD(workspace), st),
        snnlif::bn_stats_f64(CD(grad), MD(sum), nullptr, snnlif::kStatsSums, T, B, C, HW,
                             MD(workspace), st));
}

size_t snnlif_bn_fire_bp_workspace_bytes(int dtype, int64_t T, int64_t B, int64_t C, int64_t HW) {
    int rc = SNNLIF_OK;
    const size_t es = bn_element_size(dtype, &rc);
    if (es == 0 || bn_shape_error(T, B, C, HW) != SNNLIF_OK) return 0;
    if (T == 0 || B * C * HW == 0) return 0;
    return snnlif::bn_backward_workspace_elems(T, B, C, HW) * es;
}

// Shared argument checks of the three backward entry points; `needs_workspace` = sweep 1 runs.
static_assert(snnlif::kBnLdsBoundaryMaxT == SNNLIF_BP_NO_WORKSPACE_MAX_T &&
                  snnlif::kBnSegment == snnlif::kSegment,
              "the batch-norm backward cuts time the way the plain backward does");

static int bn_backward_checks(int dtype, int64_t T, int64_t B, int64_t C, int64_t HW,
                              const void* const* ptrs, int n, bool needs_workspace,
                              const void* workspace, size_t workspace_bytes, size_t* es_out,
                              bool* empty) {
    int rc = SNNLIF_OK;
    const size_t es = bn_element_size(dtype, &rc);
    if (es == 0) return rc;
    const int se = bn_shape_error(T, B, C, HW);
    if (se != SNNLIF_OK) return se;
    *es_out = es;
    *empty = (T == 0 || B * C * HW == 0);
    if (*empty) return SNNLIF_OK;
    for (int i = 0; i < n; ++i)
        if (ptrs[i] == nullptr) return SNNLIF_ERR_ARG;
    if (!all_aligned(ptrs, n, es)) return SNNLIF_ERR_ALIGN;
    if (needs_workspace) {
        const size_t need = snnlif::bn_backward_workspace_elems(T, B, C, HW) * es;
        if (workspace == nullptr || workspace_bytes < need) return SNNLIF_ERR_WORKSPACE;
        if (!snnlif::aligned_to(workspace, 16)) return SNNLIF_ERR_ALIGN;
    }
    return SNNLIF_OK;
}

int snnlif_bn_fire_bp(const void* spatial, const void* weight, const void* bias, const void* ivar,
                      const void* mean, const void* grad_spike, void* grad_spatial,
                      void* grad_weight, void* grad_bias, int dtype, int64_t T, int64_t B, int64_t C,
                      int64_t HW, float alpha, float thresh, float beta, float interval,
                      void* workspace, size_t workspace_bytes, void* stream) {
    const TimerScope timer_scope;
    const void* ptrs[9] = {spatial, weight, bias, ivar, mean, grad_spike, grad_spatial, grad_weight,
                           grad_bias};
    size_t es = 0;
    bool empty = false;
    const int rc = bn_backward_checks(dtype, T, B, C, HW, ptrs, 9, true, workspace, workspace_bytes,
                                      &es, &empty);
    if (rc != SNNLIF_OK || empty) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const OperationTimer whole_operation(st);
    return SNNLIF_BN_DISPATCH(
        es,
        snnlif::bn_backward_f32(CF(spatial), CF(weight), CF(bias), CF(ivar), CF(mean), CF(grad_spike),
                                MF(grad_spatial), MF(grad_weight), MF(grad_bias), T, B, C, HW, alpha,
                                thresh, beta, interval, MF(workspace), st),
        snnlif::bn_backward_f64(CD(spatial), CD(weight), CD(bias), CD(ivar), CD(mean), CD(grad_spike),
                                MD(grad_spatial), MD(grad_weight), MD(grad_bias), T, B, C, HW, alpha,
                                thresh, beta, interval, MD(workspace), st));
}

int snnlif_bn_fire_bp_static(const void* spatial, const void* weight, const void* bias,
                             const void* ivar, const void* mean, const void* grad_spike,
                             void* grad_spatial, void* grad_weight, void* grad_bias, int dtype,
                             int64_t T, int64_t B, int64_t C, int64_t HW, float alpha, float thresh,
                             float beta, float interval, void* stream) {
    const TimerScope timer_scope;
    const void* ptrs[9] = {spatial, weight, bias, ivar, mean, grad_spike, grad_spatial, grad_weight,
                           grad_bias};
    size_t es = 0;
    bool empty = false;
    int rc = bn_backward_checks(dtype, T, B, C, HW, ptrs, 9, false, nullptr, 0, &es, &empty);
    if (rc != SNNLIF_OK || empty) return rc;
    if (snnlif::bn_backward_workspace_elems(T, B, C, HW) * es > SNNLIF_STATIC_SCRATCH_BYTES)
        return SNNLIF_ERR_SCRATCH;
    void* workspace = nullptr;
    rc = static_scratch(&workspace);
    if (rc != SNNLIF_OK) return rc;
    // Every value the reduction reads from the scratch array is written by sweep 1 of this same call,
    // so nothing has to be cleared between calls.
    hipStream_t st = static_cast<hipStream_t>(stream);
    const OperationTimer whole_operation(st);
    return SNNLIF_BN_DISPATCH(
        es,
        snnlif::bn_backward_f32(CF(spatial), CF(weight), CF(bias), CF(ivar), CF(mean), CF(grad_spike),
                                MF(grad_spatial), MF(grad_weight), MF(grad_bias), T, B, C, HW, alpha,
                                thresh, beta, interval, MF(workspace), st),
        snnlif::bn_backward_f64(CD(spatial), CD(weight), CD(bias), CD(ivar), CD(mean), CD(grad_spike),
                                MD(grad_spatial), MD(grad_weight), MD(grad_bias), T, B, C, HW, alpha,
                                thresh, beta, interval, MD(workspace), st));
}

int snnlif_bn_fire_bp_dist1(const void* spatial, const void* weight, const void* bias,
                            const void* ivar, const void* mean, const void* grad_spike,
                            void* mean_gxhat, void* mean_gxhatx, void* grad_weight, void* grad_bias,
                            int dtype, int64_t T, int64_t B, int64_t C, int64_t HW, float alpha,
                            float thresh, float beta, float interval, void* workspace,
                            size_t workspace_bytes, void* stream) {
    const TimerScope timer_scope;
    const void* ptrs[10] = {spatial, weight, bias, ivar, mean, grad_spike, mean_gxhat, mean_gxhatx,
                            grad_weight, grad_bias};
    size_t es = 0;
    bool empty = false;
    // an empty batch has no statistics to report: the channel arrays are left untouched
    const int rc = bn_backward_checks(dtype, T, B, C, HW, ptrs, 10, true, workspace,
                                      workspace_bytes, &es, &empty);
    if (rc != SNNLIF_OK || empty) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const OperationTimer whole_operation(st);
    return SNNLIF_BN_DISPATCH(
        es,
        snnlif::bn_backward_stats_f32(CF(spatial), CF(weight), CF(bias), CF(ivar), CF(mean),
                                      CF(grad_spike), MF(grad_weight), MF(grad_bias), MF(mean_gxhat),
                                      MF(mean_gxhatx), T, B, C, HW, alpha, thresh, beta, interval,
                                      MF(workspace), st),
        snnlif::bn_backward_stats_f64(CD(spatial), CD(weight), CD(bias), CD(ivar), CD(mean),
                                      CD(grad_spike), MD(grad_weight), MD(grad_bias), MD(mean_gxhat),
                                      MD(mean_gxhatx), T, B, C, HW, alpha, thresh, beta, interval,
                                      MD(workspace), st));
}

int snnlif_bn_fire_bp_dist2(const void* spatial, const void* weight, const void* bias,
                            const void* ivar, const void* mean, const void* grad_spike,
                            const void* grad_xhat, const void* grad_xhatx, void* grad_spatial,
                            int dtype, int64_t T, int64_t B, int64_t C, int64_t HW, float alpha,
                            float thresh, float beta, float interval, void* stream) {
    const TimerScope timer_scope;
    const void* ptrs[9] = {spatial, weight, bias, ivar, mean, grad_spike, grad_xhat, grad_xhatx,
                           grad_spatial};
    size_t es = 0;
    bool empty = false;
    const int rc = bn_backward_checks(dtype, T, B, C, HW, ptrs, 9, false, nullptr, 0, &es, &empty);
    if (rc != SNNLIF_OK || empty) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    return SNNLIF_BN_DISPATCH(
        es,
        snnlif::bn_backward_input_f32(CF(spatial), CF(weight), CF(bias), CF(ivar), CF(mean),
                                      CF(grad_spike), CF(grad_xhat), CF(grad_xhatx), MF(grad_spatial),
                                      T, B, C, HW, alpha, thresh, beta, interval, st),
        snnlif::bn_backward_input_f64(CD(spatial), CD(weight), CD(bias), CD(ivar), CD(mean),
                                      CD(grad_spike), CD(grad_xhat), CD(grad_xhatx), MD(grad_spatial),
                                      T, B, C, HW, alpha, thresh, beta, interval, st));
}

// ---- plain batch norm (no fire recurrence) --------------------------------------------------------

int snnlif_bn_fp(const void* x_bn, const void* weight, const void* bias, const void* var,
                 const void* mean, void* ivar, void* y_bn, int dtype, int64_t T, int64_t B, int64_t C,
                 int64_t HW, float eps, void* stream) {
    const TimerScope timer_scope;
    int rc = SNNLIF_OK;
    const size_t es = bn_element_size(dtype, &rc);
    if (es == 0) return rc;
    const int se = bn_shape_error(T, B, C, HW);
    if (se != SNNLIF_OK) return se;
    if (T == 0 || B * C * HW == 0) return SNNLIF_OK;
    if (!x_bn || !weight || !bias || !var || !mean || !ivar || !y_bn) return SNNLIF_ERR_ARG;
    const void* ptrs[7] = {x_bn, weight, bias, var, mean, ivar, y_bn};
    if (!all_aligned(ptrs, 7, es)) return SNNLIF_ERR_ALIGN;
    hipStream_t st = static_cast<hipStream_t>(stream);
    return SNNLIF_BN_DISPATCH(
        es,
        snnlif::bn_plain_forward_f32(CF(x_bn), CF(weight), CF(bias), CF(var), CF(mean), MF(ivar),
                                     MF(y_bn), T, B, C, HW, eps, st),
        snnlif::bn_plain_forward_f64(CD(x_bn), CD(weight), CD(bias), CD(var), CD(mean), MD(ivar),
                                     MD(y_bn), T, B, C, HW, eps, st));
}

size_t snnlif_bn_bp_workspace_bytes(int dtype, int64_t T, int64_t B, int64_t C, int64_t HW) {
    int rc = SNNLIF_OK;
    const size_t es = bn_element_size(dtype, &rc);
    if (es == 0 || bn_shape_error(T, B, C, HW) != SNNLIF_OK) return 0;
    if (T == 0 || B * C * HW == 0) return 0;
    return snnlif::bn_plain_workspace_elems(T, B, C, HW) * es;
}

// Shared argument checks of the three plain batch-norm backward entry points.
static int bn_plain_backward_checks(int dtype, int64_t T, int64_t B, int64_t C, int64_t HW,
                                    const void* const* ptrs, int n, bool needs_workspace,
                                    const void* workspace, size_t workspace_bytes, size_t* es_out,
                                    bool* empty) {
    int rc = SNNLIF_OK;
    const size_t es = bn_element_size(dtype, &rc);
    if (es == 0) return rc;
    const int se = bn_shape_error(T, B, C, HW);
    if (se != SNNLIF_OK) return se;
    *es_out = es;
    *empty = (T == 0 || B * C * HW == 0);
    if (*empty) return SNNLIF_OK;
    for (int i = 0; i < n; ++i)
        if (ptrs[i] == nullptr) return SNNLIF_ERR_ARG;
    if (!all_aligned(ptrs, n, es)) return SNNLIF_ERR_ALIGN;
    if (needs_workspace) {
        const size_t need = snnlif::bn_plain_workspace_elems(T, B, C, HW) * es;
        if (workspace == nullptr || workspace_bytes < need) return SNNLIF_ERR_WORKSPACE;
        if (!snnlif::aligned_to(workspace, 16)) return SNNLIF_ERR_ALIGN;
    }
    return SNNLIF_OK;
}

int snnlif_bn_bp(const void* x_bn, const void* weight, const void* ivar, const void* mean,
                 const void* grad_y_bn, void* grad_x_bn, void* grad_weight, void* grad_bias, int dtype,
                 int64_t T, int64_t B, int64_t C, int64_t HW, void* workspace, size_t workspace_bytes,
                 void* stream) {
    const TimerScope timer_scope;
    const void* ptrs[8] = {x_bn, weight, ivar, mean, grad_y_bn, grad_x_bn, grad_weight, grad_bias};
    size_t es = 0;
    bool empty = false;
    const int rc = bn_plain_backward_checks(dtype, T, B, C, HW, ptrs, 8, true, workspace,
                                            workspace_bytes, &es, &empty);
    if (rc != SNNLIF_OK || empty) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const OperationTimer whole_operation(st);
    return SNNLIF_BN_DISPATCH(
        es,
        snnlif::bn_plain_backward_f32(CF(x_bn), CF(weight), CF(ivar), CF(mean), CF(grad_y_bn),
                                      MF(grad_x_bn), MF(grad_weight), MF(grad_bias), T, B, C, HW,
                                      MF(workspace), st),
        snnlif::bn_plain_backward_f64(CD(x_bn), CD(weight), CD(ivar), CD(mean), CD(grad_y_bn),
                                      MD(grad_x_bn), MD(grad_weight), MD(grad_bias), T, B, C, HW,
                                      MD(workspace), st));
}

int snnlif_bn_bp_dist1(const void* x_bn, const void* weight, const void* ivar, const void* mean,
                       const void* grad_y_bn, void* mean_gxhat, void* mean_gxhatx, void* grad_weight,
                       void* grad_bias, int dtype, int64_t T, int64_t B, int64_t C, int64_t HW,
                       void* workspace, size_t workspace_bytes, void* stream) {
    const TimerScope timer_scope;
    const void* ptrs[9] = {x_bn, weight, ivar, mean, grad_y_bn, mean_gxhat, mean_gxhatx, grad_weight,
                           grad_bias};
    size_t es = 0;
    bool empty = false;
    // an empty batch has no statistics to report: the channel arrays are left untouched
    const int rc = bn_plain_backward_checks(dtype, T, B, C, HW, ptrs, 9, true, workspace,
                                            workspace_bytes, &es, &empty);
    if (rc != SNNLIF_OK || empty) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const OperationTimer whole_operation(st);
    return SNNLIF_BN_DISPATCH(
        es,
        snnlif::bn_plain_backward_stats_f32(CF(x_bn), CF(weight), CF(ivar), CF(mean), CF(grad_y_bn),
                                            MF(grad_weight), MF(grad_bias), MF(mean_gxhat),
                                            MF(mean_gxhatx), T, B, C, HW, MF(workspace), st),
        snnlif::bn_plain_backward_stats_f64(CD(x_bn), CD(weight), CD(ivar), CD(mean), CD(grad_y_bn),
                                            MD(grad_weight), MD(grad_bias), MD(mean_gxhat),
                                            MD(mean_gxhatx), T, B, C, HW, MD(workspace), st));
}

int snnlif_bn_bp_dist2(const void* x_bn, const void* weight, const void* ivar, const void* mean,
                       const void* grad_y_bn, const void* grad_xhat, const void* grad_xhatx,
                       void* grad_x_bn, int dtype, int64_t T, int64_t B, int64_t C, int64_t HW,
                       void* stream) {
    const TimerScope timer_scope;
    const void* ptrs[8] = {x_bn, weight, ivar, mean, grad_y_bn, grad_xhat, grad_xhatx, grad_x_bn};
    size_t es = 0;
    bool empty = false;
    const int rc = bn_plain_backward_checks(dtype, T, B, C, HW, ptrs, 8, false, nullptr, 0, &es, &empty);
    if (rc != SNNLIF_OK || empty) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    return SNNLIF_BN_DISPATCH(
        es,
        snnlif::bn_plain_backward_input_f32(CF(x_bn), CF(weight), CF(ivar), CF(mean), CF(grad_y_bn),
                                            CF(grad_xhat), CF(grad_xhatx), MF(grad_x_bn), T, B, C, HW,
                                            st),
        snnlif::bn_plain_backward_input_f64(CD(x_bn), CD(weight), CD(ivar), CD(mean), CD(grad_y_bn),
                                            CD(grad_xhat), CD(grad_xhatx), MD(grad_x_bn), T, B, C, HW,
                                            st));
}

#undef SNNLIF_BN_DISPATCH
#undef CF
#undef MF
#undef CD
#undef MD

}  // extern "C"
