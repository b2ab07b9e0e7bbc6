// C ABI of libsnnlif_gfx950.so (include/snnlib_lif.h): argument checks and dtype dispatch in front
// of the per-dtype kernel launchers.  No device code lives in this file.
#include "lif_bn.h"
#include "lif_kernels.h"

namespace snnlif {
thread_local KernelTimer tl_kernel_timer;
}  // namespace snnlif

namespace {

inline size_t arith_size(int dtype) {
    switch (dtype) {
        case SNNLIF_DTYPE_F32: return sizeof(float);
        case SNNLIF_DTYPE_F64: return sizeof(double);
        case SNNLIF_DTYPE_BF16: return sizeof(float);
        default: return 0;
    }
}

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
        case SNNLIF_ERR_DTYPE: return "snnlif: unsupported dtype (expected SNNLIF_DTYPE_F32, _F64 or _BF16)";
        case SNNLIF_ERR_WORKSPACE: return "snnlif: workspace missing or smaller than snnlif_fire_bp_workspace_bytes()";
        case SNNLIF_ERR_ALIGN: return "snnlif: pointer not aligned to its element size (workspace: 16 bytes)";
        case SNNLIF_ERR_UNSUPPORTED: return "snnlif: not implemented for these arguments (batch-norm fire: fp32 only, backward T <= 1024)";
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
        case SNNLIF_DTYPE_F32: return snnlif::forward_f32(spatial, mem, spike, T, N, alpha, thresh, st);
        case SNNLIF_DTYPE_F64: return snnlif::forward_f64(spatial, mem, spike, T, N, alpha, thresh, st);
        default: return snnlif::forward_bf16(spatial, mem, spike, T, N, alpha, thresh, st);
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
    if (T <= SNNLIF_BP_NO_WORKSPACE_MAX_T) return 0;
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
            return snnlif::backward_f32(spatial, grad_spike, grad_spatial, T, N, alpha, thresh, beta, interval, workspace, workspace_bytes, st);
        case SNNLIF_DTYPE_F64:
            return snnlif::backward_f64(spatial, grad_spike, grad_spatial, T, N, alpha, thresh, beta, interval, workspace, workspace_bytes, st);
        default:
            return snnlif::backward_bf16(spatial, grad_spike, grad_spatial, T, N, alpha, thresh, beta, interval, workspace, workspace_bytes, st);
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

int snnlif_bn_fire_s_fp(const void* spatial, const void* weight, const void* bias, const void* var,
                        const void* mean, void* ivar, void* spike, int dtype, int64_t T, int64_t B,
                        int64_t C, int64_t HW, float eps, float alpha, float thresh, void* stream) {
    if (arith_size(dtype) == 0) return SNNLIF_ERR_DTYPE;
    if (dtype != SNNLIF_DTYPE_F32) return SNNLIF_ERR_UNSUPPORTED;
    const int se = bn_shape_error(T, B, C, HW);
    if (se != SNNLIF_OK) return se;
    if (T == 0 || B * C * HW == 0) return SNNLIF_OK;
    if (!spatial || !weight || !bias || !var || !mean || !ivar || !spike) return SNNLIF_ERR_ARG;
    const void* ptrs[7] = {spatial, weight, bias, var, mean, ivar, spike};
    for (const void* p : ptrs)
        if (!snnlif::aligned_to(p, sizeof(float))) return SNNLIF_ERR_ALIGN;
    return snnlif::bn_forward_f32(
        static_cast<const float*>(spatial), static_cast<const float*>(weight),
        static_cast<const float*>(bias), static_cast<const float*>(var),
        static_cast<const float*>(mean), static_cast<float*>(ivar), static_cast<float*>(spike),
        /*from_ivar=*/false, T, B, C, HW, eps, alpha, thresh, static_cast<hipStream_t>(stream));
}

int snnlif_bn_fire_s_recompute(const void* spatial, const void* weight, const void* bias,
                               const void* ivar, const void* mean, void* spike, int dtype, int64_t T,
                               int64_t B, int64_t C, int64_t HW, float alpha, float thresh,
                               void* stream) {
    if (arith_size(dtype) == 0) return SNNLIF_ERR_DTYPE;
    if (dtype != SNNLIF_DTYPE_F32) return SNNLIF_ERR_UNSUPPORTED;
    const int se = bn_shape_error(T, B, C, HW);
    if (se != SNNLIF_OK) return se;
    if (T == 0 || B * C * HW == 0) return SNNLIF_OK;
    if (!spatial || !weight || !bias || !ivar || !mean || !spike) return SNNLIF_ERR_ARG;
    const void* ptrs[6] = {spatial, weight, bias, ivar, mean, spike};
    for (const void* p : ptrs)
        if (!snnlif::aligned_to(p, sizeof(float))) return SNNLIF_ERR_ALIGN;
    return snnlif::bn_forward_f32(
        static_cast<const float*>(spatial), static_cast<const float*>(weight),
        static_cast<const float*>(bias), static_cast<const float*>(ivar),
        static_cast<const float*>(mean), nullptr, static_cast<float*>(spike), /*from_ivar=*/true, T,
        B, C, HW, 0.f, alpha, thresh, static_cast<hipStream_t>(stream));
}

size_t snnlif_bn_fire_bp_workspace_bytes(int dtype, int64_t T, int64_t B, int64_t C, int64_t HW) {
    if (dtype != SNNLIF_DTYPE_F32 || bn_shape_error(T, B, C, HW) != SNNLIF_OK) return 0;
    if (T == 0 || B * C * HW == 0) return 0;
    return snnlif::bn_backward_workspace_floats(B, C, HW) * sizeof(float);
}

int snnlif_bn_fire_bp(const void* spatial, const void* weight, const void* bias, const void* ivar,
                      const void* mean, const void* grad_spike, void* grad_spatial,
                      void* grad_weight, void* grad_bias, int dtype, int64_t T, int64_t B, int64_t C,
                      int64_t HW, float alpha, float thresh, float beta, float interval,
                      void* workspace, size_t workspace_bytes, void* stream) {
    if (arith_size(dtype) == 0) return SNNLIF_ERR_DTYPE;
    if (dtype != SNNLIF_DTYPE_F32) return SNNLIF_ERR_UNSUPPORTED;
    const int se = bn_shape_error(T, B, C, HW);
    if (se != SNNLIF_OK) return se;
    if (T == 0 || B * C * HW == 0) return SNNLIF_OK;
    if (T > SNNLIF_BP_NO_WORKSPACE_MAX_T) return SNNLIF_ERR_UNSUPPORTED;
    if (!spatial || !weight || !bias || !ivar || !mean || !grad_spike || !grad_spatial ||
        !grad_weight || !grad_bias)
        return SNNLIF_ERR_ARG;
    const void* ptrs[9] = {spatial, weight, bias, ivar, mean, grad_spike, grad_spatial, grad_weight, grad_bias};
    for (const void* p : ptrs)
        if (!snnlif::aligned_to(p, sizeof(float))) return SNNLIF_ERR_ALIGN;
    const size_t need = snnlif::bn_backward_workspace_floats(B, C, HW) * sizeof(float);
    if (workspace == nullptr || workspace_bytes < need) return SNNLIF_ERR_WORKSPACE;
    if (!snnlif::aligned_to(workspace, 16)) return SNNLIF_ERR_ALIGN;
    return snnlif::bn_backward_f32(
        static_cast<const float*>(spatial), static_cast<const float*>(weight),
        static_cast<const float*>(bias), static_cast<const float*>(ivar),
        static_cast<const float*>(mean), static_cast<const float*>(grad_spike),
        static_cast<float*>(grad_spatial), static_cast<float*>(grad_weight),
        static_cast<float*>(grad_bias), T, B, C, HW, alpha, thresh, beta, interval,
        static_cast<float*>(workspace), static_cast<hipStream_t>(stream));
}

int snnlif_bn_fire_bp_dist1(const void* spatial, const void* weight, const void* bias,
                            const void* ivar, const void* mean, const void* grad_spike,
                            void* mean_gxhat, void* mean_gxhatx, void* grad_weight, void* grad_bias,
                            int dtype, int64_t T, int64_t B, int64_t C, int64_t HW, float alpha,
                            float thresh, float beta, float interval, void* workspace,
                            size_t workspace_bytes, void* stream) {
    if (arith_size(dtype) == 0) return SNNLIF_ERR_DTYPE;
    if (dtype != SNNLIF_DTYPE_F32) return SNNLIF_ERR_UNSUPPORTED;
    const int se = bn_shape_error(T, B, C, HW);
    if (se != SNNLIF_OK) return se;
    // an empty batch has no statistics to report: the channel arrays are left untouched
    if (T == 0 || B * C * HW == 0) return SNNLIF_OK;
    if (T > SNNLIF_BP_NO_WORKSPACE_MAX_T) return SNNLIF_ERR_UNSUPPORTED;
    if (!spatial || !weight || !bias || !ivar || !mean || !grad_spike || !mean_gxhat ||
        !mean_gxhatx || !grad_weight || !grad_bias)
        return SNNLIF_ERR_ARG;
    const void* ptrs[10] = {spatial, weight, bias, ivar, mean, grad_spike, mean_gxhat, mean_gxhatx,
                            grad_weight, grad_bias};
    for (const void* p : ptrs)
        if (!snnlif::aligned_to(p, sizeof(float))) return SNNLIF_ERR_ALIGN;
    const size_t need = snnlif::bn_backward_workspace_floats(B, C, HW) * sizeof(float);
    if (workspace == nullptr || workspace_bytes < need) return SNNLIF_ERR_WORKSPACE;
    if (!snnlif::aligned_to(workspace, 16)) return SNNLIF_ERR_ALIGN;
    return snnlif::bn_backward_stats_f32(
        static_cast<const float*>(spatial), static_cast<const float*>(weight),
        static_cast<const float*>(bias), static_cast<const float*>(ivar),
        static_cast<const float*>(mean), static_cast<const float*>(grad_spike),
        static_cast<float*>(grad_weight), static_cast<float*>(grad_bias),
        static_cast<float*>(mean_gxhat), static_cast<float*>(mean_gxhatx), T, B, C, HW, alpha,
        thresh, beta, interval, static_cast<float*>(workspace), static_cast<hipStream_t>(stream));
}

int snnlif_bn_fire_bp_dist2(const void* spatial, const void* weight, const void* bias,
                            const void* ivar, const void* mean, const void* grad_spike,
                            const void* grad_xhat, const void* grad_xhatx, void* grad_spatial,
                            int dtype, int64_t T, int64_t B, int64_t C, int64_t HW, float alpha,
                            float thresh, float beta, float interval, void* stream) {
    if (arith_size(dtype) == 0) return SNNLIF_ERR_DTYPE;
    if (dtype != SNNLIF_DTYPE_F32) return SNNLIF_ERR_UNSUPPORTED;
    const int se = bn_shape_error(T, B, C, HW);
    if (se != SNNLIF_OK) return se;
    if (T == 0 || B * C * HW == 0) return SNNLIF_OK;
    if (T > SNNLIF_BP_NO_WORKSPACE_MAX_T) return SNNLIF_ERR_UNSUPPORTED;
    if (!spatial || !weight || !bias || !ivar || !mean || !grad_spike || !grad_xhat || !grad_xhatx ||
        !grad_spatial)
        return SNNLIF_ERR_ARG;
    const void* ptrs[9] = {spatial, weight, bias, ivar, mean, grad_spike, grad_xhat, grad_xhatx,
                           grad_spatial};
    for (const void* p : ptrs)
        if (!snnlif::aligned_to(p, sizeof(float))) return SNNLIF_ERR_ALIGN;
    return snnlif::bn_backward_input_f32(
        static_cast<const float*>(spatial), static_cast<const float*>(weight),
        static_cast<const float*>(bias), static_cast<const float*>(ivar),
        static_cast<const float*>(mean), static_cast<const float*>(grad_spike),
        static_cast<const float*>(grad_xhat), static_cast<const float*>(grad_xhatx),
        static_cast<float*>(grad_spatial), T, B, C, HW, alpha, thresh, beta, interval,
        static_cast<hipStream_t>(stream));
}

}  // extern "C"
