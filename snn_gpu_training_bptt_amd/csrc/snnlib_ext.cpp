// Python extension module `snnlib` for PyTorch-ROCm: the operator boundary that
// snnlib_func.FireFunc calls (reference: snnlib/example/snnlib_func.py:25-34).
//
// It exposes the reference's positional signatures (snnlib/cuda/snn.cpp:11-17, 270-279, bound at
// :799 and :813)
//     fire_s_fp(spatial, alpha, thresh)                               -> spike
//     fire_bp(spatial, grad_spike, alpha, thresh, beta, interval)     -> grad_spatial
// plus fire_us_fp(spatial, alpha, thresh) -> (mem, spike), the public face of the reference's
// internal fire_us_fp_kernel (snnlib/cuda/snn_kernel_bp.cu:54-93), and the fire-then-linear /
// fire-then-convolution layer ops with the reference's signatures
// (snnlib/cuda/snn.cpp:112-120, 206-223, 569-582, 740-761; bound at :806, :810, :817, :821)
//     fire_fc_fp(spatial, weight_fc, bias_fc, alpha, thresh)                              -> fc
//     fire_fc_bp(spatial, grad_fc, weight_fc, bias_fc, dim_fc, alpha, thresh, beta, interval)
//                                                     -> [grad_spatial, grad_weight_fc, grad_bias_fc]
//     fire_conv_fp(spatial, weight_conv, bias_conv, stride, padding, dilation, groups, benchmark,
//                  deterministic, alpha, thresh)                                           -> conv
//     fire_conv_bp(spatial, grad_conv, weight_conv, stride, padding, dilation, groups, benchmark,
//                  deterministic, allow_tf32, dim_conv, alpha, thresh, beta, interval)
//                                                 -> [grad_spatial, grad_weight_conv, grad_bias_conv]
// and the batch-norm + fire op (snnlib/cuda/snn.cpp:20-40 region for bn_fire_s_fp, :800; bn_fire_bp :814)
//     bn_fire_s_fp(spatial, weight_bn, bias_bn, var, mean, eps_bn, alpha, thresh)  -> [ivar, spike]
//     bn_fire_bp(spatial, weight_bn, bias_bn, ivar, mean, dim_bn, grad_spike, alpha, thresh, beta,
//                interval)                       -> [grad_spatial, grad_weight_bn, grad_bias_bn]
// and the remaining single-GPU layer ops of the reference's binding table, same positional
// signatures (snnlib/cuda/snn.cpp:30-40, 85-101, 130-137, 162-188, 239-253, 293-304, 484-506,
// 594-603, 630-660, 779-795; bound at :802-803, :805, :807, :809, :811, :816, :818, :820, :822):
//     bn_fp, bn_bp, bn_fire_fc_fp, bn_fire_fc_bp, fc_fp, fc_bp, bn_fire_conv_fp, bn_fire_conv_bp,
//     conv_fp, conv_bp
// (the *_dist1 / *_dist2 halves for multi-GPU synchronised batch norm are not provided),
// in which the fire part runs on this library's kernels and the linear / convolution part stays on
// PyTorch-ROCm (rocBLAS / MIOpen through ATen), issued once with the time axis folded into the
// batch instead of once per time step as the reference's host loops do
// (snnlib/cuda/snn_kernel_fp.cu:314-326, 444-447; snnlib/cuda/snn_kernel_bp.cu:1099-1117, 1382-1390).
//
// This file only validates tensors, allocates outputs and forwards raw device pointers to the C ABI
// of libsnnlif_gfx950.so (include/snnlib_lif.h); all device code lives there.  Unlike the reference
// launchers (snnlib/cuda/snn_kernel_fp.cu:55-73: no checks, legacy default stream, no device guard),
// it checks device / dtype / shape, makes the input dense, switches to the tensor's device and
// launches on PyTorch's current stream for that device.

#include <torch/extension.h>

#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <tuple>
#include <vector>

#include "snnlib_lif.h"

namespace {

int storage_dtype(const torch::Tensor& t, const char* op) {
    switch (t.scalar_type()) {
        case at::kFloat: return SNNLIF_DTYPE_F32;
        case at::kDouble: return SNNLIF_DTYPE_F64;
        case at::kBFloat16: return SNNLIF_DTYPE_BF16;
        default:
            TORCH_CHECK(false, "snnlib.", op, ": unsupported dtype ", t.scalar_type(),
                        " (supported: float32, float64, bfloat16)");
    }
    return -1;
}

void check_input(const torch::Tensor& t, const char* op, const char* name) {
    TORCH_CHECK(t.defined(), "snnlib.", op, ": ", name, " is undefined");
    TORCH_CHECK(t.is_cuda(), "snnlib.", op, ": ", name,
                " must live on a ROCm GPU (this build has no CPU path), got device ", t.device());
    TORCH_CHECK(t.dim() >= 2, "snnlib.", op, ": ", name,
                " must be shaped [T, B, ...], got ", t.dim(), " dimension(s)");
    TORCH_CHECK(!t.is_complex(), "snnlib.", op, ": complex tensors are not supported");
}

void check_rc(int rc, const char* op) {
    TORCH_CHECK(rc == SNNLIF_OK, "snnlib.", op, ": ", snnlif_strerror(rc), " (code ", rc, ")");
}

struct Dims {
    int64_t T;
    int64_t N;
};

Dims dims_of(const torch::Tensor& t) {
    const int64_t T = t.size(0);
    return Dims{T, T == 0 ? 0 : t.numel() / T};
}

torch::Tensor fire_s_fp(torch::Tensor spatial, float alpha, float thresh) {
    check_input(spatial, "fire_s_fp", "spatial");
    const int dtype = storage_dtype(spatial, "fire_s_fp");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(spatial.device());
    torch::Tensor x = spatial.contiguous();
    torch::Tensor spike = torch::empty_like(x, at::MemoryFormat::Contiguous);
    const Dims d = dims_of(x);
    auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
    check_rc(snnlif_fire_s_fp(x.data_ptr(), spike.data_ptr(), dtype, d.T, d.N, alpha, thresh,
                              stream.stream()),
             "fire_s_fp");
    return spike;
}

std::tuple<torch::Tensor, torch::Tensor> fire_us_fp(torch::Tensor spatial, float alpha,
                                                    float thresh) {
    check_input(spatial, "fire_us_fp", "spatial");
    const int dtype = storage_dtype(spatial, "fire_us_fp");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(spatial.device());
    torch::Tensor x = spatial.contiguous();
    torch::Tensor mem = torch::empty_like(x, at::MemoryFormat::Contiguous);
    torch::Tensor spike = torch::empty_like(x, at::MemoryFormat::Contiguous);
    const Dims d = dims_of(x);
    auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
    check_rc(snnlif_fire_us_fp(x.data_ptr(), mem.data_ptr(), spike.data_ptr(), dtype, d.T, d.N,
                               alpha, thresh, stream.stream()),
             "fire_us_fp");
    return std::make_tuple(mem, spike);
}

torch::Tensor fire_bp(torch::Tensor spatial, torch::Tensor grad_spike, float alpha, float thresh,
                      float beta, float interval) {
    check_input(spatial, "fire_bp", "spatial");
    check_input(grad_spike, "fire_bp", "grad_spike");
    TORCH_CHECK(spatial.sizes() == grad_spike.sizes(), "snnlib.fire_bp: spatial ", spatial.sizes(),
                " and grad_spike ", grad_spike.sizes(), " must have the same shape");
    TORCH_CHECK(spatial.scalar_type() == grad_spike.scalar_type(), "snnlib.fire_bp: spatial (",
                spatial.scalar_type(), ") and grad_spike (", grad_spike.scalar_type(),
                ") must have the same dtype");
    TORCH_CHECK(spatial.device() == grad_spike.device(), "snnlib.fire_bp: spatial (",
                spatial.device(), ") and grad_spike (", grad_spike.device(),
                ") must be on the same device");
    const int dtype = storage_dtype(spatial, "fire_bp");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(spatial.device());
    torch::Tensor x = spatial.contiguous();
    torch::Tensor g = grad_spike.contiguous();
    torch::Tensor grad_spatial = torch::empty_like(x, at::MemoryFormat::Contiguous);
    const Dims d = dims_of(x);

    // Windows longer than SNNLIF_BP_FUSED_MAX_T stage the recomputed membrane potential in a
    // workspace from the caching allocator; it is released back to the allocator on return and
    // stays valid for the work already queued because later users are ordered on the same stream.
    const size_t ws_bytes = snnlif_fire_bp_workspace_bytes(dtype, d.T, d.N);
    torch::Tensor workspace;
    void* ws_ptr = nullptr;
    if (ws_bytes > 0) {
        workspace = torch::empty({static_cast<int64_t>(ws_bytes)},
                                 x.options().dtype(at::kByte));
        ws_ptr = workspace.data_ptr();
    }
    auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
    check_rc(snnlif_fire_bp(x.data_ptr(), g.data_ptr(), grad_spatial.data_ptr(), dtype, d.T, d.N,
                            alpha, thresh, beta, interval, ws_ptr, ws_bytes, stream.stream()),
             "fire_bp");
    return grad_spatial;
}

// ---- fire followed by a fully connected layer ---------------------------------------------------

// [T, B, ...] -> [T*B, prod(...)]
torch::Tensor fold_time_flat(const torch::Tensor& t) {
    return t.reshape({t.size(0) * t.size(1), -1});
}

void check_param(const torch::Tensor& p, const torch::Tensor& like, const char* op, const char* name) {
    TORCH_CHECK(p.defined(), "snnlib.", op, ": ", name, " is undefined");
    TORCH_CHECK(p.device() == like.device(), "snnlib.", op, ": ", name, " (", p.device(),
                ") must be on the device of spatial (", like.device(), ")");
    TORCH_CHECK(p.scalar_type() == like.scalar_type(), "snnlib.", op, ": ", name, " (",
                p.scalar_type(), ") must have the dtype of spatial (", like.scalar_type(), ")");
}

torch::Tensor fire_fc_fp(torch::Tensor spatial, torch::Tensor weight_fc, torch::Tensor bias_fc,
                         float alpha, float thresh) {
    check_input(spatial, "fire_fc_fp", "spatial");
    check_param(weight_fc, spatial, "fire_fc_fp", "weight_fc");
    check_param(bias_fc, spatial, "fire_fc_fp", "bias_fc");
    TORCH_CHECK(weight_fc.dim() == 2, "snnlib.fire_fc_fp: weight_fc must be [cout, cin]");
    const int64_t T = spatial.size(0), B = spatial.size(1);
    const int64_t cin = (T * B) ? spatial.numel() / (T * B) : weight_fc.size(1);
    TORCH_CHECK(weight_fc.size(1) == cin, "snnlib.fire_fc_fp: weight_fc expects ", weight_fc.size(1),
                " inputs per sample, spatial has ", cin);
    torch::Tensor spike = fire_s_fp(spatial, alpha, thresh);
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(spatial.device());
    torch::Tensor fc = at::linear(fold_time_flat(spike), weight_fc, bias_fc);
    return fc.view({T, B, weight_fc.size(0)});
}

std::vector<torch::Tensor> fire_fc_bp(torch::Tensor spatial, torch::Tensor grad_fc,
                                      torch::Tensor weight_fc, torch::Tensor bias_fc,
                                      std::vector<int64_t> dim_fc, float alpha, float thresh,
                                      float beta, float interval) {
    check_input(spatial, "fire_fc_bp", "spatial");
    check_param(weight_fc, spatial, "fire_fc_bp", "weight_fc");
    check_param(grad_fc, spatial, "fire_fc_bp", "grad_fc");
    const int64_t T = spatial.size(0), B = spatial.size(1);
    TORCH_CHECK(grad_fc.dim() == 3 && grad_fc.size(0) == T && grad_fc.size(1) == B &&
                    grad_fc.size(2) == weight_fc.size(0),
                "snnlib.fire_fc_bp: grad_fc must be [T, B, cout] = [", T, ", ", B, ", ",
                weight_fc.size(0), "], got ", grad_fc.sizes());
    (void)bias_fc;  // kept for signature parity; the bias gradient needs only grad_fc
    // recompute the spikes (only the input current is saved between forward and backward)
    torch::Tensor spike = fire_s_fp(spatial, alpha, thresh);
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(spatial.device());
    torch::Tensor g2 = fold_time_flat(grad_fc.contiguous());           // [T*B, cout]
    torch::Tensor grad_spike = at::mm(g2, weight_fc).view(spatial.sizes());
    torch::Tensor grad_weight = at::mm(g2.t(), fold_time_flat(spike));  // [cout, cin]
    torch::Tensor grad_bias = at::sum(grad_fc, dim_fc);
    torch::Tensor grad_spatial = fire_bp(spatial, grad_spike, alpha, thresh, beta, interval);
    return {grad_spatial, grad_weight, grad_bias};
}

// ---- fire followed by a 2-d convolution ---------------------------------------------------------

// [T, B, C, H, W] -> [T*B, C, H, W]
torch::Tensor fold_time_image(const torch::Tensor& t) {
    return t.reshape({t.size(0) * t.size(1), t.size(2), t.size(3), t.size(4)});
}

torch::Tensor fire_conv_fp(torch::Tensor spatial, torch::Tensor weight_conv,
                           torch::Tensor bias_conv, std::vector<int64_t> stride,
                           std::vector<int64_t> padding, std::vector<int64_t> dilation,
                           int64_t groups, bool benchmark, bool deterministic, float alpha,
                           float thresh) {
    // `benchmark` / `deterministic` select cuDNN behaviour in the reference; on ROCm the
    // convolution algorithm is MIOpen's choice under torch.backends.cudnn.{benchmark,deterministic}.
    (void)benchmark;
    (void)deterministic;
    check_input(spatial, "fire_conv_fp", "spatial");
    TORCH_CHECK(spatial.dim() == 5, "snnlib.fire_conv_fp: spatial must be [T, B, C, H, W]");
    check_param(weight_conv, spatial, "fire_conv_fp", "weight_conv");
    check_param(bias_conv, spatial, "fire_conv_fp", "bias_conv");
    const int64_t T = spatial.size(0), B = spatial.size(1);
    torch::Tensor spike = fire_s_fp(spatial, alpha, thresh);
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(spatial.device());
    torch::Tensor conv = at::convolution(fold_time_image(spike), weight_conv, bias_conv, stride,
                                         padding, dilation, /*transposed=*/false,
                                         /*output_padding=*/{0, 0}, groups);
    return conv.view({T, B, conv.size(1), conv.size(2), conv.size(3)});
}

std::vector<torch::Tensor> fire_conv_bp(torch::Tensor spatial, torch::Tensor grad_conv,
                                        torch::Tensor weight_conv, std::vector<int64_t> stride,
                                        std::vector<int64_t> padding,
                                        std::vector<int64_t> dilation, int64_t groups,
                                        bool benchmark, bool deterministic, bool allow_tf32,
                                        std::vector<int64_t> dim_conv, float alpha, float thresh,
                                        float beta, float interval) {
    (void)benchmark;
    (void)deterministic;
    (void)allow_tf32;
    check_input(spatial, "fire_conv_bp", "spatial");
    TORCH_CHECK(spatial.dim() == 5, "snnlib.fire_conv_bp: spatial must be [T, B, C, H, W]");
    check_param(weight_conv, spatial, "fire_conv_bp", "weight_conv");
    check_param(grad_conv, spatial, "fire_conv_bp", "grad_conv");
    TORCH_CHECK(grad_conv.dim() == 5 && grad_conv.size(0) == spatial.size(0) &&
                    grad_conv.size(1) == spatial.size(1) && grad_conv.size(2) == weight_conv.size(0),
                "snnlib.fire_conv_bp: grad_conv must be [T, B, cout, Hout, Wout], got ",
                grad_conv.sizes());
    torch::Tensor spike = fire_s_fp(spatial, alpha, thresh);
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(spatial.device());
    auto grads = at::convolution_backward(
        fold_time_image(grad_conv.contiguous()), fold_time_image(spike), weight_conv,
        /*bias_sizes=*/c10::nullopt, stride, padding, dilation, /*transposed=*/false,
        /*output_padding=*/{0, 0}, groups, /*output_mask=*/{true, true, false});
    torch::Tensor grad_spike = std::get<0>(grads).view(spatial.sizes());
    torch::Tensor grad_weight = std::get<1>(grads);
    torch::Tensor grad_bias = at::sum(grad_conv, dim_conv);
    torch::Tensor grad_spatial = fire_bp(spatial, grad_spike, alpha, thresh, beta, interval);
    return {grad_spatial, grad_weight, grad_bias};
}

// ---- batch norm folded into the fire recurrence -------------------------------------------------

struct BnDims {
    int64_t T, B, C, HW;
};

BnDims bn_dims_of(const torch::Tensor& t, const char* op) {
    TORCH_CHECK(t.dim() >= 3, "snnlib.", op, ": spatial must be shaped [T, B, C, ...]");
    const int64_t T = t.size(0), B = t.size(1), C = t.size(2);
    const int64_t tbc = T * B * C;
    return BnDims{T, B, C, tbc ? t.numel() / tbc : 0};
}

torch::Tensor channel_param(const torch::Tensor& p, const torch::Tensor& like, int64_t C,
                            const char* op, const char* name) {
    check_param(p, like, op, name);
    TORCH_CHECK(p.numel() == C, "snnlib.", op, ": ", name, " must have one value per channel (", C,
                "), got ", p.sizes());
    return p.contiguous();
}

std::vector<torch::Tensor> bn_fire_s_fp(torch::Tensor spatial, torch::Tensor weight_bn,
                                        torch::Tensor bias_bn, torch::Tensor var,
                                        torch::Tensor mean, float eps_bn, float alpha,
                                        float thresh) {
    check_input(spatial, "bn_fire_s_fp", "spatial");
    TORCH_CHECK(spatial.scalar_type() == at::kFloat,
                "snnlib.bn_fire_s_fp: only float32 is supported, got ", spatial.scalar_type());
    const BnDims d = bn_dims_of(spatial, "bn_fire_s_fp");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(spatial.device());
    torch::Tensor x = spatial.contiguous();
    torch::Tensor w = channel_param(weight_bn, x, d.C, "bn_fire_s_fp", "weight_bn");
    torch::Tensor b = channel_param(bias_bn, x, d.C, "bn_fire_s_fp", "bias_bn");
    torch::Tensor v = channel_param(var, x, d.C, "bn_fire_s_fp", "var");
    torch::Tensor m = channel_param(mean, x, d.C, "bn_fire_s_fp", "mean");
    torch::Tensor ivar = torch::empty_like(v, at::MemoryFormat::Contiguous);
    torch::Tensor spike = torch::empty_like(x, at::MemoryFormat::Contiguous);
    auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
    check_rc(snnlif_bn_fire_s_fp(x.data_ptr(), w.data_ptr(), b.data_ptr(), v.data_ptr(),
                                 m.data_ptr(), ivar.data_ptr(), spike.data_ptr(), SNNLIF_DTYPE_F32,
                                 d.T, d.B, d.C, d.HW, eps_bn, alpha, thresh, stream.stream()),
             "bn_fire_s_fp");
    return {ivar, spike};
}

std::vector<torch::Tensor> bn_fire_bp(torch::Tensor spatial, torch::Tensor weight_bn,
                                      torch::Tensor bias_bn, torch::Tensor ivar, torch::Tensor mean,
                                      std::vector<int64_t> dim_bn, torch::Tensor grad_spike,
                                      float alpha, float thresh, float beta, float interval) {
    // dim_bn names the reduced axes ((0,1) or (0,1,3,4)); they follow from the shape here
    (void)dim_bn;
    check_input(spatial, "bn_fire_bp", "spatial");
    check_input(grad_spike, "bn_fire_bp", "grad_spike");
    TORCH_CHECK(spatial.scalar_type() == at::kFloat,
                "snnlib.bn_fire_bp: only float32 is supported, got ", spatial.scalar_type());
    TORCH_CHECK(spatial.sizes() == grad_spike.sizes() &&
                    spatial.scalar_type() == grad_spike.scalar_type() &&
                    spatial.device() == grad_spike.device(),
                "snnlib.bn_fire_bp: spatial and grad_spike must agree in shape, dtype and device");
    const BnDims d = bn_dims_of(spatial, "bn_fire_bp");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(spatial.device());
    torch::Tensor x = spatial.contiguous();
    torch::Tensor g = grad_spike.contiguous();
    torch::Tensor w = channel_param(weight_bn, x, d.C, "bn_fire_bp", "weight_bn");
    torch::Tensor b = channel_param(bias_bn, x, d.C, "bn_fire_bp", "bias_bn");
    torch::Tensor iv = channel_param(ivar, x, d.C, "bn_fire_bp", "ivar");
    torch::Tensor m = channel_param(mean, x, d.C, "bn_fire_bp", "mean");
    torch::Tensor grad_spatial = torch::empty_like(x, at::MemoryFormat::Contiguous);
    torch::Tensor grad_weight = torch::empty_like(w, at::MemoryFormat::Contiguous);
    torch::Tensor grad_bias = torch::empty_like(w, at::MemoryFormat::Contiguous);
    const size_t ws_bytes = snnlif_bn_fire_bp_workspace_bytes(SNNLIF_DTYPE_F32, d.T, d.B, d.C, d.HW);
    torch::Tensor workspace = torch::empty({static_cast<int64_t>(ws_bytes)}, x.options().dtype(at::kByte));
    auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
    check_rc(snnlif_bn_fire_bp(x.data_ptr(), w.data_ptr(), b.data_ptr(), iv.data_ptr(), m.data_ptr(),
                               g.data_ptr(), grad_spatial.data_ptr(), grad_weight.data_ptr(),
                               grad_bias.data_ptr(), SNNLIF_DTYPE_F32, d.T, d.B, d.C, d.HW, alpha,
                               thresh, beta, interval, ws_bytes ? workspace.data_ptr() : nullptr,
                               ws_bytes, stream.stream()),
             "bn_fire_bp");
    return {grad_spatial, grad_weight.view_as(weight_bn), grad_bias.view_as(weight_bn)};
}


// ---- shared dense halves (ATen: rocBLAS / MIOpen), time folded into the batch -------------------

torch::Tensor linear_folded(const torch::Tensor& in, const torch::Tensor& weight,
                            const torch::Tensor& bias) {
    const int64_t T = in.size(0), B = in.size(1);
    return at::linear(fold_time_flat(in), weight, bias).view({T, B, weight.size(0)});
}

// -> {grad_in (shaped like `in`), grad_weight, grad_bias}
std::vector<torch::Tensor> linear_backward_folded(const torch::Tensor& in,
                                                  const torch::Tensor& grad_fc,
                                                  const torch::Tensor& weight,
                                                  const std::vector<int64_t>& dim_fc) {
    torch::Tensor g2 = fold_time_flat(grad_fc.contiguous());
    torch::Tensor grad_in = at::mm(g2, weight).view(in.sizes());
    torch::Tensor grad_weight = at::mm(g2.t(), fold_time_flat(in));
    return {grad_in, grad_weight, at::sum(grad_fc, dim_fc)};
}

torch::Tensor conv_folded(const torch::Tensor& in, const torch::Tensor& weight,
                          const torch::Tensor& bias, const std::vector<int64_t>& stride,
                          const std::vector<int64_t>& padding, const std::vector<int64_t>& dilation,
                          int64_t groups) {
    const int64_t T = in.size(0), B = in.size(1);
    torch::Tensor conv = at::convolution(fold_time_image(in), weight, bias, stride, padding,
                                         dilation, /*transposed=*/false, /*output_padding=*/{0, 0},
                                         groups);
    return conv.view({T, B, conv.size(1), conv.size(2), conv.size(3)});
}

// -> {grad_in (shaped like `in`), grad_weight, grad_bias}
std::vector<torch::Tensor> conv_backward_folded(const torch::Tensor& in,
                                                const torch::Tensor& grad_conv,
                                                const torch::Tensor& weight,
                                                const std::vector<int64_t>& stride,
                                                const std::vector<int64_t>& padding,
                                                const std::vector<int64_t>& dilation,
                                                int64_t groups,
                                                const std::vector<int64_t>& dim_conv) {
    auto grads = at::convolution_backward(
        fold_time_image(grad_conv.contiguous()), fold_time_image(in), weight,
        /*bias_sizes=*/c10::nullopt, stride, padding, dilation, /*transposed=*/false,
        /*output_padding=*/{0, 0}, groups, /*output_mask=*/{true, true, false});
    return {std::get<0>(grads).view(in.sizes()), std::get<1>(grads), at::sum(grad_conv, dim_conv)};
}

void check_fc_shapes(const torch::Tensor& spatial, const torch::Tensor& weight_fc, const char* op) {
    TORCH_CHECK(weight_fc.dim() == 2, "snnlib.", op, ": weight_fc must be [cout, cin]");
    const int64_t tb = spatial.size(0) * spatial.size(1);
    const int64_t cin = tb ? spatial.numel() / tb : weight_fc.size(1);
    TORCH_CHECK(weight_fc.size(1) == cin, "snnlib.", op, ": weight_fc expects ", weight_fc.size(1),
                " inputs per sample, spatial has ", cin);
}

// Spikes of the bn + fire layer from the statistics saved by its forward (backward-side scale).
torch::Tensor bn_fire_spikes_from_ivar(const torch::Tensor& spatial, const torch::Tensor& weight_bn,
                                       const torch::Tensor& bias_bn, const torch::Tensor& ivar,
                                       const torch::Tensor& mean, float alpha, float thresh,
                                       const char* op) {
    check_input(spatial, op, "spatial");
    TORCH_CHECK(spatial.scalar_type() == at::kFloat, "snnlib.", op,
                ": only float32 is supported, got ", spatial.scalar_type());
    const BnDims d = bn_dims_of(spatial, op);
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(spatial.device());
    torch::Tensor x = spatial.contiguous();
    torch::Tensor w = channel_param(weight_bn, x, d.C, op, "weight_bn");
    torch::Tensor b = channel_param(bias_bn, x, d.C, op, "bias_bn");
    torch::Tensor iv = channel_param(ivar, x, d.C, op, "ivar");
    torch::Tensor m = channel_param(mean, x, d.C, op, "mean");
    torch::Tensor spike = torch::empty_like(x, at::MemoryFormat::Contiguous);
    auto stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
    check_rc(snnlif_bn_fire_s_recompute(x.data_ptr(), w.data_ptr(), b.data_ptr(), iv.data_ptr(),
                                        m.data_ptr(), spike.data_ptr(), SNNLIF_DTYPE_F32, d.T, d.B,
                                        d.C, d.HW, alpha, thresh, stream.stream()),
             op);
    return spike;
}

// ---- plain batch norm with given statistics (ATen) ------------------------------------------------

// [T, B, C, ...] -> [T*B, C, ...]
torch::Tensor fold_time(const torch::Tensor& t) {
    std::vector<int64_t> sizes = {t.size(0) * t.size(1)};
    for (int64_t i = 2; i < t.dim(); ++i) sizes.push_back(t.size(i));
    return t.reshape(sizes);
}

std::vector<torch::Tensor> bn_fp(torch::Tensor x_bn, torch::Tensor weight_bn, torch::Tensor bias_bn,
                                 torch::Tensor var, torch::Tensor mean, float eps_bn) {
    check_input(x_bn, "bn_fp", "x_bn");
    const BnDims d = bn_dims_of(x_bn, "bn_fp");
    for (const auto* p : {&weight_bn, &bias_bn, &var, &mean}) channel_param(*p, x_bn, d.C, "bn_fp", "parameter");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(x_bn.device());
    // y = (x - mean) * weight / sqrt(var + eps) + bias with the statistics the caller supplies
    torch::Tensor y = at::batch_norm(fold_time(x_bn), weight_bn, bias_bn, mean.detach(), var.detach(),
                                     /*training=*/false, /*momentum=*/0.0, eps_bn,
                                     /*cudnn_enabled=*/true);
    torch::Tensor ivar = at::rsqrt(var.detach() + eps_bn);
    return {ivar, y.view(x_bn.sizes())};
}

std::vector<torch::Tensor> bn_bp(torch::Tensor x_bn, torch::Tensor weight_bn, torch::Tensor bias_bn,
                                 torch::Tensor ivar, torch::Tensor mean, std::vector<int64_t> dim_bn,
                                 torch::Tensor grad_y_bn) {
    (void)bias_bn;
    (void)dim_bn;
    check_input(x_bn, "bn_bp", "x_bn");
    check_param(grad_y_bn, x_bn, "bn_bp", "grad_y_bn");
    TORCH_CHECK(grad_y_bn.sizes() == x_bn.sizes(), "snnlib.bn_bp: grad_y_bn must have the shape of x_bn");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(x_bn.device());
    // training-mode batch-norm backward with the saved batch statistics
    auto grads = at::native_batch_norm_backward(
        fold_time(grad_y_bn.contiguous()), fold_time(x_bn.contiguous()), weight_bn,
        /*running_mean=*/c10::nullopt, /*running_var=*/c10::nullopt, /*save_mean=*/mean,
        /*save_invstd=*/ivar, /*train=*/true, /*eps=*/0.0, {true, true, true});
    return {std::get<0>(grads).view(x_bn.sizes()), std::get<1>(grads), std::get<2>(grads)};
}

// ---- fully connected / convolution without fire -------------------------------------------------

torch::Tensor fc_fp(torch::Tensor spatial, torch::Tensor weight_fc, torch::Tensor bias_fc) {
    check_input(spatial, "fc_fp", "spatial");
    check_param(weight_fc, spatial, "fc_fp", "weight_fc");
    check_param(bias_fc, spatial, "fc_fp", "bias_fc");
    check_fc_shapes(spatial, weight_fc, "fc_fp");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(spatial.device());
    return linear_folded(spatial, weight_fc, bias_fc);
}

std::vector<torch::Tensor> fc_bp(torch::Tensor spatial, torch::Tensor grad_fc,
                                 torch::Tensor weight_fc, torch::Tensor bias_fc,
                                 std::vector<int64_t> dim_fc) {
    (void)bias_fc;
    check_input(spatial, "fc_bp", "spatial");
    check_param(weight_fc, spatial, "fc_bp", "weight_fc");
    check_param(grad_fc, spatial, "fc_bp", "grad_fc");
    check_fc_shapes(spatial, weight_fc, "fc_bp");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(spatial.device());
    return linear_backward_folded(spatial, grad_fc, weight_fc, dim_fc);
}

torch::Tensor conv_fp(torch::Tensor spatial, torch::Tensor weight_conv, torch::Tensor bias_conv,
                      std::vector<int64_t> stride, std::vector<int64_t> padding,
                      std::vector<int64_t> dilation, int64_t groups, bool benchmark,
                      bool deterministic) {
    (void)benchmark;
    (void)deterministic;
    check_input(spatial, "conv_fp", "spatial");
    TORCH_CHECK(spatial.dim() == 5, "snnlib.conv_fp: spatial must be [T, B, C, H, W]");
    check_param(weight_conv, spatial, "conv_fp", "weight_conv");
    check_param(bias_conv, spatial, "conv_fp", "bias_conv");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(spatial.device());
    return conv_folded(spatial, weight_conv, bias_conv, stride, padding, dilation, groups);
}

std::vector<torch::Tensor> conv_bp(torch::Tensor spatial, torch::Tensor grad_conv,
                                   torch::Tensor weight_conv, std::vector<int64_t> stride,
                                   std::vector<int64_t> padding, std::vector<int64_t> dilation,
                                   int64_t groups, bool benchmark, bool deterministic,
                                   bool allow_tf32, std::vector<int64_t> dim_conv) {
    (void)benchmark;
    (void)deterministic;
    (void)allow_tf32;
    check_input(spatial, "conv_bp", "spatial");
    TORCH_CHECK(spatial.dim() == 5, "snnlib.conv_bp: spatial must be [T, B, C, H, W]");
    check_param(weight_conv, spatial, "conv_bp", "weight_conv");
    check_param(grad_conv, spatial, "conv_bp", "grad_conv");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(spatial.device());
    return conv_backward_folded(spatial, grad_conv, weight_conv, stride, padding, dilation, groups,
                                dim_conv);
}

// ---- batch norm + fire followed by a fully connected layer / a convolution ------------------------

std::vector<torch::Tensor> bn_fire_fc_fp(torch::Tensor spatial, torch::Tensor weight_bn,
                                         torch::Tensor bias_bn, torch::Tensor var,
                                         torch::Tensor mean, float eps_bn, torch::Tensor weight_fc,
                                         torch::Tensor bias_fc, float alpha, float thresh) {
    check_input(spatial, "bn_fire_fc_fp", "spatial");
    check_param(weight_fc, spatial, "bn_fire_fc_fp", "weight_fc");
    check_param(bias_fc, spatial, "bn_fire_fc_fp", "bias_fc");
    check_fc_shapes(spatial, weight_fc, "bn_fire_fc_fp");
    auto fired = bn_fire_s_fp(spatial, weight_bn, bias_bn, var, mean, eps_bn, alpha, thresh);
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(spatial.device());
    return {fired[0], linear_folded(fired[1], weight_fc, bias_fc)};
}

std::vector<torch::Tensor> bn_fire_fc_bp(torch::Tensor spatial, torch::Tensor weight_bn,
                                         torch::Tensor bias_bn, torch::Tensor ivar,
                                         torch::Tensor mean, std::vector<int64_t> dim_bn,
                                         torch::Tensor grad_fc, torch::Tensor weight_fc,
                                         torch::Tensor bias_fc, std::vector<int64_t> dim_fc,
                                         float alpha, float thresh, float beta, float interval) {
    (void)bias_fc;
    check_param(weight_fc, spatial, "bn_fire_fc_bp", "weight_fc");
    check_param(grad_fc, spatial, "bn_fire_fc_bp", "grad_fc");
    check_fc_shapes(spatial, weight_fc, "bn_fire_fc_bp");
    torch::Tensor spike = bn_fire_spikes_from_ivar(spatial, weight_bn, bias_bn, ivar, mean, alpha,
                                                   thresh, "bn_fire_fc_bp");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(spatial.device());
    auto dense = linear_backward_folded(spike, grad_fc, weight_fc, dim_fc);
    auto bn = bn_fire_bp(spatial, weight_bn, bias_bn, ivar, mean, dim_bn, dense[0], alpha, thresh,
                         beta, interval);
    return {bn[0], bn[1], bn[2], dense[1], dense[2]};
}

std::vector<torch::Tensor> bn_fire_conv_fp(torch::Tensor spatial, torch::Tensor weight_bn,
                                           torch::Tensor bias_bn, torch::Tensor var,
                                           torch::Tensor mean, float eps_bn,
                                           torch::Tensor weight_conv, torch::Tensor bias_conv,
                                           std::vector<int64_t> stride,
                                           std::vector<int64_t> padding,
                                           std::vector<int64_t> dilation, int64_t groups,
                                           bool benchmark, bool deterministic, float alpha,
                                           float thresh) {
    (void)benchmark;
    (void)deterministic;
    check_input(spatial, "bn_fire_conv_fp", "spatial");
    TORCH_CHECK(spatial.dim() == 5, "snnlib.bn_fire_conv_fp: spatial must be [T, B, C, H, W]");
    check_param(weight_conv, spatial, "bn_fire_conv_fp", "weight_conv");
    check_param(bias_conv, spatial, "bn_fire_conv_fp", "bias_conv");
    auto fired = bn_fire_s_fp(spatial, weight_bn, bias_bn, var, mean, eps_bn, alpha, thresh);
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(spatial.device());
    return {fired[0], conv_folded(fired[1], weight_conv, bias_conv, stride, padding, dilation, groups)};
}

std::vector<torch::Tensor> bn_fire_conv_bp(torch::Tensor spatial, torch::Tensor weight_bn,
                                           torch::Tensor bias_bn, torch::Tensor ivar,
                                           torch::Tensor mean, std::vector<int64_t> dim_bn,
                                           torch::Tensor grad_conv, torch::Tensor weight_conv,
                                           std::vector<int64_t> stride,
                                           std::vector<int64_t> padding,
                                           std::vector<int64_t> dilation, int64_t groups,
                                           bool benchmark, bool deterministic, bool allow_tf32,
                                           std::vector<int64_t> dim_conv, float alpha, float thresh,
                                           float beta, float interval) {
    (void)benchmark;
    (void)deterministic;
    (void)allow_tf32;
    TORCH_CHECK(spatial.dim() == 5, "snnlib.bn_fire_conv_bp: spatial must be [T, B, C, H, W]");
    check_param(weight_conv, spatial, "bn_fire_conv_bp", "weight_conv");
    check_param(grad_conv, spatial, "bn_fire_conv_bp", "grad_conv");
    torch::Tensor spike = bn_fire_spikes_from_ivar(spatial, weight_bn, bias_bn, ivar, mean, alpha,
                                                   thresh, "bn_fire_conv_bp");
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(spatial.device());
    auto dense = conv_backward_folded(spike, grad_conv, weight_conv, stride, padding, dilation,
                                      groups, dim_conv);
    auto bn = bn_fire_bp(spatial, weight_bn, bias_bn, ivar, mean, dim_bn, dense[0], alpha, thresh,
                         beta, interval);
    return {bn[0], bn[1], bn[2], dense[1], dense[2]};
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "snnlib LIF fire operators for MI355X (gfx950)";
    m.attr("__backend__") = "hip-gfx950";
    m.attr("__abi_version__") = snnlif_abi_version();
    m.def("fire_s_fp", &fire_s_fp, "fire (spike) forward");
    m.def("fire_us_fp", &fire_us_fp, "fire (membrane potential, spike) forward");
    m.def("fire_bp", &fire_bp, "fire backward");
    m.def("bn_fire_s_fp", &bn_fire_s_fp, "bn fire (spike) forward");
    m.def("bn_fire_bp", &bn_fire_bp, "bn fire backward");
    m.def("bn_fp", &bn_fp, "bn forward");
    m.def("bn_bp", &bn_bp, "bn backward");
    m.def("bn_fire_fc_fp", &bn_fire_fc_fp, "bn fire fc forward");
    m.def("bn_fire_fc_bp", &bn_fire_fc_bp, "bn fire fc backward");
    m.def("fc_fp", &fc_fp, "fc forward");
    m.def("fc_bp", &fc_bp, "fc backward");
    m.def("bn_fire_conv_fp", &bn_fire_conv_fp, "bn fire conv forward");
    m.def("bn_fire_conv_bp", &bn_fire_conv_bp, "bn fire conv backward");
    m.def("conv_fp", &conv_fp, "conv forward");
    m.def("conv_bp", &conv_bp, "conv backward");
    m.def("fire_fc_fp", &fire_fc_fp, "fire fc forward");
    m.def("fire_fc_bp", &fire_fc_bp, "fire fc backward");
    m.def("fire_conv_fp", &fire_conv_fp, "fire conv forward");
    m.def("fire_conv_bp", &fire_conv_bp, "fire conv backward");
}
