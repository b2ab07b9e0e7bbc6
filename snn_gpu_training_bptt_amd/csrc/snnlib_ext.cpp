// Python extension module `snnlib` for PyTorch-ROCm: the operator boundary the autograd functions
// of snnlib_func.py call (reference: snnlib/example/snnlib_func.py:22-253).
//
// Every entry of the reference's binding table (snnlib/cuda/snn.cpp:798-829) is provided with the
// same name and positional signature:
//
//   fire_s_fp(spatial, alpha, thresh) -> spike                                      snn.cpp:11-17
//   fire_bp(spatial, grad_spike, alpha, thresh, beta, interval) -> grad_spatial     snn.cpp:270-279
//   bn_fire_s_fp(spatial, weight_bn, bias_bn, var, mean, eps_bn, alpha, thresh) -> [ivar, spike]
//                                                                                   snn.cpp:55-66
//   bn_fire_bp(spatial, weight_bn, bias_bn, ivar, mean, dim_bn, grad_spike, alpha, thresh, beta,
//              interval) -> [grad_spatial, grad_weight_bn, grad_bias_bn]            snn.cpp:373-388
//   bn_fp / bn_bp                                                                   snn.cpp:30-40, 293-304
//   fc_fp / fc_bp, conv_fp / conv_bp                                                snn.cpp:130-137, 594-603, 239-253, 779-795
//   fire_fc_fp / fire_fc_bp, fire_conv_fp / fire_conv_bp                            snn.cpp:112-120, 569-582, 206-223, 740-761
//   bn_fire_fc_fp / bn_fire_fc_bp, bn_fire_conv_fp / bn_fire_conv_bp                snn.cpp:85-101, 484-506, 162-188, 630-660
//
// plus fire_us_fp(spatial, alpha, thresh) -> (mem, spike), the public face of the reference's
// internal fire_us_fp_kernel (snnlib/cuda/snn_kernel_bp.cu:54-93), bn_stats(spatial) -> [var, mean] and
// bn_moments(spatial) -> [E[x], E[x^2]], the batch statistics the reference's layers take from
// torch.var_mean / torch.mean (snnlib/example/snnlib_op.py:78, 263-264), and the halves that a batch sharded
// over several GPUs runs on either side of its all-reduce (the all-reduce itself is the caller's):
//
//   bn_bp_dist1 / bn_bp_dist2                                                       snn.cpp:317-355
//   bn_fire_bp_dist1 / bn_fire_bp_dist2                                             snn.cpp:405-460
//   bn_fire_fc_bp_dist1, bn_fire_conv_bp_dist1                                      snn.cpp:528-550, 687-716
//
// Division of labour: the fire recurrences (with or without the batch norm folded in) run on the
// hand-written kernels behind the C ABI of libsnnlif_gfx950.so (include/snnlib_lif.h), and so does the
// plain batch norm; linear and convolution stay on PyTorch-ROCm (rocBLAS / MIOpen through ATen) and are
// issued once with the time axis folded into the batch, not once per time step as the reference's
// host loops do (snnlib/cuda/snn_kernel_fp.cu:314-326, 444-447; snnlib/cuda/snn_kernel_bp.cu:1099-1117,
// 1382-1390).  As in the reference, backward ops receive only what the forward saved (inputs and
// batch statistics) and recompute spikes themselves.
//
// This file validates tensors, allocates outputs and forwards raw device pointers; it holds no
// device code and no fallback.  Unlike the reference launchers (snnlib/cuda/snn_kernel_fp.cu:55-73: no
// checks, legacy default stream, no device guard) it checks device / dtype / shape, makes inputs
// dense, switches to the tensor's device and launches on PyTorch's current stream for that device.

#include <torch/extension.h>

#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <tuple>
#include <vector>

#include "snnlib_lif.h"

namespace {

using torch::Tensor;
using IntList = std::vector<int64_t>;
using DeviceGuard = c10::hip::HIPGuardMasqueradingAsCUDA;

// ---- checks -------------------------------------------------------------------------------------

int storage_dtype(const Tensor& t, const char* op) {
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

// A [T, B, ...] activation on a ROCm device.
void check_input(const Tensor& t, const char* op, const char* name) {
    TORCH_CHECK(t.defined(), "snnlib.", op, ": ", name, " is undefined");
    TORCH_CHECK(t.is_cuda(), "snnlib.", op, ": ", name,
                " must live on a ROCm GPU (this build has no CPU path), got device ", t.device());
    TORCH_CHECK(t.dim() >= 2, "snnlib.", op, ": ", name,
                " must be shaped [T, B, ...], got ", t.dim(), " dimension(s)");
    TORCH_CHECK(!t.is_complex(), "snnlib.", op, ": complex tensors are not supported");
}

// A parameter or gradient that must share device and dtype with the activation.
void check_like(const Tensor& p, const Tensor& like, const char* op, const char* name) {
    TORCH_CHECK(p.defined(), "snnlib.", op, ": ", name, " is undefined");
    TORCH_CHECK(p.device() == like.device(), "snnlib.", op, ": ", name, " (", p.device(),
                ") must be on the device of spatial (", like.device(), ")");
    TORCH_CHECK(p.scalar_type() == like.scalar_type(), "snnlib.", op, ": ", name, " (",
                p.scalar_type(), ") must have the dtype of spatial (", like.scalar_type(), ")");
}

void check_same_shape(const Tensor& a, const Tensor& b, const char* op, const char* an,
                      const char* bn) {
    TORCH_CHECK(a.sizes() == b.sizes(), "snnlib.", op, ": ", an, " ", a.sizes(), " and ", bn, " ",
                b.sizes(), " must have the same shape");
}

void check_image(const Tensor& t, const char* op) {
    TORCH_CHECK(t.dim() == 5, "snnlib.", op, ": spatial must be [T, B, C, H, W], got ", t.sizes());
}

void check_fc_weight(const Tensor& spatial, const Tensor& weight_fc, const char* op) {
    TORCH_CHECK(weight_fc.dim() == 2, "snnlib.", op, ": weight_fc must be [cout, cin]");
    const int64_t tb = spatial.size(0) * spatial.size(1);
    const int64_t cin = tb ? spatial.numel() / tb : weight_fc.size(1);
    TORCH_CHECK(weight_fc.size(1) == cin, "snnlib.", op, ": weight_fc expects ", weight_fc.size(1),
                " inputs per sample, spatial has ", cin);
}

void check_rc(int rc, const char* op) {
    TORCH_CHECK(rc == SNNLIF_OK, "snnlib.", op, ": ", snnlif_strerror(rc), " (code ", rc, ")");
}

void* current_stream() {
    return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
}

// ---- shapes -------------------------------------------------------------------------------------

struct Dims {  // [T, N]
    int64_t T, N;
};

Dims dims_of(const Tensor& t) {
    const int64_t T = t.size(0);
    return Dims{T, T == 0 ? 0 : t.numel() / T};
}

struct BnDims {  // [T, B, C, HW]
    int64_t T, B, C, HW;
};

BnDims bn_dims_of(const Tensor& t, const char* op) {
    TORCH_CHECK(t.dim() >= 3, "snnlib.", op, ": spatial must be shaped [T, B, C, ...]");
    const int64_t T = t.size(0), B = t.size(1), C = t.size(2);
    const int64_t tbc = T * B * C;
    return BnDims{T, B, C, tbc ? t.numel() / tbc : 0};
}

// A dense per-channel vector of the activation's dtype and device.
Tensor channel_param(const Tensor& p, const Tensor& like, int64_t C, const char* op,
                     const char* name) {
    check_like(p, like, op, name);
    TORCH_CHECK(p.numel() == C, "snnlib.", op, ": ", name, " must have one value per channel (", C,
                "), got ", p.sizes());
    return p.contiguous();
}

// A per-channel result of a backward op.  The kernels write every channel whenever the activation has
// elements; only for an empty activation (which they leave alone) is it filled with zeros: an empty
// local batch contributes nothing to the all-reduce and leaves the parameter gradients untouched.
Tensor channel_result(const Tensor& like, const Tensor& activation) {
    return activation.numel() == 0 ? torch::zeros_like(like, at::MemoryFormat::Contiguous)
                                   : torch::empty_like(like, at::MemoryFormat::Contiguous);
}

// A freshly computed tensor under another shape, handed out as a tensor of its own rather than as
// an autograd view: callers modify layer outputs in place (the residual `x += ...` of
// snnlib/example/models.py:122-125), which autograd forbids on a view made inside a custom Function.
Tensor reshaped_result(const Tensor& t, at::IntArrayRef sizes) {
    return at::_unsafe_view(t, sizes);
}

// [T, B, ...] -> [T*B, ...], [T*B, prod(...)]
Tensor fold_time(const Tensor& t) {
    IntList sizes = {t.size(0) * t.size(1)};
    for (int64_t i = 2; i < t.dim(); ++i) sizes.push_back(t.size(i));
    return t.reshape(sizes);
}

Tensor fold_time_flat(const Tensor& t) {
    return t.reshape({t.size(0) * t.size(1), -1});
}

// ---- dense halves (ATen: rocBLAS / MIOpen), time folded into the batch ---------------------------

Tensor linear_folded(const Tensor& in, const Tensor& weight, const Tensor& bias) {
    return reshaped_result(at::linear(fold_time_flat(in), weight, bias),
                           {in.size(0), in.size(1), weight.size(0)});
}

// -> {grad_in (shaped like `in`), grad_weight, grad_bias}
std::vector<Tensor> linear_backward_folded(const Tensor& in, const Tensor& grad_fc,
                                           const Tensor& weight, const IntList& dim_fc,
                                           const char* op) {
    TORCH_CHECK(grad_fc.dim() == 3 && grad_fc.size(0) == in.size(0) &&
                    grad_fc.size(1) == in.size(1) && grad_fc.size(2) == weight.size(0),
                "snnlib.", op, ": grad_fc must be [T, B, cout] = [", in.size(0), ", ", in.size(1),
                ", ", weight.size(0), "], got ", grad_fc.sizes());
    Tensor g2 = fold_time_flat(grad_fc.contiguous());  // [T*B, cout]
    Tensor grad_in = reshaped_result(at::mm(g2, weight), in.sizes());
    Tensor grad_weight = at::mm(g2.t(), fold_time_flat(in));  // [cout, cin]
    return {grad_in, grad_weight, at::sum(grad_fc, dim_fc)};
}

// The reference hands `benchmark` and `deterministic` to cuDNN with every convolution call
// (snnlib/cuda/snn_kernel_fp.cu:404-407, snnlib/cuda/snn_kernel_bp.cu:1107-1118).  PyTorch-ROCm takes
// them from the process-wide settings (torch.backends.cudnn.benchmark / .deterministic) when it calls
// MIOpen -- benchmark = true lets MIOpen search for the fastest algorithm of a shape the first time it
// sees it, false takes its immediate choice -- so the caller's flags are put there for the duration
// of the dense call and the previous settings restored afterwards.
class ConvSearchGuard {
public:
    ConvSearchGuard(bool benchmark, bool deterministic)
        : benchmark_(at::globalContext().benchmarkCuDNN()),
          deterministic_(at::globalContext().deterministicCuDNN()) {
        at::globalContext().setBenchmarkCuDNN(benchmark);
        at::globalContext().setDeterministicCuDNN(deterministic);
    }
    ~ConvSearchGuard() {
        at::globalContext().setBenchmarkCuDNN(benchmark_);
        at::globalContext().setDeterministicCuDNN(deterministic_);
    }
    ConvSearchGuard(const ConvSearchGuard&) = delete;
    ConvSearchGuard& operator=(const ConvSearchGuard&) = delete;

private:
    bool benchmark_, deterministic_;
};

Tensor conv_folded(const Tensor& in, const Tensor& weight, const Tensor& bias,
                   const IntList& stride, const IntList& padding, const IntList& dilation,
                   int64_t groups, bool benchmark, bool deterministic) {
    const ConvSearchGuard search(benchmark, deterministic);
    Tensor conv = at::convolution(fold_time(in), weight, bias, stride, padding, dilation,
                                  /*transposed=*/false, /*output_padding=*/{0, 0}, groups);
    return reshaped_result(conv, {in.size(0), in.size(1), conv.size(1), conv.size(2), conv.size(3)});
}

// The bias gradient of the layers that end in a convolution: at::sum(grad_conv, dim_conv) in the
// reference (snnlib/cuda/snn_kernel_bp.cu:1261, 1338, 1401, 1435).  For the dim_conv its layers pass --
// every axis but the channel's, (0, 1, 3, 4) -- a dense fp32 / fp64 gradient with planes of at least
// kChannelSumMinPlane positions takes the hand-written per-channel reduction (snnlif_channel_sum, one
// pass at the rate of the batch statistics; the framework's reduction over these axes runs at a
// third of it); any other reduction stays with ATen.
constexpr int64_t kChannelSumMinPlane = 32;

bool all_axes_but_channel(const IntList& dims, int64_t rank) {
    if (rank < 4 || static_cast<int64_t>(dims.size()) != rank - 1) return false;
    std::vector<bool> seen(static_cast<size_t>(rank), false);
    for (int64_t d : dims) {
        if (d < 0) d += rank;
        if (d < 0 || d >= rank || d == 2 || seen[static_cast<size_t>(d)]) return false;
        seen[static_cast<size_t>(d)] = true;
    }
    return true;
}

Tensor bias_gradient(const Tensor& grad, const IntList& dims, const char* op) {
    const bool native_type = grad.scalar_type() == at::kFloat || grad.scalar_type() == at::kDouble;
    if (!grad.is_cuda() || !native_type || !all_axes_but_channel(dims, grad.dim()) ||
        grad.numel() == 0)
        return at::sum(grad, dims);
    const BnDims d = bn_dims_of(grad, op);
    if (d.HW < kChannelSumMinPlane) return at::sum(grad, dims);
    const int dtype = grad.scalar_type() == at::kFloat ? SNNLIF_DTYPE_F32 : SNNLIF_DTYPE_F64;
    const DeviceGuard guard(grad.device());
    Tensor g = grad.contiguous();
    Tensor sum = torch::empty({d.C}, g.options());
    const size_t ws_bytes = snnlif_bn_stats_workspace_bytes(dtype, d.T, d.B, d.C, d.HW);
    Tensor workspace =
        torch::empty({static_cast<int64_t>(ws_bytes)}, g.options().dtype(at::kByte));
    check_rc(snnlif_channel_sum(g.data_ptr(), sum.data_ptr(), dtype, d.T, d.B, d.C, d.HW,
                                ws_bytes ? workspace.data_ptr() : nullptr, ws_bytes,
                                current_stream()),
             op);
    return sum;
}

// -> {grad_in (shaped like `in`), grad_weight, grad_bias}
std::vector<Tensor> conv_backward_folded(const Tensor& in, const Tensor& grad_conv,
                                         const Tensor& weight, const IntList& stride,
                                         const IntList& padding, const IntList& dilation,
                                         int64_t groups, bool benchmark, bool deterministic,
                                         const IntList& dim_conv, const char* op) {
    const ConvSearchGuard search(benchmark, deterministic);
    TORCH_CHECK(grad_conv.dim() == 5 && grad_conv.size(0) == in.size(0) &&
                    grad_conv.size(1) == in.size(1) && grad_conv.size(2) == weight.size(0),
                "snnlib.", op, ": grad_conv must be [T, B, cout, Hout, Wout], got ",
                grad_conv.sizes());
    const Tensor grad_dense = grad_conv.contiguous();
    auto grads = at::convolution_backward(
        fold_time(grad_dense), fold_time(in), weight, /*bias_sizes=*/c10::nullopt,
        stride, padding, dilation, /*transposed=*/false, /*output_padding=*/{0, 0}, groups,
        /*output_mask=*/{true, true, false});
    return {reshaped_result(std::get<0>(grads), in.sizes()), std::get<1>(grads),
            bias_gradient(grad_dense, dim_conv, op)};
}

// ---- fire ---------------------------------------------------------------------------------------

Tensor fire_s_fp(Tensor spatial, float alpha, float thresh) {
    check_input(spatial, "fire_s_fp", "spatial");
    const int dtype = storage_dtype(spatial, "fire_s_fp");
    const DeviceGuard guard(spatial.device());
    Tensor x = spatial.contiguous();
    Tensor spike = torch::empty_like(x, at::MemoryFormat::Contiguous);
    const Dims d = dims_of(x);
    check_rc(snnlif_fire_s_fp(x.data_ptr(), spike.data_ptr(), dtype, d.T, d.N, alpha, thresh,
                              current_stream()),
             "fire_s_fp");
    return spike;
}

std::tuple<Tensor, Tensor> fire_us_fp(Tensor spatial, float alpha, float thresh) {
    check_input(spatial, "fire_us_fp", "spatial");
    const int dtype = storage_dtype(spatial, "fire_us_fp");
    const DeviceGuard guard(spatial.device());
    Tensor x = spatial.contiguous();
    Tensor mem = torch::empty_like(x, at::MemoryFormat::Contiguous);
    Tensor spike = torch::empty_like(x, at::MemoryFormat::Contiguous);
    const Dims d = dims_of(x);
    check_rc(snnlif_fire_us_fp(x.data_ptr(), mem.data_ptr(), spike.data_ptr(), dtype, d.T, d.N,
                               alpha, thresh, current_stream()),
             "fire_us_fp");
    return std::make_tuple(mem, spike);
}

Tensor fire_bp(Tensor spatial, Tensor grad_spike, float alpha, float thresh, float beta,
               float interval) {
    check_input(spatial, "fire_bp", "spatial");
    check_input(grad_spike, "fire_bp", "grad_spike");
    check_same_shape(spatial, grad_spike, "fire_bp", "spatial", "grad_spike");
    TORCH_CHECK(spatial.scalar_type() == grad_spike.scalar_type(), "snnlib.fire_bp: spatial (",
                spatial.scalar_type(), ") and grad_spike (", grad_spike.scalar_type(),
                ") must have the same dtype");
    TORCH_CHECK(spatial.device() == grad_spike.device(), "snnlib.fire_bp: spatial (",
                spatial.device(), ") and grad_spike (", grad_spike.device(),
                ") must be on the same device");
    const int dtype = storage_dtype(spatial, "fire_bp");
    const DeviceGuard guard(spatial.device());
    Tensor x = spatial.contiguous();
    Tensor grad_spatial = torch::empty_like(x, at::MemoryFormat::Contiguous);
    const Dims d = dims_of(x);
    // A gradient that is one [N] row expanded over time (stride 0 on the time axis: what autograd
    // hands over after `spike.sum(dim=0)`) is read in place, N values instead of T*N; any other
    // layout is made dense, as the reference's binding requires of its caller.
    Tensor g;
    int64_t grad_row_stride = d.N;
    if (grad_spike.dim() >= 2 && grad_spike.size(0) > 1 && grad_spike.stride(0) == 0 &&
        grad_spike.select(0, 0).is_contiguous()) {
        g = grad_spike.select(0, 0);
        grad_row_stride = 0;
    } else {
        g = grad_spike.contiguous();
    }

    // Windows longer than SNNLIF_BP_FUSED_MAX_T stage the recomputed membrane potential in a
    // workspace from the caching allocator; it goes back to the allocator on return and stays
    // valid for the work already queued because later users are ordered on the same stream.
    const size_t ws_bytes = snnlif_fire_bp_workspace_bytes(dtype, d.T, d.N);
    Tensor workspace;
    void* ws_ptr = nullptr;
    if (ws_bytes > 0) {
        workspace = torch::empty({static_cast<int64_t>(ws_bytes)}, x.options().dtype(at::kByte));
        ws_ptr = workspace.data_ptr();
    }
    check_rc(snnlif_fire_bp_strided(x.data_ptr(), g.data_ptr(), grad_spatial.data_ptr(), dtype, d.T,
                                    d.N, grad_row_stride, alpha, thresh, beta, interval, ws_ptr,
                                    ws_bytes, current_stream()),
             "fire_bp");
    return grad_spatial;
}

// ---- batch norm folded into the fire recurrence (fp32) -------------------------------------------

struct BnOperands {
    BnDims d;
    int dtype;  // SNNLIF_DTYPE_F32 or SNNLIF_DTYPE_F64; the per-channel tensors share it
    Tensor x, weight, bias, stat, mean;
};

// `stat` is the variance (forward) or the inverse standard deviation (backward side).
BnOperands bn_operands(const Tensor& spatial, const Tensor& weight_bn, const Tensor& bias_bn,
                       const Tensor& stat, const Tensor& mean, const char* op,
                       const char* stat_name) {
    check_input(spatial, op, "spatial");
    TORCH_CHECK(spatial.scalar_type() == at::kFloat || spatial.scalar_type() == at::kDouble,
                "snnlib.", op, ": only float32 and float64 are supported, got ",
                spatial.scalar_type());
    BnOperands o;
    o.dtype = spatial.scalar_type() == at::kFloat ? SNNLIF_DTYPE_F32 : SNNLIF_DTYPE_F64;
    o.d = bn_dims_of(spatial, op);
    o.x = spatial.contiguous();
    o.weight = channel_param(weight_bn, o.x, o.d.C, op, "weight_bn");
    o.bias = channel_param(bias_bn, o.x, o.d.C, op, "bias_bn");
    o.stat = channel_param(stat, o.x, o.d.C, op, stat_name);
    o.mean = channel_param(mean, o.x, o.d.C, op, "mean");
    return o;
}

// Per-channel batch statistics over every axis but the channel's (axis 2), on the hand-written
// reduction behind snnlif_bn_stats: what the layers of snnlib/example/snnlib_op.py obtain from
// torch.var_mean(x, dim_bn, unbiased=False) (:78) or, for a sharded batch, from torch.mean(x) and
// torch.mean(x**2) (:265-266) before they call a batch-norm op.  Not part of the reference's binding
// table.  raw_moments = false -> {var (biased), mean}; true -> {E[x], E[x^2]}.
std::vector<Tensor> batch_statistics(const Tensor& spatial, bool raw_moments, const char* op) {
    check_input(spatial, op, "spatial");
    TORCH_CHECK(spatial.scalar_type() == at::kFloat || spatial.scalar_type() == at::kDouble,
                "snnlib.", op, ": only float32 and float64 are supported, got ",
                spatial.scalar_type());
    const int dtype = spatial.scalar_type() == at::kFloat ? SNNLIF_DTYPE_F32 : SNNLIF_DTYPE_F64;
    const BnDims d = bn_dims_of(spatial, op);
    TORCH_CHECK(d.C == 0 || (d.T > 0 && d.B > 0 && d.HW > 0), "snnlib.", op,
                ": no elements per channel in a tensor shaped ", spatial.sizes());
    const DeviceGuard guard(spatial.device());
    Tensor x = spatial.contiguous();
    Tensor first = torch::empty({d.C}, x.options());
    Tensor second = torch::empty({d.C}, x.options());
    const size_t ws_bytes = snnlif_bn_stats_workspace_bytes(dtype, d.T, d.B, d.C, d.HW);
    Tensor workspace =
        torch::empty({static_cast<int64_t>(ws_bytes)}, x.options().dtype(at::kByte));
    check_rc(snnlif_bn_stats(x.data_ptr(), first.data_ptr(), second.data_ptr(), dtype, d.T, d.B, d.C,
                             d.HW, raw_moments ? 1 : 0, ws_bytes ? workspace.data_ptr() : nullptr,
                             ws_bytes, current_stream()),
             op);
    if (raw_moments) return {first, second};
    return {second, first};  // the order of torch.var_mean
}

std::vector<Tensor> bn_stats(Tensor spatial) { return batch_statistics(spatial, false, "bn_stats"); }

// bn_stats with the layer's running statistics advanced in the same pass:
//   -> {var, mean, running_var * keep + var * gain_var, running_mean * keep + mean * gain_mean}
// what the reference's layers compute in Python after torch.var_mean in training mode
// (snnlib/example/snnlib_op.py:78-80), bit for bit, without the six small element-wise launches.
std::vector<Tensor> bn_stats_running(Tensor spatial, Tensor running_var, Tensor running_mean,
                                     double keep, double gain_var, double gain_mean) {
    const char* op = "bn_stats_running";
    check_input(spatial, op, "spatial");
    TORCH_CHECK(spatial.scalar_type() == at::kFloat || spatial.scalar_type() == at::kDouble,
                "snnlib.", op, ": only float32 and float64 are supported, got ",
                spatial.scalar_type());
    const int dtype = spatial.scalar_type() == at::kFloat ? SNNLIF_DTYPE_F32 : SNNLIF_DTYPE_F64;
    const BnDims d = bn_dims_of(spatial, op);
    TORCH_CHECK(d.C == 0 || (d.T > 0 && d.B > 0 && d.HW > 0), "snnlib.", op,
                ": no elements per channel in a tensor shaped ", spatial.sizes());
    const DeviceGuard guard(spatial.device());
    Tensor x = spatial.contiguous();
    Tensor rv = channel_param(running_var.detach(), x, d.C, op, "running_var");
    Tensor rm = channel_param(running_mean.detach(), x, d.C, op, "running_mean");
    Tensor mean = torch::empty({d.C}, x.options());
    Tensor var = torch::empty({d.C}, x.options());
    Tensor new_rv = torch::empty({d.C}, x.options());
    Tensor new_rm = torch::empty({d.C}, x.options());
    const size_t ws_bytes = snnlif_bn_stats_workspace_bytes(dtype, d.T, d.B, d.C, d.HW);
    Tensor workspace =
        torch::empty({static_cast<int64_t>(ws_bytes)}, x.options().dtype(at::kByte));
    check_rc(snnlif_bn_stats_running(x.data_ptr(), mean.data_ptr(), var.data_ptr(), rm.data_ptr(),
                                     rv.data_ptr(), new_rm.data_ptr(), new_rv.data_ptr(), keep,
                                     gain_mean, gain_var, dtype, d.T, d.B, d.C, d.HW,
                                     ws_bytes ? workspace.data_ptr() : nullptr, ws_bytes,
                                     current_stream()),
             op);
    return {var, mean, new_rv, new_rm};
}

// The statistics of a sharded batch from its all-reduced moments and the running pair, one small
// kernel for the ten element-wise ops of snnlib/example/snnlib_op.py:271-275, with their bits:
//   -> {var, mean, running_var * keep + var * gain_var, running_mean * keep + mean * gain_mean}
std::vector<Tensor> bn_moments_finish(Tensor first, Tensor second, double world_size,
                                      Tensor running_var, Tensor running_mean, double keep,
                                      double gain_var, double gain_mean) {
    const char* op = "bn_moments_finish";
    TORCH_CHECK(first.defined() && first.is_cuda(), "snnlib.", op,
                ": first must live on a ROCm GPU (this build has no CPU path)");
    TORCH_CHECK(first.scalar_type() == at::kFloat || first.scalar_type() == at::kDouble, "snnlib.",
                op, ": only float32 and float64 are supported, got ", first.scalar_type());
    TORCH_CHECK(world_size >= 1.0, "snnlib.", op, ": world_size must be at least 1");
    const int dtype = first.scalar_type() == at::kFloat ? SNNLIF_DTYPE_F32 : SNNLIF_DTYPE_F64;
    const int64_t C = first.numel();
    const DeviceGuard guard(first.device());
    Tensor a = first.contiguous();
    Tensor b = channel_param(second, a, C, op, "second");
    Tensor rv = channel_param(running_var.detach(), a, C, op, "running_var");
    Tensor rm = channel_param(running_mean.detach(), a, C, op, "running_mean");
    Tensor mean = torch::empty({C}, a.options());
    Tensor var = torch::empty({C}, a.options());
    Tensor new_rv = torch::empty({C}, a.options());
    Tensor new_rm = torch::empty({C}, a.options());
    check_rc(snnlif_bn_moments_finish(a.data_ptr(), b.data_ptr(), mean.data_ptr(), var.data_ptr(),
                                      rm.data_ptr(), rv.data_ptr(), new_rm.data_ptr(),
                                      new_rv.data_ptr(), world_size, keep, gain_mean, gain_var, dtype,
                                      C, current_stream()),
             op);
    return {var, mean, new_rv, new_rm};
}

std::vector<Tensor> bn_moments(Tensor spatial) { return batch_statistics(spatial, true, "bn_moments"); }

std::vector<Tensor> bn_fire_s_fp(Tensor spatial, Tensor weight_bn, Tensor bias_bn, Tensor var,
                                 Tensor mean, float eps_bn, float alpha, float thresh) {
    const BnOperands o = bn_operands(spatial, weight_bn, bias_bn, var, mean, "bn_fire_s_fp", "var");
    const DeviceGuard guard(spatial.device());
    Tensor ivar = torch::empty_like(o.stat, at::MemoryFormat::Contiguous);
    Tensor spike = torch::empty_like(o.x, at::MemoryFormat::Contiguous);
    check_rc(snnlif_bn_fire_s_fp(o.x.data_ptr(), o.weight.data_ptr(), o.bias.data_ptr(),
                                 o.stat.data_ptr(), o.mean.data_ptr(), ivar.data_ptr(),
                                 spike.data_ptr(), o.dtype, o.d.T, o.d.B, o.d.C, o.d.HW,
                                 eps_bn, alpha, thresh, current_stream()),
             "bn_fire_s_fp");
    return {ivar, spike};
}

// Spikes of the bn + fire layer from the statistics its forward saved (backward-side scale
// weight * ivar, as the reference's bn_fire_us_fp_kernel uses: snnlib/cuda/snn_kernel_bp.cu:481-530).
Tensor bn_fire_spikes_from_ivar(const Tensor& spatial, const Tensor& weight_bn,
                                const Tensor& bias_bn, const Tensor& ivar, const Tensor& mean,
                                float alpha, float thresh, const char* op) {
    const BnOperands o = bn_operands(spatial, weight_bn, bias_bn, ivar, mean, op, "ivar");
    const DeviceGuard guard(spatial.device());
    Tensor spike = torch::empty_like(o.x, at::MemoryFormat::Contiguous);
    check_rc(snnlif_bn_fire_s_recompute(o.x.data_ptr(), o.weight.data_ptr(), o.bias.data_ptr(),
                                        o.stat.data_ptr(), o.mean.data_ptr(), spike.data_ptr(),
                                        o.dtype, o.d.T, o.d.B, o.d.C, o.d.HW, alpha, thresh,
                                        current_stream()),
             op);
    return spike;
}

std::vector<Tensor> bn_fire_bp(Tensor spatial, Tensor weight_bn, Tensor bias_bn, Tensor ivar,
                               Tensor mean, IntList dim_bn, Tensor grad_spike, float alpha,
                               float thresh, float beta, float interval) {
    (void)dim_bn;  // names the reduced axes ((0,1) or (0,1,3,4)); they follow from the shape here
    const BnOperands o = bn_operands(spatial, weight_bn, bias_bn, ivar, mean, "bn_fire_bp", "ivar");
    check_input(grad_spike, "bn_fire_bp", "grad_spike");
    check_like(grad_spike, spatial, "bn_fire_bp", "grad_spike");
    check_same_shape(spatial, grad_spike, "bn_fire_bp", "spatial", "grad_spike");
    const DeviceGuard guard(spatial.device());
    Tensor g = grad_spike.contiguous();
    Tensor grad_spatial = torch::empty_like(o.x, at::MemoryFormat::Contiguous);
    Tensor grad_weight = torch::empty_like(o.weight, at::MemoryFormat::Contiguous);
    Tensor grad_bias = torch::empty_like(o.weight, at::MemoryFormat::Contiguous);
    const size_t ws_bytes =
        snnlif_bn_fire_bp_workspace_bytes(o.dtype, o.d.T, o.d.B, o.d.C, o.d.HW);
    Tensor workspace =
        torch::empty({static_cast<int64_t>(ws_bytes)}, o.x.options().dtype(at::kByte));
    check_rc(snnlif_bn_fire_bp(o.x.data_ptr(), o.weight.data_ptr(), o.bias.data_ptr(),
                               o.stat.data_ptr(), o.mean.data_ptr(), g.data_ptr(),
                               grad_spatial.data_ptr(), grad_weight.data_ptr(), grad_bias.data_ptr(),
                               o.dtype, o.d.T, o.d.B, o.d.C, o.d.HW, alpha, thresh, beta,
                               interval, ws_bytes ? workspace.data_ptr() : nullptr, ws_bytes,
                               current_stream()),
             "bn_fire_bp");
    return {grad_spatial, reshaped_result(grad_weight, weight_bn.sizes()),
            reshaped_result(grad_bias, weight_bn.sizes())};
}

// The two halves of bn_fire_bp that a batch sharded over several GPUs runs before and after the
// all-reduce of the per-channel means (snnlib/cuda/snn_kernel_bp.cu:753-854).
std::vector<Tensor> bn_fire_bp_dist1(Tensor spatial, Tensor weight_bn, Tensor bias_bn, Tensor ivar,
                                     Tensor mean, IntList dim_bn, Tensor grad_spike, float alpha,
                                     float thresh, float beta, float interval) {
    (void)dim_bn;
    const char* op = "bn_fire_bp_dist1";
    const BnOperands o = bn_operands(spatial, weight_bn, bias_bn, ivar, mean, op, "ivar");
    check_input(grad_spike, op, "grad_spike");
    check_like(grad_spike, spatial, op, "grad_spike");
    check_same_shape(spatial, grad_spike, op, "spatial", "grad_spike");
    const DeviceGuard guard(spatial.device());
    Tensor g = grad_spike.contiguous();
    Tensor mean_gxhat = channel_result(o.weight, o.x);
    Tensor mean_gxhatx = channel_result(o.weight, o.x);
    Tensor grad_weight = channel_result(o.weight, o.x);
    Tensor grad_bias = channel_result(o.weight, o.x);
    const size_t ws_bytes =
        snnlif_bn_fire_bp_workspace_bytes(o.dtype, o.d.T, o.d.B, o.d.C, o.d.HW);
    Tensor workspace =
        torch::empty({static_cast<int64_t>(ws_bytes)}, o.x.options().dtype(at::kByte));
    check_rc(snnlif_bn_fire_bp_dist1(o.x.data_ptr(), o.weight.data_ptr(), o.bias.data_ptr(),
                                     o.stat.data_ptr(), o.mean.data_ptr(), g.data_ptr(),
                                     mean_gxhat.data_ptr(), mean_gxhatx.data_ptr(),
                                     grad_weight.data_ptr(), grad_bias.data_ptr(), o.dtype,
                                     o.d.T, o.d.B, o.d.C, o.d.HW, alpha, thresh, beta, interval,
                                     ws_bytes ? workspace.data_ptr() : nullptr, ws_bytes,
                                     current_stream()),
             op);
    return {mean_gxhat, mean_gxhatx, reshaped_result(grad_weight, weight_bn.sizes()),
            reshaped_result(grad_bias, weight_bn.sizes())};
}

Tensor bn_fire_bp_dist2(Tensor spatial, Tensor weight_bn, Tensor bias_bn, Tensor ivar, Tensor mean,
                        Tensor grad_spike, Tensor grad_xhat, Tensor grad_xhatx, float alpha,
                        float thresh, float beta, float interval) {
    const char* op = "bn_fire_bp_dist2";
    const BnOperands o = bn_operands(spatial, weight_bn, bias_bn, ivar, mean, op, "ivar");
    check_input(grad_spike, op, "grad_spike");
    check_like(grad_spike, spatial, op, "grad_spike");
    check_same_shape(spatial, grad_spike, op, "spatial", "grad_spike");
    Tensor gxhat = channel_param(grad_xhat, o.x, o.d.C, op, "grad_xhat");
    Tensor gxhatx = channel_param(grad_xhatx, o.x, o.d.C, op, "grad_xhatx");
    const DeviceGuard guard(spatial.device());
    Tensor g = grad_spike.contiguous();
    Tensor grad_spatial = torch::empty_like(o.x, at::MemoryFormat::Contiguous);
    check_rc(snnlif_bn_fire_bp_dist2(o.x.data_ptr(), o.weight.data_ptr(), o.bias.data_ptr(),
                                     o.stat.data_ptr(), o.mean.data_ptr(), g.data_ptr(),
                                     gxhat.data_ptr(), gxhatx.data_ptr(), grad_spatial.data_ptr(),
                                     o.dtype, o.d.T, o.d.B, o.d.C, o.d.HW, alpha, thresh,
                                     beta, interval, current_stream()),
             op);
    return grad_spatial;
}

// ---- plain batch norm (hand-written kernels behind snnlif_bn_fp / snnlif_bn_bp*) -------------------

struct PlainBnOperands {
    BnDims d;
    int dtype;  // SNNLIF_DTYPE_F32 or SNNLIF_DTYPE_F64; the per-channel tensors share it
    Tensor x;
};

PlainBnOperands plain_bn_operands(const Tensor& x_bn, const char* op) {
    check_input(x_bn, op, "x_bn");
    TORCH_CHECK(x_bn.scalar_type() == at::kFloat || x_bn.scalar_type() == at::kDouble, "snnlib.", op,
                ": only float32 and float64 are supported, got ", x_bn.scalar_type());
    PlainBnOperands o;
    o.dtype = x_bn.scalar_type() == at::kFloat ? SNNLIF_DTYPE_F32 : SNNLIF_DTYPE_F64;
    o.d = bn_dims_of(x_bn, op);
    o.x = x_bn.contiguous();
    return o;
}

// A gradient shaped, typed and placed like the activation, made dense.
Tensor dense_gradient(const Tensor& g, const Tensor& like, const char* op, const char* name) {
    check_input(g, op, name);
    check_like(g, like, op, name);
    check_same_shape(like, g, op, "x_bn", name);
    return g.contiguous();
}

Tensor byte_workspace(size_t bytes, const Tensor& like) {
    return torch::empty({static_cast<int64_t>(bytes)}, like.options().dtype(at::kByte));
}

std::vector<Tensor> bn_fp(Tensor x_bn, Tensor weight_bn, Tensor bias_bn, Tensor var, Tensor mean,
                          float eps_bn) {
    const char* op = "bn_fp";
    const PlainBnOperands o = plain_bn_operands(x_bn, op);
    Tensor w = channel_param(weight_bn, o.x, o.d.C, op, "weight_bn");
    Tensor b = channel_param(bias_bn, o.x, o.d.C, op, "bias_bn");
    Tensor v = channel_param(var, o.x, o.d.C, op, "var");
    Tensor m = channel_param(mean, o.x, o.d.C, op, "mean");
    const DeviceGuard guard(x_bn.device());
    Tensor ivar = torch::empty_like(v, at::MemoryFormat::Contiguous);
    Tensor y = torch::empty_like(o.x, at::MemoryFormat::Contiguous);
    check_rc(snnlif_bn_fp(o.x.data_ptr(), w.data_ptr(), b.data_ptr(), v.data_ptr(), m.data_ptr(),
                          ivar.data_ptr(), y.data_ptr(), o.dtype, o.d.T, o.d.B, o.d.C, o.d.HW, eps_bn,
                          current_stream()),
             op);
    return {ivar, y};
}

std::vector<Tensor> bn_bp(Tensor x_bn, Tensor weight_bn, Tensor bias_bn, Tensor ivar, Tensor mean,
                          IntList dim_bn, Tensor grad_y_bn) {
    (void)bias_bn;  // the gradients do not depend on it
    (void)dim_bn;   // names the reduced axes ((0,1) or (0,1,3,4)); they follow from the shape here
    const char* op = "bn_bp";
    const PlainBnOperands o = plain_bn_operands(x_bn, op);
    Tensor w = channel_param(weight_bn, o.x, o.d.C, op, "weight_bn");
    Tensor iv = channel_param(ivar, o.x, o.d.C, op, "ivar");
    Tensor m = channel_param(mean, o.x, o.d.C, op, "mean");
    Tensor g = dense_gradient(grad_y_bn, x_bn, op, "grad_y_bn");
    const DeviceGuard guard(x_bn.device());
    Tensor grad_x = torch::empty_like(o.x, at::MemoryFormat::Contiguous);
    Tensor grad_weight = channel_result(w, o.x);
    Tensor grad_bias = channel_result(w, o.x);
    const size_t ws_bytes = snnlif_bn_bp_workspace_bytes(o.dtype, o.d.T, o.d.B, o.d.C, o.d.HW);
    Tensor workspace = byte_workspace(ws_bytes, o.x);
    check_rc(snnlif_bn_bp(o.x.data_ptr(), w.data_ptr(), iv.data_ptr(), m.data_ptr(), g.data_ptr(),
                          grad_x.data_ptr(), grad_weight.data_ptr(), grad_bias.data_ptr(), o.dtype,
                          o.d.T, o.d.B, o.d.C, o.d.HW, ws_bytes ? workspace.data_ptr() : nullptr,
                          ws_bytes, current_stream()),
             op);
    return {grad_x, reshaped_result(grad_weight, weight_bn.sizes()),
            reshaped_result(grad_bias, weight_bn.sizes())};
}

// The two halves of bn_bp for a sharded batch (snnlib/cuda/snn_kernel_bp.cu:348-425): local
// parameter gradients and per-channel means, then the input gradient from the averaged means.
std::vector<Tensor> bn_bp_dist1(Tensor x_bn, Tensor weight_bn, Tensor bias_bn, Tensor ivar,
                                Tensor mean, IntList dim_bn, Tensor grad_y_bn) {
    (void)bias_bn;
    (void)dim_bn;
    const char* op = "bn_bp_dist1";
    const PlainBnOperands o = plain_bn_operands(x_bn, op);
    Tensor w = channel_param(weight_bn, o.x, o.d.C, op, "weight_bn");
    Tensor iv = channel_param(ivar, o.x, o.d.C, op, "ivar");
    Tensor m = channel_param(mean, o.x, o.d.C, op, "mean");
    Tensor g = dense_gradient(grad_y_bn, x_bn, op, "grad_y_bn");
    const DeviceGuard guard(x_bn.device());
    Tensor mean_gxhat = channel_result(w, o.x);
    Tensor mean_gxhatx = channel_result(w, o.x);
    Tensor grad_weight = channel_result(w, o.x);
    Tensor grad_bias = channel_result(w, o.x);
    const size_t ws_bytes = snnlif_bn_bp_workspace_bytes(o.dtype, o.d.T, o.d.B, o.d.C, o.d.HW);
    Tensor workspace = byte_workspace(ws_bytes, o.x);
    check_rc(snnlif_bn_bp_dist1(o.x.data_ptr(), w.data_ptr(), iv.data_ptr(), m.data_ptr(),
                                g.data_ptr(), mean_gxhat.data_ptr(), mean_gxhatx.data_ptr(),
                                grad_weight.data_ptr(), grad_bias.data_ptr(), o.dtype, o.d.T, o.d.B,
                                o.d.C, o.d.HW, ws_bytes ? workspace.data_ptr() : nullptr, ws_bytes,
                                current_stream()),
             op);
    return {mean_gxhat, mean_gxhatx, grad_weight, grad_bias};
}

Tensor bn_bp_dist2(Tensor x_bn, Tensor weight_bn, Tensor bias_bn, Tensor ivar, Tensor mean,
                   IntList dim_bn, Tensor grad_y_bn, Tensor grad_xhat, Tensor grad_xhatx) {
    (void)bias_bn;
    (void)dim_bn;
    const char* op = "bn_bp_dist2";
    const PlainBnOperands o = plain_bn_operands(x_bn, op);
    Tensor w = channel_param(weight_bn, o.x, o.d.C, op, "weight_bn");
    Tensor iv = channel_param(ivar, o.x, o.d.C, op, "ivar");
    Tensor m = channel_param(mean, o.x, o.d.C, op, "mean");
    Tensor gxhat = channel_param(grad_xhat, o.x, o.d.C, op, "grad_xhat");
    Tensor gxhatx = channel_param(grad_xhatx, o.x, o.d.C, op, "grad_xhatx");
    Tensor g = dense_gradient(grad_y_bn, x_bn, op, "grad_y_bn");
    const DeviceGuard guard(x_bn.device());
    Tensor grad_x = torch::empty_like(o.x, at::MemoryFormat::Contiguous);
    check_rc(snnlif_bn_bp_dist2(o.x.data_ptr(), w.data_ptr(), iv.data_ptr(), m.data_ptr(),
                                g.data_ptr(), gxhat.data_ptr(), gxhatx.data_ptr(), grad_x.data_ptr(),
                                o.dtype, o.d.T, o.d.B, o.d.C, o.d.HW, current_stream()),
             op);
    return grad_x;
}

// ---- dense layers without fire (ATen only) --------------------------------------------------------

Tensor fc_fp(Tensor spatial, Tensor weight_fc, Tensor bias_fc) {
    check_input(spatial, "fc_fp", "spatial");
    check_like(weight_fc, spatial, "fc_fp", "weight_fc");
    check_like(bias_fc, spatial, "fc_fp", "bias_fc");
    check_fc_weight(spatial, weight_fc, "fc_fp");
    const DeviceGuard guard(spatial.device());
    return linear_folded(spatial, weight_fc, bias_fc);
}

std::vector<Tensor> fc_bp(Tensor spatial, Tensor grad_fc, Tensor weight_fc, Tensor bias_fc,
                          IntList dim_fc) {
    (void)bias_fc;  // kept for signature parity; the bias gradient needs only grad_fc
    check_input(spatial, "fc_bp", "spatial");
    check_like(weight_fc, spatial, "fc_bp", "weight_fc");
    check_like(grad_fc, spatial, "fc_bp", "grad_fc");
    check_fc_weight(spatial, weight_fc, "fc_bp");
    const DeviceGuard guard(spatial.device());
    return linear_backward_folded(spatial, grad_fc, weight_fc, dim_fc, "fc_bp");
}

// `benchmark` / `deterministic` reach MIOpen through ConvSearchGuard; `allow_tf32` has no meaning on
// this hardware and is ignored.
Tensor conv_fp(Tensor spatial, Tensor weight_conv, Tensor bias_conv, IntList stride,
               IntList padding, IntList dilation, int64_t groups, bool benchmark,
               bool deterministic) {
    check_input(spatial, "conv_fp", "spatial");
    check_image(spatial, "conv_fp");
    check_like(weight_conv, spatial, "conv_fp", "weight_conv");
    check_like(bias_conv, spatial, "conv_fp", "bias_conv");
    const DeviceGuard guard(spatial.device());
    return conv_folded(spatial, weight_conv, bias_conv, stride, padding, dilation, groups, benchmark,
                       deterministic);
}

std::vector<Tensor> conv_bp(Tensor spatial, Tensor grad_conv, Tensor weight_conv, IntList stride,
                            IntList padding, IntList dilation, int64_t groups, bool benchmark,
                            bool deterministic, bool /*allow_tf32*/, IntList dim_conv) {
    check_input(spatial, "conv_bp", "spatial");
    check_image(spatial, "conv_bp");
    check_like(weight_conv, spatial, "conv_bp", "weight_conv");
    check_like(grad_conv, spatial, "conv_bp", "grad_conv");
    const DeviceGuard guard(spatial.device());
    return conv_backward_folded(spatial, grad_conv, weight_conv, stride, padding, dilation, groups,
                                benchmark, deterministic, dim_conv, "conv_bp");
}

// ---- fire, then a fully connected layer / a convolution -------------------------------------------

Tensor fire_fc_fp(Tensor spatial, Tensor weight_fc, Tensor bias_fc, float alpha, float thresh) {
    check_input(spatial, "fire_fc_fp", "spatial");
    check_like(weight_fc, spatial, "fire_fc_fp", "weight_fc");
    check_like(bias_fc, spatial, "fire_fc_fp", "bias_fc");
    check_fc_weight(spatial, weight_fc, "fire_fc_fp");
    Tensor spike = fire_s_fp(spatial, alpha, thresh);
    const DeviceGuard guard(spatial.device());
    return linear_folded(spike, weight_fc, bias_fc);
}

std::vector<Tensor> fire_fc_bp(Tensor spatial, Tensor grad_fc, Tensor weight_fc, Tensor bias_fc,
                               IntList dim_fc, float alpha, float thresh, float beta,
                               float interval) {
    (void)bias_fc;
    check_input(spatial, "fire_fc_bp", "spatial");
    check_like(weight_fc, spatial, "fire_fc_bp", "weight_fc");
    check_like(grad_fc, spatial, "fire_fc_bp", "grad_fc");
    check_fc_weight(spatial, weight_fc, "fire_fc_bp");
    Tensor spike = fire_s_fp(spatial, alpha, thresh);  // recomputed: only the input current is saved
    const DeviceGuard guard(spatial.device());
    auto dense = linear_backward_folded(spike, grad_fc, weight_fc, dim_fc, "fire_fc_bp");
    return {fire_bp(spatial, dense[0], alpha, thresh, beta, interval), dense[1], dense[2]};
}

Tensor fire_conv_fp(Tensor spatial, Tensor weight_conv, Tensor bias_conv, IntList stride,
                    IntList padding, IntList dilation, int64_t groups, bool benchmark,
                    bool deterministic, float alpha, float thresh) {
    check_input(spatial, "fire_conv_fp", "spatial");
    check_image(spatial, "fire_conv_fp");
    check_like(weight_conv, spatial, "fire_conv_fp", "weight_conv");
    check_like(bias_conv, spatial, "fire_conv_fp", "bias_conv");
    Tensor spike = fire_s_fp(spatial, alpha, thresh);
    const DeviceGuard guard(spatial.device());
    return conv_folded(spike, weight_conv, bias_conv, stride, padding, dilation, groups, benchmark,
                       deterministic);
}

std::vector<Tensor> fire_conv_bp(Tensor spatial, Tensor grad_conv, Tensor weight_conv,
                                 IntList stride, IntList padding, IntList dilation, int64_t groups,
                                 bool benchmark, bool deterministic, bool /*allow_tf32*/,
                                 IntList dim_conv, float alpha, float thresh, float beta,
                                 float interval) {
    check_input(spatial, "fire_conv_bp", "spatial");
    check_image(spatial, "fire_conv_bp");
    check_like(weight_conv, spatial, "fire_conv_bp", "weight_conv");
    check_like(grad_conv, spatial, "fire_conv_bp", "grad_conv");
    Tensor spike = fire_s_fp(spatial, alpha, thresh);
    const DeviceGuard guard(spatial.device());
    auto dense = conv_backward_folded(spike, grad_conv, weight_conv, stride, padding, dilation,
                                      groups, benchmark, deterministic, dim_conv, "fire_conv_bp");
    return {fire_bp(spatial, dense[0], alpha, thresh, beta, interval), dense[1], dense[2]};
}

// ---- batch norm + fire, then a fully connected layer / a convolution ------------------------------

std::vector<Tensor> bn_fire_fc_fp(Tensor spatial, Tensor weight_bn, Tensor bias_bn, Tensor var,
                                  Tensor mean, float eps_bn, Tensor weight_fc, Tensor bias_fc,
                                  float alpha, float thresh) {
    check_input(spatial, "bn_fire_fc_fp", "spatial");
    check_like(weight_fc, spatial, "bn_fire_fc_fp", "weight_fc");
    check_like(bias_fc, spatial, "bn_fire_fc_fp", "bias_fc");
    check_fc_weight(spatial, weight_fc, "bn_fire_fc_fp");
    auto fired = bn_fire_s_fp(spatial, weight_bn, bias_bn, var, mean, eps_bn, alpha, thresh);
    const DeviceGuard guard(spatial.device());
    return {fired[0], linear_folded(fired[1], weight_fc, bias_fc)};
}

std::vector<Tensor> bn_fire_fc_bp(Tensor spatial, Tensor weight_bn, Tensor bias_bn, Tensor ivar,
                                  Tensor mean, IntList dim_bn, Tensor grad_fc, Tensor weight_fc,
                                  Tensor bias_fc, IntList dim_fc, float alpha, float thresh,
                                  float beta, float interval) {
    (void)bias_fc;
    check_input(spatial, "bn_fire_fc_bp", "spatial");
    check_like(weight_fc, spatial, "bn_fire_fc_bp", "weight_fc");
    check_like(grad_fc, spatial, "bn_fire_fc_bp", "grad_fc");
    check_fc_weight(spatial, weight_fc, "bn_fire_fc_bp");
    Tensor spike = bn_fire_spikes_from_ivar(spatial, weight_bn, bias_bn, ivar, mean, alpha, thresh,
                                            "bn_fire_fc_bp");
    const DeviceGuard guard(spatial.device());
    auto dense = linear_backward_folded(spike, grad_fc, weight_fc, dim_fc, "bn_fire_fc_bp");
    auto bn = bn_fire_bp(spatial, weight_bn, bias_bn, ivar, mean, dim_bn, dense[0], alpha, thresh,
                         beta, interval);
    return {bn[0], bn[1], bn[2], dense[1], dense[2]};
}

std::vector<Tensor> bn_fire_conv_fp(Tensor spatial, Tensor weight_bn, Tensor bias_bn, Tensor var,
                                    Tensor mean, float eps_bn, Tensor weight_conv,
                                    Tensor bias_conv, IntList stride, IntList padding,
                                    IntList dilation, int64_t groups, bool benchmark,
                                    bool deterministic, float alpha, float thresh) {
    check_input(spatial, "bn_fire_conv_fp", "spatial");
    check_image(spatial, "bn_fire_conv_fp");
    check_like(weight_conv, spatial, "bn_fire_conv_fp", "weight_conv");
    check_like(bias_conv, spatial, "bn_fire_conv_fp", "bias_conv");
    auto fired = bn_fire_s_fp(spatial, weight_bn, bias_bn, var, mean, eps_bn, alpha, thresh);
    const DeviceGuard guard(spatial.device());
    return {fired[0],
            conv_folded(fired[1], weight_conv, bias_conv, stride, padding, dilation, groups, benchmark,
                        deterministic)};
}

std::vector<Tensor> bn_fire_conv_bp(Tensor spatial, Tensor weight_bn, Tensor bias_bn, Tensor ivar,
                                    Tensor mean, IntList dim_bn, Tensor grad_conv,
                                    Tensor weight_conv, IntList stride, IntList padding,
                                    IntList dilation, int64_t groups, bool benchmark,
                                    bool deterministic, bool /*allow_tf32*/, IntList dim_conv,
                                    float alpha, float thresh, float beta, float interval) {
    check_input(spatial, "bn_fire_conv_bp", "spatial");
    check_image(spatial, "bn_fire_conv_bp");
    check_like(weight_conv, spatial, "bn_fire_conv_bp", "weight_conv");
    check_like(grad_conv, spatial, "bn_fire_conv_bp", "grad_conv");
    Tensor spike = bn_fire_spikes_from_ivar(spatial, weight_bn, bias_bn, ivar, mean, alpha, thresh,
                                            "bn_fire_conv_bp");
    const DeviceGuard guard(spatial.device());
    auto dense = conv_backward_folded(spike, grad_conv, weight_conv, stride, padding, dilation,
                                      groups, benchmark, deterministic, dim_conv, "bn_fire_conv_bp");
    auto bn = bn_fire_bp(spatial, weight_bn, bias_bn, ivar, mean, dim_bn, dense[0], alpha, thresh,
                         beta, interval);
    return {bn[0], bn[1], bn[2], dense[1], dense[2]};
}

// Sharded-batch form of bn_fire_fc_bp / bn_fire_conv_bp: everything up to the all-reduce, with the
// gradient of the spikes handed back for bn_fire_bp_dist2
// (snnlib/cuda/snn_kernel_bp.cu:966-1061, 1265-1340).
std::vector<Tensor> bn_fire_fc_bp_dist1(Tensor spatial, Tensor weight_bn, Tensor bias_bn,
                                        Tensor ivar, Tensor mean, IntList dim_bn, Tensor grad_fc,
                                        Tensor weight_fc, Tensor bias_fc, IntList dim_fc, float alpha,
                                        float thresh, float beta, float interval) {
    (void)bias_fc;
    const char* op = "bn_fire_fc_bp_dist1";
    check_input(spatial, op, "spatial");
    check_like(weight_fc, spatial, op, "weight_fc");
    check_like(grad_fc, spatial, op, "grad_fc");
    check_fc_weight(spatial, weight_fc, op);
    Tensor spike = bn_fire_spikes_from_ivar(spatial, weight_bn, bias_bn, ivar, mean, alpha, thresh, op);
    const DeviceGuard guard(spatial.device());
    auto dense = linear_backward_folded(spike, grad_fc, weight_fc, dim_fc, op);
    auto bn = bn_fire_bp_dist1(spatial, weight_bn, bias_bn, ivar, mean, dim_bn, dense[0], alpha,
                               thresh, beta, interval);
    return {dense[0], bn[0], bn[1], bn[2], bn[3], dense[1], dense[2]};
}

std::vector<Tensor> bn_fire_conv_bp_dist1(Tensor spatial, Tensor weight_bn, Tensor bias_bn,
                                          Tensor ivar, Tensor mean, IntList dim_bn, Tensor grad_conv,
                                          Tensor weight_conv, IntList stride, IntList padding,
                                          IntList dilation, int64_t groups, bool benchmark,
                                          bool deterministic, bool /*allow_tf32*/,
                                          IntList dim_conv, float alpha, float thresh, float beta,
                                          float interval) {
    const char* op = "bn_fire_conv_bp_dist1";
    check_input(spatial, op, "spatial");
    check_image(spatial, op);
    check_like(weight_conv, spatial, op, "weight_conv");
    check_like(grad_conv, spatial, op, "grad_conv");
    Tensor spike = bn_fire_spikes_from_ivar(spatial, weight_bn, bias_bn, ivar, mean, alpha, thresh, op);
    const DeviceGuard guard(spatial.device());
    auto dense = conv_backward_folded(spike, grad_conv, weight_conv, stride, padding, dilation,
                                      groups, benchmark, deterministic, dim_conv, op);
    auto bn = bn_fire_bp_dist1(spatial, weight_bn, bias_bn, ivar, mean, dim_bn, dense[0], alpha,
                               thresh, beta, interval);
    return {dense[0], bn[0], bn[1], bn[2], bn[3], dense[1], dense[2]};
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "snnlib layer operators for MI355X (gfx950): LIF fire kernels + PyTorch-ROCm dense ops";
    m.attr("__backend__") = "hip-gfx950";
    m.attr("__abi_version__") = snnlif_abi_version();

    m.def("fire_s_fp", &fire_s_fp, "fire (spike) forward");
    m.def("fire_us_fp", &fire_us_fp, "fire (membrane potential, spike) forward");
    m.def("bn_fire_s_fp", &bn_fire_s_fp, "bn fire (spike) forward");

    m.def("bn_stats", &bn_stats, "per-channel [biased variance, mean] of a [T, B, C, ...] tensor");
    m.def("bn_moments", &bn_moments, "per-channel [E[x], E[x^2]] of a [T, B, C, ...] tensor");
    m.def("bn_stats_running", &bn_stats_running,
          "bn_stats plus the running statistics: [var, mean, new_running_var, new_running_mean]");
    m.def("bn_moments_finish", &bn_moments_finish,
          "[var, mean, new_running_var, new_running_mean] from a sharded batch's all-reduced moments");

    m.def("bn_fp", &bn_fp, "bn forward");
    m.def("bn_bp", &bn_bp, "bn backward");

    m.def("bn_fire_fc_fp", &bn_fire_fc_fp, "bn fire fc forward");
    m.def("fire_fc_fp", &fire_fc_fp, "fire fc forward");
    m.def("fc_fp", &fc_fp, "fc forward");

    m.def("bn_fire_conv_fp", &bn_fire_conv_fp, "bn fire conv forward");
    m.def("fire_conv_fp", &fire_conv_fp, "fire conv forward");
    m.def("conv_fp", &conv_fp, "conv forward");

    m.def("fire_bp", &fire_bp, "fire backward");
    m.def("bn_fire_bp", &bn_fire_bp, "bn fire backward");

    m.def("bn_fire_fc_bp", &bn_fire_fc_bp, "bn fire fc backward");
    m.def("fire_fc_bp", &fire_fc_bp, "fire fc backward");
    m.def("fc_bp", &fc_bp, "fc backward");

    m.def("bn_fire_conv_bp", &bn_fire_conv_bp, "bn fire conv backward");
    m.def("fire_conv_bp", &fire_conv_bp, "fire conv backward");
    m.def("conv_bp", &conv_bp, "conv backward");

    m.def("bn_bp_dist1", &bn_bp_dist1, "bn backward, sharded batch: before the all-reduce");
    m.def("bn_bp_dist2", &bn_bp_dist2, "bn backward, sharded batch: after the all-reduce");
    m.def("bn_fire_bp_dist1", &bn_fire_bp_dist1, "bn fire backward, sharded batch: before the all-reduce");
    m.def("bn_fire_bp_dist2", &bn_fire_bp_dist2, "bn fire backward, sharded batch: after the all-reduce");
    m.def("bn_fire_fc_bp_dist1", &bn_fire_fc_bp_dist1, "bn fire fc backward, sharded batch: before the all-reduce");
    m.def("bn_fire_conv_bp_dist1", &bn_fire_conv_bp_dist1, "bn fire conv backward, sharded batch: before the all-reduce");
}
