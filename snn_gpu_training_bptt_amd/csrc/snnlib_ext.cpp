// Python extension module `snnlib` for PyTorch-ROCm: the operator boundary that
// snnlib_func.FireFunc calls (reference: snnlib/example/snnlib_func.py:25-34).
//
// It exposes the reference's positional signatures (snnlib/cuda/snn.cpp:11-17, 270-279, bound at
// :799 and :813)
//     fire_s_fp(spatial, alpha, thresh)                               -> spike
//     fire_bp(spatial, grad_spike, alpha, thresh, beta, interval)     -> grad_spatial
// plus fire_us_fp(spatial, alpha, thresh) -> (mem, spike), the public face of the reference's
// internal fire_us_fp_kernel (snnlib/cuda/snn_kernel_bp.cu:54-93).
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

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "snnlib LIF fire operators for MI355X (gfx950)";
    m.attr("__backend__") = "hip-gfx950";
    m.attr("__abi_version__") = snnlif_abi_version();
    m.def("fire_s_fp", &fire_s_fp, "fire (spike) forward");
    m.def("fire_us_fp", &fire_us_fp, "fire (membrane potential, spike) forward");
    m.def("fire_bp", &fire_bp, "fire backward");
}
