"""CPU-only checks of the boundary: the C-ABI library loads and exports every symbol the header
declares, argument validation that needs no GPU, the ``snnlib`` module surface, and the Python
mirror of the reference's interface (snnlib/example/snnlib_func.py:10-36,
snnlib/example/snnlib_op.py:11-16).  No kernel is launched here.
"""
import ctypes
import os
import re
import subprocess
import sys

import pytest
import torch

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(REPO, "include", "snnlib_lif.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(snnlif_\w+)\s*\(", text)))


def test_header_and_ctypes_table_agree():
    from snn_gpu_training_bptt_amd import lif_cabi
    assert declared_functions() == sorted(lif_cabi.SYMBOLS)


def test_library_exports_every_declared_symbol():
    from snn_gpu_training_bptt_amd import lif_cabi
    lib = ctypes.CDLL(lif_cabi.LIB_PATH)
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} is declared in include/snnlib_lif.h but not exported"


def test_constants_match_the_header():
    from snn_gpu_training_bptt_amd import lif_cabi
    text = open(HEADER).read()
    macros = dict(re.findall(r"#define\s+(SNNLIF_\w+)\s+(-?\d+)", text))
    assert int(macros["SNNLIF_DTYPE_F32"]) == lif_cabi.DTYPE_F32
    assert int(macros["SNNLIF_DTYPE_F64"]) == lif_cabi.DTYPE_F64
    assert int(macros["SNNLIF_DTYPE_BF16"]) == lif_cabi.DTYPE_BF16
    hexes = dict(re.findall(r"#define\s+(SNNLIF_\w+)\s+(0x[0-9a-fA-F]+)", text))
    assert int(hexes["SNNLIF_KEEP_SPATIAL"], 16) == lif_cabi.KEEP_SPATIAL
    assert int(hexes["SNNLIF_STREAM_SPATIAL"], 16) == lif_cabi.STREAM_SPATIAL
    assert int(macros["SNNLIF_ERR_ARG"]) == lif_cabi.ERR_ARG
    assert int(macros["SNNLIF_ERR_DTYPE"]) == lif_cabi.ERR_DTYPE
    assert int(macros["SNNLIF_ERR_WORKSPACE"]) == lif_cabi.ERR_WORKSPACE
    assert int(macros["SNNLIF_ERR_ALIGN"]) == lif_cabi.ERR_ALIGN
    assert int(macros["SNNLIF_ERR_UNSUPPORTED"]) == lif_cabi.ERR_UNSUPPORTED
    assert int(macros["SNNLIF_ERR_SCRATCH"]) == lif_cabi.ERR_SCRATCH
    shift = re.search(r"#define\s+SNNLIF_STATIC_SCRATCH_BYTES\s+\((\d+)u\s*<<\s*(\d+)\)", text)
    assert int(shift.group(1)) << int(shift.group(2)) == lif_cabi.STATIC_SCRATCH_BYTES
    assert int(macros["SNNLIF_BP_FUSED_MAX_T"]) == lif_cabi.BP_FUSED_MAX_T
    assert int(macros["SNNLIF_BP_NO_WORKSPACE_MAX_T"]) == lif_cabi.BP_NO_WORKSPACE_MAX_T
    lib = lif_cabi.load()
    assert lib.snnlif_abi_version() == int(macros["SNNLIF_ABI_VERSION"]) == lif_cabi.ABI_VERSION == 3
    assert lif_cabi.bn_bp_workspace_bytes(lif_cabi.DTYPE_F32, 8, 64, 128, 1024) == (2 * 64 * 128 * 16 + 2 * 128) * 4
    assert lif_cabi.bn_bp_workspace_bytes(lif_cabi.DTYPE_F64, 6, 2, 8, 1) == (2 * 2 * 8 + 2 * 8) * 8
    assert lif_cabi.bn_bp_workspace_bytes(lif_cabi.DTYPE_BF16, 6, 2, 8, 1) == 0
    assert lib.snnlif_target_arch() == b"gfx950"


def test_host_side_queries_need_no_gpu():
    from snn_gpu_training_bptt_amd import lif_cabi
    lib = lif_cabi.load()
    f32, f64, bf16 = lif_cabi.DTYPE_F32, lif_cabi.DTYPE_F64, lif_cabi.DTYPE_BF16
    assert lif_cabi.fire_bp_workspace_bytes(f32, 8, 1 << 23) == 0
    assert lif_cabi.fire_bp_workspace_bytes(f32, 32, 100) == 0
    assert lif_cabi.fire_bp_workspace_bytes(f32, 33, 100) == 0            # segmented on chip
    assert lif_cabi.fire_bp_workspace_bytes(f32, 1024, 100) == 0
    assert lif_cabi.fire_bp_workspace_bytes(f32, 1025, 100) == 1025 * 100 * 4
    assert lif_cabi.fire_bp_workspace_bytes(f64, 2000, 10) == 2000 * 10 * 8
    assert lif_cabi.fire_bp_workspace_bytes(bf16, 2000, 10) == 2000 * 10 * 4   # fp32 arithmetic
    assert lif_cabi.fire_bp_workspace_bytes(7, 2000, 10) == 0
    assert lif_cabi.fire_bp_workspace_bytes(f32, -1, 10) == 0
    for code in (0, -1, -2, -3, -4, -99):
        assert lif_cabi.strerror(code)
    assert "workspace" in lif_cabi.strerror(lif_cabi.ERR_WORKSPACE)
    # argument errors are reported before any device work
    assert lib.snnlif_fire_s_fp(None, None, 9, 4, 8, 0.25, 0.5, None) == lif_cabi.ERR_DTYPE
    assert lib.snnlif_fire_s_fp(None, None, f32, -4, 8, 0.25, 0.5, None) == lif_cabi.ERR_ARG
    assert lib.snnlif_fire_s_fp(None, None, f32, 4, 8, 0.25, 0.5, None) == lif_cabi.ERR_ARG
    assert lib.snnlif_fire_s_fp(None, None, f32, 0, 8, 0.25, 0.5, None) == lif_cabi.OK       # empty: no-op
    assert lib.snnlif_fire_bp(None, None, None, f32, 4, 0, 0.25, 0.5, 1.0, 0.5, None, 0, None) == lif_cabi.OK
    assert lib.snnlif_fire_bp(None, None, None, f32, 4, 8, 0.25, 0.5, 1.0, 0.5, None, 0, None) == lif_cabi.ERR_ARG
    assert lib.snnlif_fire_us_fp(None, None, None, f32, 1 << 40, 1 << 40, 0.25, 0.5, None) == lif_cabi.ERR_ARG
    # cache hints ride in the dtype argument: either one is fine, both or unknown bits are not
    for hint in (lif_cabi.KEEP_SPATIAL, lif_cabi.STREAM_SPATIAL):
        assert lib.snnlif_fire_s_fp(None, None, f32 | hint, 0, 8, 0.25, 0.5, None) == lif_cabi.OK
        assert lif_cabi.fire_bp_workspace_bytes(f64 | hint, 2000, 10) == 2000 * 10 * 8
    both = lif_cabi.KEEP_SPATIAL | lif_cabi.STREAM_SPATIAL
    assert lib.snnlif_fire_s_fp(None, None, f32 | both, 0, 8, 0.25, 0.5, None) == lif_cabi.ERR_DTYPE
    assert lib.snnlif_fire_s_fp(None, None, f32 | 0x1000, 0, 8, 0.25, 0.5, None) == lif_cabi.ERR_DTYPE


def test_snnlib_module_surface_and_cpu_rejection():
    from snn_gpu_training_bptt_amd import snnlib_func as sf
    import snnlib  # registered under the reference's top-level name by the package
    assert snnlib is sf.snnlib
    assert snnlib.__backend__ == "hip-gfx950"
    for name in ("fire_s_fp", "fire_bp", "fire_us_fp", "bn_stats", "bn_moments", "bn_stats_running",
                 "bn_moments_finish"):
        assert callable(getattr(snnlib, name))
    # positional signatures of the reference binding (snnlib/cuda/snn.cpp:11-17, 270-279)
    with pytest.raises(TypeError):
        snnlib.fire_s_fp(torch.zeros(2, 3))
    with pytest.raises(TypeError):
        snnlib.fire_bp(torch.zeros(2, 3), torch.zeros(2, 3), 0.25, 0.5)
    # no CPU path: a host tensor is an error, never a silent fallback
    with pytest.raises(RuntimeError, match="ROCm GPU"):
        snnlib.fire_s_fp(torch.zeros(2, 3), 0.25, 0.5)
    with pytest.raises(RuntimeError, match="ROCm GPU"):
        snnlib.fire_bp(torch.zeros(2, 3), torch.zeros(2, 3), 0.25, 0.5, 1.0, 0.5)
    with pytest.raises(RuntimeError, match="ROCm GPU"):
        snnlib.bn_stats(torch.zeros(2, 3, 4))


def test_python_interface_mirrors_the_reference():
    from snn_gpu_training_bptt_amd import snnlib_func as sf
    from snn_gpu_training_bptt_amd import snnlib_op as sop
    # hyper-parameter globals and their defaults (snnlib/example/snnlib_func.py:10-15)
    assert (sf.alpha, sf.beta, sf.interval, sf.thresh, sf.time_step) == (0.25, 1.0, 0.5, 0.25, 6)
    assert issubclass(sf.FireFunc, torch.autograd.Function)
    assert sf.fire_func == sf.FireFunc.apply
    # every layer and autograd function of the reference's two files, the sharded-batch ones included
    for name in ("Fire", "Bn", "BnFire", "BnFireFc", "FireFc", "Fc", "BnFireConv", "FireConv", "Conv",
                 "BnDist", "BnFireFcDist", "BnFireConvDist"):
        assert issubclass(getattr(sop, name), torch.nn.Module), name
    for name in ("fire", "bn", "bn_fire", "bn_fire_fc", "fire_fc", "fc", "bn_fire_conv", "fire_conv", "conv",
                 "bn_dist", "bn_fire_fc_dist", "bn_fire_conv_dist"):
        cls = getattr(sf, "".join(w.capitalize() for w in name.split("_")) + "Func")
        assert issubclass(cls, torch.autograd.Function) and callable(getattr(sf, name + "_func")), name
    for name in ("bn_bp_dist1", "bn_bp_dist2", "bn_fire_bp_dist1", "bn_fire_bp_dist2",
                 "bn_fire_fc_bp_dist1", "bn_fire_conv_bp_dist1"):     # snnlib/cuda/snn.cpp:824-829
        assert callable(getattr(sf.snnlib, name)), name
    fire = sop.Fire()
    assert isinstance(fire, torch.nn.Module)
    assert list(fire.parameters()) == [] and list(fire.buffers()) == []
    assert fire.state_dict() == {}
    # a CPU tensor reaches the native op and is refused there (no pure-PyTorch fallback)
    with pytest.raises(RuntimeError, match="ROCm GPU"):
        fire(torch.zeros(6, 2, 8, requires_grad=True))


def test_missing_library_fails_loudly(tmp_path, monkeypatch):
    from snn_gpu_training_bptt_amd import lif_cabi
    monkeypatch.setattr(lif_cabi, "_lib", None)
    monkeypatch.setattr(lif_cabi, "LIB_PATH", str(tmp_path / "libsnnlif_gfx950.so"))
    with pytest.raises(ImportError, match="no CPU or PyTorch fallback"):
        lif_cabi.load()


def test_product_never_imports_the_oracle():
    pkg = os.path.join(REPO, "snn_gpu_training_bptt_amd")
    for root, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".h")):
                text = open(os.path.join(root, f)).read()
                assert "oracle" not in text.lower().replace("no cpu or pytorch fallback", ""), \
                    f"{f} mentions the oracle; the shipped package must not depend on test infrastructure"


def test_bench_refuses_more_than_one_gpu():
    proc = subprocess.run([sys.executable, os.path.join(REPO, "bench.py"), "--gpus", "2"],
                          capture_output=True, text=True)
    assert proc.returncode != 0
    assert "one GPU" in proc.stderr


ROUTE_A = r"""
import sys
sys.path.insert(0, sys.argv[1])          # the directory that holds snnlib.so, nothing else of this build
import torch
import snnlib                            # what the reference's snnlib_func.py does (its line 8)
assert "snn_gpu_training_bptt_amd" not in sys.modules
names = ["fire_s_fp", "fire_bp", "bn_fire_s_fp", "bn_fire_bp", "bn_fp", "bn_bp", "fc_fp", "fc_bp", "conv_fp",
         "conv_bp", "fire_fc_fp", "fire_fc_bp", "fire_conv_fp", "fire_conv_bp", "bn_fire_fc_fp", "bn_fire_fc_bp",
         "bn_fire_conv_fp", "bn_fire_conv_bp", "bn_bp_dist1", "bn_bp_dist2", "bn_fire_bp_dist1",
         "bn_fire_bp_dist2", "bn_fire_fc_bp_dist1", "bn_fire_conv_bp_dist1"]
missing = [n for n in names if not callable(getattr(snnlib, n, None))]
assert not missing, missing
if len(sys.argv) > 2:                    # on a GPU: a user-side autograd function written against the module
    class UserFire(torch.autograd.Function):
        @staticmethod
        def forward(ctx, x):
            ctx.save_for_backward(x)
            return snnlib.fire_s_fp(x, 0.25, 0.5)
        @staticmethod
        def backward(ctx, g):
            (x,) = ctx.saved_tensors
            return snnlib.fire_bp(x.contiguous(), g.contiguous(), 0.25, 0.5, 1.0, 0.5)
    x = torch.full((3, 2, 4), 0.6, device="cuda", requires_grad=True)
    s = UserFire.apply(x)
    s.sum().backward()
    # u = 0.6, 0.6, 0.6 (each step fires and resets): spikes all one, every step inside the window
    assert bool((s == 1).all()) and x.grad.shape == x.shape and bool(torch.isfinite(x.grad).all())
print("route-a-ok")
"""


def _run_route_a(*extra):
    lib_dir = os.path.join(REPO, "snn_gpu_training_bptt_amd", "lib")
    proc = subprocess.run([sys.executable, "-c", ROUTE_A, lib_dir, *extra], capture_output=True, text=True,
                          cwd="/tmp", timeout=300)
    assert proc.returncode == 0 and "route-a-ok" in proc.stdout, proc.stderr[-2000:]


def test_module_binds_under_its_reference_name_from_the_lib_directory_alone():
    """`import snnlib` with nothing but the directory of the two shared objects on the path, every
    entry of the reference's binding table present (snnlib/cuda/snn.cpp:798-829)."""
    _run_route_a()


@pytest.mark.gpu
def test_user_autograd_function_against_the_bare_module():
    _run_route_a("gpu")


def test_layer_parameters_carry_the_reference_names_and_order():
    """A state dict saved from the reference's layers must load here: same parameter names, same
    registration order, same shapes (snnlib/example/snnlib_op.py:19-405; the running statistics are
    nn.Parameter objects there too)."""
    from snn_gpu_training_bptt_amd import snnlib_op as sop
    bn = ["weight_bn", "bias_bn", "running_var", "running_mean"]
    fc = ["weight_fc", "bias_fc"]
    conv = ["weight_conv", "bias_conv"]
    cases = [
        (sop.Fire(), [], {}),
        (sop.Bn(8, (0, 1, 3, 4)), bn, {"weight_bn": (8,), "running_var": (8,)}),
        (sop.BnFire(8, (0, 1)), bn, {"bias_bn": (8,), "running_mean": (8,)}),
        (sop.BnFireFc(4 * 4 * 8, 10, dim_bn=(0, 1, 3, 4), cin_bn=8), bn + fc,
         {"weight_bn": (8,), "weight_fc": (10, 128), "bias_fc": (10,)}),
        (sop.BnFireFc(16, 10, dim_bn=(0, 1)), bn + fc, {"weight_bn": (16,), "weight_fc": (10, 16)}),
        (sop.FireFc(16, 10), fc, {"weight_fc": (10, 16), "bias_fc": (10,)}),
        (sop.Fc(16, 10), fc, {"weight_fc": (10, 16)}),
        (sop.BnFireConv(8, 5, kernel_size=(3, 3), stride=(2, 2)), bn + conv,
         {"weight_bn": (8,), "weight_conv": (5, 8, 3, 3), "bias_conv": (5,)}),
        (sop.FireConv(8, 5, kernel_size=(1, 1), stride=(2, 2), padding=(0, 0)), conv, {"weight_conv": (5, 8, 1, 1)}),
        (sop.Conv(3, 5, kernel_size=(7, 7), stride=(2, 2), padding=(3, 3)), conv, {"weight_conv": (5, 3, 7, 7)}),
        (sop.BnDist(8, (0, 1, 3, 4)), bn, {"weight_bn": (8,)}),
        (sop.BnFireFcDist(7 * 7 * 8, 10, dim_bn=(0, 1, 3, 4), cin_bn=8), bn + fc, {"weight_fc": (10, 392)}),
        (sop.BnFireConvDist(8, 5), bn + conv, {"weight_conv": (5, 8, 3, 3)}),
    ]
    for layer, names, shapes in cases:
        what = type(layer).__name__
        assert [n for n, _ in layer.named_parameters()] == names, what
        assert list(layer.state_dict()) == names, what
        for n, shape in shapes.items():
            assert tuple(getattr(layer, n).shape) == shape, (what, n)
        assert list(layer.buffers()) == [], what
        if "weight_bn" in names:
            assert layer.train_bn is True and layer.factor is None, what
            assert bool((layer.weight_bn == 1).all()) and bool((layer.running_mean == 0).all()), what


def test_ctypes_helpers_reject_mismatched_buffers_before_any_launch():
    """The C ABI sees pointers only and sizes everything from ``spatial``; the ctypes helpers are the
    one place that can catch a buffer that is too small or of another type.  Host tensors suffice to
    show that the size checks come first (a consistent set of host tensors is then refused for
    living on the host)."""
    from snn_gpu_training_bptt_amd import lif_cabi
    x = torch.zeros(4, 2, 8, 3, 3)
    per_channel = torch.ones(8)
    with pytest.raises(ValueError, match="spike has shape"):
        lif_cabi.fire_s_fp_into(x, torch.zeros(4, 2, 8, 3, 2), 0.25, 0.5)
    with pytest.raises(ValueError, match="grad_spatial has dtype"):
        lif_cabi.fire_bp_into(x, x.clone(), x.double(), 0.25, 0.5, 1.0, 0.5)
    with pytest.raises(ValueError, match="mem has shape"):
        lif_cabi.fire_us_fp_into(x, x[:3].clone(), None, 0.25, 0.5)
    long_window = torch.zeros(1030, 1, 4)
    with pytest.raises(ValueError, match="needs a workspace"):
        lif_cabi.fire_bp_into(long_window, long_window.clone(), long_window.clone(), 0.25, 0.5, 1.0, 0.5)
    with pytest.raises(ValueError, match="workspace holds 16 bytes"):
        lif_cabi.fire_bp_into(long_window, long_window.clone(), long_window.clone(), 0.25, 0.5, 1.0, 0.5,
                              workspace=torch.zeros(16, dtype=torch.uint8))
    with pytest.raises(ValueError, match="ivar has 4 values"):
        lif_cabi.bn_fire_s_fp_into(x, per_channel, per_channel, per_channel, per_channel, torch.ones(4),
                                   x.clone(), 1e-5, 0.25, 0.5)
    with pytest.raises(ValueError, match="grad_weight has dtype"):
        lif_cabi.bn_fire_bp_into(x, per_channel, per_channel, per_channel, per_channel, x.clone(), x.clone(),
                                 per_channel.double(), per_channel, 0.25, 0.5, 1.0, 0.5,
                                 torch.zeros(1 << 16, dtype=torch.uint8))
    with pytest.raises(ValueError, match="workspace must be a uint8 tensor"):
        lif_cabi.bn_fire_bp_into(x, per_channel, per_channel, per_channel, per_channel, x.clone(), x.clone(),
                                 per_channel.clone(), per_channel.clone(), 0.25, 0.5, 1.0, 0.5,
                                 torch.zeros(1 << 16))
    with pytest.raises(ValueError, match="snnlif_bn_fire_bp needs"):
        lif_cabi.bn_fire_bp_into(x, per_channel, per_channel, per_channel, per_channel, x.clone(), x.clone(),
                                 per_channel.clone(), per_channel.clone(), 0.25, 0.5, 1.0, 0.5,
                                 torch.zeros(8, dtype=torch.uint8))
    with pytest.raises(ValueError, match="grad_xhatx has 3 values"):
        lif_cabi.bn_fire_bp_dist2_into(x, per_channel, per_channel, per_channel, per_channel, x.clone(),
                                       per_channel, torch.ones(3), x.clone(), 0.25, 0.5, 1.0, 0.5)
    # sizes and types all consistent: only now is the device looked at
    with pytest.raises(ValueError, match="device tensor required"):
        lif_cabi.fire_s_fp_into(x, x.clone(), 0.25, 0.5)


def test_batch_norm_workspace_follows_the_partial_sum_layout():
    """Two partial sums per wavefront of sweep 1 (ceil(HW/64) per plane) for planes of at least 32
    positions, two per neuron plus the split staging otherwise, plus two values per channel."""
    from snn_gpu_training_bptt_amd import lif_cabi
    f32, f64 = lif_cabi.DTYPE_F32, lif_cabi.DTYPE_F64
    need = lif_cabi.bn_fire_bp_workspace_bytes
    assert need(f32, 8, 64, 128, 1024) == 4 * (2 * 64 * 128 * 16 + 2 * 128)
    assert need(f32, 8, 4, 6, 49) == 4 * (2 * 4 * 6 * 1 + 2 * 6)
    assert need(f32, 8, 4, 6, 65) == 4 * (2 * 4 * 6 * 2 + 2 * 6)
    assert need(f64, 8, 4, 6, 65) == 2 * need(f32, 8, 4, 6, 65)
    # 31 positions: one lane per neuron; the [B, C*HW] partials are summed in S = min(B, 64, ...) batch slices
    assert need(f32, 8, 4, 6, 31) == 4 * (2 * 4 * 6 * 31 + 2 * 4 * 6 * 31 + 2 * 6)
    assert need(f32, 8, 64, 1024, 1) == 4 * (2 * 64 * 1024 + 2 * 64 * 1024 + 2 * 1024)
    # beyond 1024 steps: one boundary potential per 32-step segment and neuron on top
    assert need(f32, 1025, 4, 6, 65) == need(f32, 8, 4, 6, 65) + 4 * 33 * 4 * 6 * 65
    assert need(f32, 0, 4, 6, 31) == 0 and need(lif_cabi.DTYPE_BF16, 8, 4, 6, 31) == 0


def test_static_scratch_backward_refuses_oversized_shapes_without_a_gpu():
    """The size check of the entry point that allocates nothing comes before any device call, so it
    can be seen here with stand-in (aligned, never dereferenced) pointers."""
    from snn_gpu_training_bptt_amd import lif_cabi
    lib = lif_cabi.load()
    fake = [ctypes.c_void_p(4096)] * 9
    tail = (0.25, 0.5, 1.0, 0.5, None)
    f32 = lif_cabi.DTYPE_F32
    B, C, HW = 3 << 10, 1 << 10, 1       # 3 Mi neurons, one lane each: 24 MiB of partial sums
    assert lif_cabi.bn_fire_bp_workspace_bytes(f32, 4, B, C, HW) > lif_cabi.STATIC_SCRATCH_BYTES
    assert lib.snnlif_bn_fire_bp_static(*fake, f32, 4, B, C, HW, *tail) == lif_cabi.ERR_SCRATCH
    assert lib.snnlif_bn_fire_bp_static(*fake, lif_cabi.DTYPE_BF16, 4, 2, 8, 1, *tail) == lif_cabi.ERR_UNSUPPORTED
    assert lib.snnlif_bn_fire_bp_static(*[None] * 9, f32, 4, 2, 8, 1, *tail) == lif_cabi.ERR_ARG
    assert lib.snnlif_bn_fire_bp_static(*[None] * 9, f32, 0, 2, 8, 1, *tail) == lif_cabi.OK
    assert "SNNLIF_STATIC_SCRATCH_BYTES" in lif_cabi.strerror(lif_cabi.ERR_SCRATCH)


def test_no_kernel_is_scheduled_one_request_at_a_time():
    """hipcc keeps the order "all requests of a window, then the arithmetic" for most instantiations of
    the kernels but has fallen back to one request at a time, each followed by a full wait, for some
    (a third of the bandwidth; results stay correct, so no parity test can see it).  The check
    compiles every kernel to gfx950 assembly -- no GPU involved -- and counts loads that are directly
    followed by `s_waitcnt vmcnt(0)`, and scratch memory."""
    proc = subprocess.run([sys.executable, "-m", "snn_gpu_training_bptt_amd.schedule_check"],
                          capture_output=True, text=True, cwd=REPO)
    assert proc.returncode == 0, proc.stdout[-4000:] + proc.stderr[-2000:]
    assert "0 with an unexpected schedule or scratch memory" in proc.stdout
