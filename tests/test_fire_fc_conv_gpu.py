"""``FireFc`` / ``FireConv`` (fire kernels + rocBLAS / MIOpen through ATen) against the gold
restatement of the reference's per-time-step modules (snnlib/example/gold_op.py:113-179 with
``fire=True``), in the manner of the reference's test_fire_fc.py / test_fire_conv.py: same inputs,
same parameters, loss = cross-entropy on the time-averaged, flattened output.

The spikes entering the linear / convolution are bit-exact, so differences can only come from the
dense library calls seeing ``T*B`` rows at once here and ``B`` rows per call in the gold loop:
tolerance 1e-5 relative to the tensor's scale for outputs and gradients.
"""
import pytest
import torch

from conftest import ALPHA, BETA, INTERVAL, THRESH

pytestmark = pytest.mark.gpu


@pytest.fixture()
def mods():
    from oracle import gold_fire
    from snn_gpu_training_bptt_amd import snnlib_func as sf
    from snn_gpu_training_bptt_amd import snnlib_op as sop
    saved = (sf.alpha, sf.thresh, sf.beta, sf.interval)
    sf.alpha, sf.thresh, sf.beta, sf.interval = ALPHA, THRESH, BETA, INTERVAL
    yield sf, sop, gold_fire
    sf.alpha, sf.thresh, sf.beta, sf.interval = saved


def close(a, b, what):
    scale = b.abs().max().item() + 1e-12
    err = (a - b).abs().max().item()
    assert err <= 1e-5 * scale, f"{what}: max abs err {err:.3e} vs scale {scale:.3e}"


@pytest.mark.parametrize("shape,cout", [((6, 2, 8), 8), ((6, 2, 8, 8, 8), 8), ((8, 16, 1024), 10), ((5, 3, 16, 4, 4), 33)])
def test_fire_fc_matches_gold(mods, shape, cout):
    sf, sop, gold = mods
    torch.manual_seed(21)
    x_cpu = 0.5 + torch.randn(shape)
    cin = x_cpu[0, 0].numel()
    layer = sop.FireFc(cin, cout).cuda()
    with torch.no_grad():
        layer.bias_fc.normal_()
    labels = torch.randint(0, cout, (shape[1],)).cuda()

    x = x_cpu.cuda().requires_grad_(True)
    out = layer(x)
    assert out.shape == (shape[0], shape[1], cout)
    torch.nn.functional.cross_entropy(out.mean(dim=0), labels).backward()

    xg = x_cpu.cuda().requires_grad_(True)
    w = layer.weight_fc.detach().clone().requires_grad_(True)
    b = layer.bias_fc.detach().clone().requires_grad_(True)
    ref = gold.gold_fire_fc(xg, w, b, ALPHA, THRESH, BETA, INTERVAL)
    torch.nn.functional.cross_entropy(ref.mean(dim=0), labels).backward()

    close(out.detach(), ref.detach(), "fc output")
    close(x.grad, xg.grad, "input-current gradient")
    close(layer.weight_fc.grad, w.grad, "weight gradient")
    close(layer.bias_fc.grad, b.grad, "bias gradient")


@pytest.mark.parametrize("shape,cout,stride,padding,bias", [
    ((6, 2, 8, 8, 8), 8, (1, 1), (1, 1), True),      # the reference test's conv shape
    ((4, 3, 16, 12, 10), 24, (2, 2), (1, 1), True),
    ((8, 4, 32, 16, 16), 32, (1, 1), (0, 0), False),
])
def test_fire_conv_matches_gold(mods, shape, cout, stride, padding, bias):
    sf, sop, gold = mods
    torch.manual_seed(22)
    x_cpu = 0.5 + torch.randn(shape)
    layer = sop.FireConv(shape[2], cout, (3, 3), stride, padding, if_bias_conv=bias).cuda()

    x = x_cpu.cuda().requires_grad_(True)
    out = layer(x)
    g_out = torch.randn_like(out)
    out.backward(g_out)

    xg = x_cpu.cuda().requires_grad_(True)
    w = layer.weight_conv.detach().clone().requires_grad_(True)
    b = layer.bias_conv.detach().clone().requires_grad_(True)
    ref = gold.gold_fire_conv(xg, w, b, stride, padding, ALPHA, THRESH, BETA, INTERVAL)
    ref.backward(g_out)

    assert out.shape == ref.shape
    close(out.detach(), ref.detach(), "conv output")
    close(x.grad, xg.grad, "input-current gradient")
    close(layer.weight_conv.grad, w.grad, "weight gradient")
    if bias:
        close(layer.bias_conv.grad, b.grad, "bias gradient")
    else:
        assert layer.bias_conv.grad is None


def test_layer_surfaces(mods):
    sf, sop, _ = mods
    fc = sop.FireFc(12, 5)
    assert [n for n, _ in fc.named_parameters()] == ["weight_fc", "bias_fc"]
    assert fc.weight_fc.shape == (5, 12) and fc.bias_fc.abs().sum().item() == 0.0
    conv = sop.FireConv(4, 6)
    assert [n for n, _ in conv.named_parameters()] == ["weight_conv", "bias_conv"]
    assert conv.weight_conv.shape == (6, 4, 3, 3)
    assert (conv.stride, conv.padding, conv.if_bias_conv, conv.cin) == ((1, 1), (1, 1), True, 4)
    assert sf.fire_fc_func == sf.FireFcFunc.apply and sf.fire_conv_func == sf.FireConvFunc.apply


@pytest.mark.parametrize("benchmark,deterministic", [(True, False), (False, True), (True, True)])
def test_convolution_flags_reach_the_library_for_the_call_only(mods, benchmark, deterministic):
    """The reference forwards `benchmark` / `deterministic` to the convolution with every call
    (snn_kernel_fp.cu:404-407).  Here they become the process-wide settings PyTorch-ROCm hands to MIOpen
    while the dense call runs and the previous settings come back afterwards, whichever way they were
    set; the results agree with the default call to the dense library's accuracy."""
    from snn_gpu_training_bptt_amd._loader import load_snnlib
    snnlib = load_snnlib()
    torch.manual_seed(5)
    x = (0.5 + torch.randn(4, 2, 8, 8, 8)).cuda()
    w = torch.randn(6, 8, 3, 3).cuda() * 0.2
    b = torch.randn(6).cuda()
    g = torch.randn(4, 2, 6, 8, 8).cuda()
    saved = (torch.backends.cudnn.benchmark, torch.backends.cudnn.deterministic)
    try:
        for before in ((False, False), (True, True)):
            torch.backends.cudnn.benchmark, torch.backends.cudnn.deterministic = before
            ref = snnlib.fire_conv_fp(x, w, b, (1, 1), (1, 1), (1, 1), 1, False, False, ALPHA, THRESH)
            out = snnlib.fire_conv_fp(x, w, b, (1, 1), (1, 1), (1, 1), 1, benchmark, deterministic, ALPHA, THRESH)
            assert (torch.backends.cudnn.benchmark, torch.backends.cudnn.deterministic) == before
            close(out, ref, "fire_conv_fp under the flags")
            gref = snnlib.fire_conv_bp(x, g, w, (1, 1), (1, 1), (1, 1), 1, False, False, True, (0, 1, 3, 4),
                                       ALPHA, THRESH, BETA, INTERVAL)
            gout = snnlib.fire_conv_bp(x, g, w, (1, 1), (1, 1), (1, 1), 1, benchmark, deterministic, True,
                                       (0, 1, 3, 4), ALPHA, THRESH, BETA, INTERVAL)
            assert (torch.backends.cudnn.benchmark, torch.backends.cudnn.deterministic) == before
            for a, r, what in zip(gout, gref, ("grad_spatial", "grad_weight", "grad_bias")):
                close(a, r, what)
    finally:
        torch.backends.cudnn.benchmark, torch.backends.cudnn.deterministic = saved
