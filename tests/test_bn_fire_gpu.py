"""Batch-norm + fire on the GPU.

Through the C ABI against the CPU oracle (``oracle/lif_oracle.c``, which follows the reference's
bn_fire kernels): spikes and the per-channel inverse standard deviation bit-exact (same operation
order; needs the device's fp32 divide and square root to be correctly rounded, which is part of what
is being tested); gradients within 1e-5 of the tensor's scale (the reference itself reduces the
per-channel sums in no defined order).

Through the PyTorch interface against autograd of ``batch_norm`` + the gold fire loop, the way the
reference's test_bn_fire.py compares its layer with gold_op.BnFire.
"""
import numpy as np
import pytest
import torch

from conftest import ALPHA, BETA, INTERVAL, THRESH, seed_clear_of_decision_points

pytestmark = pytest.mark.gpu
EPS = 1e-5


@pytest.fixture(scope="module")
def cabi():
    from snn_gpu_training_bptt_amd import lif_cabi
    lif_cabi.load()
    return lif_cabi


def rel_close(a, b, what, tol=1e-5):
    scale = np.abs(b).max() + 1e-12
    err = np.abs(a - b).max()
    assert err <= tol * scale, f"{what}: max abs err {err:.3e} vs scale {scale:.3e}"


def make(shape, seed):
    gen = torch.Generator().manual_seed(seed)
    C = shape[2]
    x = 0.5 + torch.randn(shape, generator=gen) * (0.5 + torch.rand((C,) + (1,) * (len(shape) - 3), generator=gen))
    g = torch.randn(shape, generator=gen)
    w = 0.5 + torch.rand(C, generator=gen)
    b = 0.2 * torch.randn(C, generator=gen)
    dims = (0, 1) + tuple(range(3, len(shape)))
    var, mean = torch.var_mean(x, dim=dims, unbiased=False)
    return x, g, w, b, var, mean


SHAPES = [
    (6, 2, 8),                # the reference test's fc shape
    (6, 2, 8, 8, 8),          # the reference test's conv shape
    (8, 16, 32, 16, 16),      # HW = 256
    (4, 5, 7, 7, 7),          # HW = 49: one partly idle wavefront per plane
    (6, 3, 6, 14, 14),        # HW = 196: four wavefronts per plane, the last with 4 active lanes
    (5, 2, 3, 4, 8),          # HW = 32: the smallest plane-aligned case
    (5, 2, 9, 31),            # HW = 31: just below it, one lane per neuron
    (13, 3, 20, 5, 3),        # window without an instantiation of its own
    (32, 2, 16, 4, 4),
    (33, 2, 6, 8, 8),         # first window beyond the registers: two segments, the second of one step
    (64, 2, 8, 4, 8),         # two full segments, plane-aligned wavefronts
    (70, 2, 5, 31),           # three segments, one lane per neuron
    (100, 3, 20),             # fully connected shape, four segments
    (1024, 1, 4, 6, 6),       # the longest window with its boundary values in LDS: 32 segments
    (1030, 1, 4, 6, 6),       # beyond it: boundary values in the workspace (sweep 1) and in gx rows (sweep 2)
    (1100, 2, 20),            # the same, fully connected: one lane per neuron
    (1057, 1, 3, 8, 8),       # 34 segments, the last of one step, plane-aligned wavefronts
    (8, 64, 1024),            # fully connected, many channels: 64 batch slices of one entry each
    (6, 200, 4, 3, 3),        # HW = 9, few channels, large batch: 64 batch slices of 4 entries, 9 positions per channel
    (8, 32, 128, 32, 32),     # few channels, many positions: 16 wavefront partials per plane
]


@pytest.mark.parametrize("shape", SHAPES)
def test_bn_fire_against_oracle(cabi, shape):
    from oracle import c_oracle
    x, g, w, b, var, mean = make(shape, seed=31)
    T, B, C = shape[:3]
    HW = int(np.prod(shape[3:])) if len(shape) > 3 else 1
    dev = lambda t: t.cuda()
    xd, gd, wd, bd, vd, md = map(dev, (x, g, w, b, var, mean))
    ivar = torch.empty_like(vd)
    spike = torch.empty_like(xd)
    cabi.bn_fire_s_fp_into(xd, wd, bd, vd, md, ivar, spike, EPS, ALPHA, THRESH)
    # the cache hint selects between two instantiations of the forward: same bits from both
    for keep in (True, False):
        ivar_h, spike_h = torch.empty_like(vd), torch.empty_like(xd)
        cabi.bn_fire_s_fp_into(xd, wd, bd, vd, md, ivar_h, spike_h, EPS, ALPHA, THRESH, keep_spatial=keep)
        assert torch.equal(ivar_h, ivar) and torch.equal(spike_h, spike), f"hint keep={keep} changes the result"
    gx, gw, gb = torch.empty_like(xd), torch.empty_like(wd), torch.empty_like(wd)
    ws = torch.empty(cabi.bn_fire_bp_workspace_bytes(cabi.DTYPE_F32, T, B, C, HW), dtype=torch.uint8, device="cuda")
    cabi.bn_fire_bp_into(xd, wd, bd, ivar, md, gd, gx, gw, gb, ALPHA, THRESH, BETA, INTERVAL, ws)
    torch.cuda.synchronize()

    ivar_o, _, spike_o = c_oracle.bn_fire_forward(x.numpy(), w.numpy(), b.numpy(), var.numpy(), mean.numpy(), EPS, ALPHA, THRESH)
    gx_o, gw_o, gb_o = c_oracle.bn_fire_backward(x.numpy(), w.numpy(), b.numpy(), ivar_o, mean.numpy(), g.numpy(),
                                                 ALPHA, THRESH, BETA, INTERVAL)
    assert np.array_equal(ivar.cpu().numpy(), ivar_o), "inverse standard deviation differs"
    assert np.array_equal(spike.cpu().numpy(), spike_o), "spikes differ from the oracle"
    rel_close(gb.cpu().numpy(), gb_o, "bias gradient")
    rel_close(gw.cpu().numpy(), gw_o, "weight gradient")
    rel_close(gx.cpu().numpy(), gx_o, "input-current gradient")

    # reproducibility: the reduction order is fixed
    gx2, gw2, gb2 = torch.empty_like(xd), torch.empty_like(wd), torch.empty_like(wd)
    cabi.bn_fire_bp_into(xd, wd, bd, ivar, md, gd, gx2, gw2, gb2, ALPHA, THRESH, BETA, INTERVAL, ws)
    assert torch.equal(gx, gx2) and torch.equal(gw, gw2) and torch.equal(gb, gb2)


def test_identity_statistics_reduce_to_plain_fire(cabi):
    """mean 0, var 1-eps, weight 1, bias 0 -> scale == 1 exactly and the spikes are those of fire."""
    gen = torch.Generator().manual_seed(32)
    x = (0.5 + torch.randn((8, 4, 16, 8, 8), generator=gen)).cuda()
    C = 16
    one = torch.ones(C, device="cuda")
    zero = torch.zeros(C, device="cuda")
    var = torch.full((C,), 1.0 - EPS, device="cuda")
    assert float(var[0] + EPS) == 1.0
    ivar, spike = torch.empty(C, device="cuda"), torch.empty_like(x)
    cabi.bn_fire_s_fp_into(x, one, zero, var, zero, ivar, spike, EPS, ALPHA, THRESH)
    plain = torch.empty_like(x)
    cabi.fire_s_fp_into(x, plain, ALPHA, THRESH)
    assert torch.equal(spike, plain)
    assert torch.equal(ivar, one)


@pytest.mark.parametrize("shape,dim_bn", [((6, 2, 8), (0, 1)), ((6, 2, 8, 8, 8), (0, 1, 3, 4)), ((8, 8, 32, 16, 16), (0, 1, 3, 4))])
@pytest.mark.parametrize("train_bn", [True, False])
def test_bn_fire_layer_like_reference_test(shape, dim_bn, train_bn):
    from oracle import gold_fire
    from snn_gpu_training_bptt_amd import snnlib_func as sf
    from snn_gpu_training_bptt_amd import snnlib_op as sop
    saved = (sf.alpha, sf.thresh, sf.beta, sf.interval)
    sf.alpha, sf.thresh, sf.beta, sf.interval = ALPHA, THRESH, BETA, INTERVAL
    try:
        C = shape[2]

        def draw(seed):
            torch.manual_seed(seed)
            return (torch.randn(shape), torch.randn(C).abs() + 0.3, torch.randn(C) * 0.3, torch.rand(C) + 0.5,
                    torch.randn(C) * 0.1)

        def potentials(seed):
            x_, w_, b_, rv_, rm_ = (t.cuda() for t in draw(seed))
            with torch.no_grad():
                return gold_fire.gold_bn_fire(x_, w_, b_, rm_, rv_, train_bn, EPS, ALPHA, THRESH, BETA, INTERVAL)[0]

        x_cpu, w0, b0, rv, rm = draw(seed_clear_of_decision_points(potentials, range(33, 4033, 100)))
        labels = torch.tensor([1, 0] + [0] * (shape[1] - 2))[: shape[1]].cuda()
        crit = torch.nn.CrossEntropyLoss()

        layer = sop.BnFire(C, dim_bn, EPS).cuda()
        layer.weight_bn, layer.bias_bn = torch.nn.Parameter(w0.clone().cuda()), torch.nn.Parameter(b0.clone().cuda())
        layer.running_var, layer.running_mean = torch.nn.Parameter(rv.clone().cuda()), torch.nn.Parameter(rm.clone().cuda())
        layer.train_bn = train_bn
        x = x_cpu.cuda().requires_grad_(True)
        spikes = layer(x)
        crit(spikes.view(shape[0], shape[1], -1).mean(dim=0), labels).backward()

        xg = x_cpu.cuda().requires_grad_(True)
        wg, bg = w0.clone().cuda().requires_grad_(True), b0.clone().cuda().requires_grad_(True)
        run_m, run_v = rm.clone().cuda(), rv.clone().cuda()
        _, s_ref = gold_fire.gold_bn_fire(xg, wg, bg, run_m, run_v, train_bn, EPS, ALPHA, THRESH, BETA, INTERVAL)
        crit(s_ref.view(shape[0], shape[1], -1).mean(dim=0), labels).backward()

        # the inputs keep every membrane potential clear of the threshold and the window edges, so the
        # two sides must agree on every spike, and then on the gradients
        assert torch.equal(spikes.detach(), s_ref.detach()), "spikes differ from the gold layer"
        rel = lambda a, b_, what: rel_close(a.cpu().numpy(), b_.cpu().numpy(), what, tol=2e-5)
        rel(layer.weight_bn.grad, wg.grad, "weight gradient")
        rel(layer.bias_bn.grad, bg.grad, "bias gradient")
        if train_bn:
            rel(x.grad, xg.grad, "input-current gradient")
        if train_bn:
            # running statistics follow nn.BatchNorm's update (momentum 0.1, unbiased variance)
            torch.testing.assert_close(layer.running_mean.detach(), run_m, rtol=1e-5, atol=1e-6)
            torch.testing.assert_close(layer.running_var.detach(), run_v, rtol=1e-5, atol=1e-6)
    finally:
        sf.alpha, sf.thresh, sf.beta, sf.interval = saved


@pytest.mark.parametrize("seed", [7, 8, 9])
def test_bn_fire_layer_on_unscreened_inputs(seed):
    """Inputs drawn without looking at where the membrane potentials fall: the layer (batch statistics
    from the hand-written reduction) and the gold layer (torch's batch norm in training mode) then differ
    in the last bits of mean and variance, and a potential that sits within those bits of the threshold
    may come out on either side.  On 1.6 million neuron-steps at most a handful may: the mismatch
    fraction is bounded, not required to be zero, and the parameter gradients stay close."""
    from oracle import gold_fire
    from snn_gpu_training_bptt_amd import snnlib_func as sf
    from snn_gpu_training_bptt_amd import snnlib_op as sop
    saved = (sf.alpha, sf.thresh, sf.beta, sf.interval)
    sf.alpha, sf.thresh, sf.beta, sf.interval = ALPHA, THRESH, BETA, INTERVAL
    try:
        shape, C = (6, 16, 64, 16, 16), 64
        torch.manual_seed(seed)
        x0, w0, b0, g0 = torch.randn(shape), torch.rand(C) + 0.5, torch.randn(C) * 0.2, torch.randn(shape)
        layer = sop.BnFire(C, (0, 1, 3, 4), EPS).cuda()
        with torch.no_grad():
            layer.weight_bn.copy_(w0)
            layer.bias_bn.copy_(b0)
        x = x0.cuda().requires_grad_(True)
        spikes = layer(x)
        spikes.backward(g0.cuda())
        xr = x0.cuda().requires_grad_(True)
        wr, br = w0.cuda().requires_grad_(True), b0.cuda().requires_grad_(True)
        _, s_ref = gold_fire.gold_bn_fire(xr, wr, br, None, None, True, EPS, ALPHA, THRESH, BETA, INTERVAL)
        s_ref.backward(g0.cuda())
        mismatch = float((spikes != s_ref).float().mean())
        assert mismatch <= 2e-5, f"{mismatch:.2e} of the spikes differ from the gold layer"
        # a flipped spike moves its neuron's gradient terms by order one; with at most ~30 of them among
        # 1.6 million the per-channel sums move by far less than 1e-3 of their scale
        for got, want, what in ((layer.weight_bn.grad, wr.grad, "weight"), (layer.bias_bn.grad, br.grad, "bias")):
            rel_close(got.cpu().numpy(), want.cpu().numpy(), what + " gradient", tol=1e-3)
        differing = float(((x.grad - xr.grad).abs() > 1e-4 * float(xr.grad.abs().max())).float().mean())
        assert differing <= 1e-3, f"{differing:.2e} of the input-gradient entries differ"
    finally:
        sf.alpha, sf.thresh, sf.beta, sf.interval = saved


def test_bn_fire_layer_with_a_window_beyond_1024_steps():
    """The layer accepts any window length in both directions (the reference's bn_fire_bp has no limit
    either, snnlib/cuda/snn_kernel_bp.cu:680-750): forward and backward of a 1030-step window against
    autograd through batch_norm + the gold fire loop."""
    from oracle import gold_fire
    from snn_gpu_training_bptt_amd import snnlib_func as sf
    from snn_gpu_training_bptt_amd import snnlib_op as sop
    saved = (sf.alpha, sf.thresh, sf.beta, sf.interval)
    sf.alpha, sf.thresh, sf.beta, sf.interval = ALPHA, THRESH, BETA, INTERVAL
    try:
        shape, C = (1030, 2, 4, 3), 4

        def draw(seed):
            torch.manual_seed(seed)
            return torch.randn(shape), torch.rand(C) + 0.5, torch.randn(C) * 0.2, torch.randn(shape)

        def potentials(seed):
            x_, w_, b_, _ = (t.cuda() for t in draw(seed))
            with torch.no_grad():
                return gold_fire.gold_bn_fire(x_, w_, b_, None, None, True, EPS, ALPHA, THRESH, BETA, INTERVAL)[0]

        x0, w0, b0, g0 = draw(seed_clear_of_decision_points(potentials, range(37, 4037, 100)))
        layer = sop.BnFire(C, (0, 1, 3), EPS).cuda()
        with torch.no_grad():
            layer.weight_bn.copy_(w0)
            layer.bias_bn.copy_(b0)
        x = x0.cuda().requires_grad_(True)
        spikes = layer(x)
        spikes.backward(g0.cuda())
        xr = x0.cuda().requires_grad_(True)
        wr, br = w0.cuda().requires_grad_(True), b0.cuda().requires_grad_(True)
        _, s_ref = gold_fire.gold_bn_fire(xr, wr, br, None, None, True, EPS, ALPHA, THRESH, BETA, INTERVAL)
        s_ref.backward(g0.cuda())
        assert torch.equal(spikes, s_ref), "spikes differ from the gold layer"
        for got, want, what in ((x.grad, xr.grad, "input"), (layer.weight_bn.grad, wr.grad, "weight"),
                                (layer.bias_bn.grad, br.grad, "bias")):
            rel_close(got.cpu().numpy(), want.cpu().numpy(), what + " gradient", tol=5e-5)
    finally:
        sf.alpha, sf.thresh, sf.beta, sf.interval = saved


def test_bn_fire_errors(cabi):
    import snnlib
    x = torch.zeros(4, 2, 8, device="cuda")
    p = torch.ones(8, device="cuda")
    with pytest.raises(RuntimeError, match="float32 and float64"):
        snnlib.bn_fire_s_fp(x.bfloat16(), p.bfloat16(), p.bfloat16(), p.bfloat16(), p.bfloat16(), EPS, ALPHA, THRESH)
    with pytest.raises(RuntimeError, match="dtype of spatial"):
        snnlib.bn_fire_s_fp(x.double(), p, p, p, p, EPS, ALPHA, THRESH)
    with pytest.raises(RuntimeError, match="per channel"):
        snnlib.bn_fire_s_fp(x, p[:4], p, p, p, EPS, ALPHA, THRESH)
    lib = cabi.load()
    # windows beyond 1024 steps also keep their segment boundaries in the workspace
    f32 = cabi.DTYPE_F32
    assert (cabi.bn_fire_bp_workspace_bytes(f32, 1025, 2, 8, 1) - cabi.bn_fire_bp_workspace_bytes(f32, 1024, 2, 8, 1)
            == 4 * 33 * 16)
    rc = lib.snnlif_bn_fire_bp(x.data_ptr(), p.data_ptr(), p.data_ptr(), p.data_ptr(), p.data_ptr(), x.data_ptr(),
                               x.data_ptr(), p.data_ptr(), p.data_ptr(), 0, 4, 2, 8, 1, ALPHA, THRESH, BETA, INTERVAL,
                               None, 0, None)
    assert rc == cabi.ERR_WORKSPACE
    torch.cuda.synchronize()


@pytest.mark.parametrize("shape", [(6, 2, 8), (6, 2, 8, 8, 8), (8, 8, 32, 16, 16), (4, 5, 7, 7, 7), (5, 2, 9, 31),
                                   (13, 3, 20, 5, 3), (32, 2, 16, 4, 4), (40, 2, 6, 8, 8), (8, 64, 256)])
def test_bn_fire_double_precision_against_oracle(cabi, shape):
    """float64 storage and arithmetic: spikes and the inverse standard deviation bit-identical to the
    fp64 oracle loops, gradients to double rounding level; the two sharded halves equal the unsplit
    backward bit for bit."""
    from oracle import c_oracle
    x, g, w, b, var, mean = (t.double() for t in make(shape, seed=35))
    dims = (0, 1) + tuple(range(3, len(shape)))
    var, mean = torch.var_mean(x, dim=dims, unbiased=False)
    T, B, C = shape[:3]
    HW = int(np.prod(shape[3:])) if len(shape) > 3 else 1
    xd, gd, wd, bd, vd, md = (t.cuda() for t in (x, g, w, b, var, mean))
    ivar, spike = torch.empty_like(vd), torch.empty_like(xd)
    cabi.bn_fire_s_fp_into(xd, wd, bd, vd, md, ivar, spike, EPS, ALPHA, THRESH)
    again = torch.empty_like(xd)
    cabi.bn_fire_s_recompute_into(xd, wd, bd, ivar, md, again, ALPHA, THRESH)
    for keep in (True, False):
        hinted = torch.empty_like(xd)
        cabi.bn_fire_s_recompute_into(xd, wd, bd, ivar, md, hinted, ALPHA, THRESH, keep_spatial=keep)
        assert torch.equal(hinted, again)
    gx, gw, gb = torch.empty_like(xd), torch.empty_like(wd), torch.empty_like(wd)
    ws_bytes = cabi.bn_fire_bp_workspace_bytes(cabi.DTYPE_F64, T, B, C, HW)
    assert ws_bytes == 2 * cabi.bn_fire_bp_workspace_bytes(cabi.DTYPE_F32, T, B, C, HW)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
    cabi.bn_fire_bp_into(xd, wd, bd, ivar, md, gd, gx, gw, gb, ALPHA, THRESH, BETA, INTERVAL, ws)
    m1, m2, gw2, gb2 = (torch.empty_like(wd) for _ in range(4))
    cabi.bn_fire_bp_dist1_into(xd, wd, bd, ivar, md, gd, m1, m2, gw2, gb2, ALPHA, THRESH, BETA, INTERVAL, ws)
    gx2 = torch.empty_like(xd)
    cabi.bn_fire_bp_dist2_into(xd, wd, bd, ivar, md, gd, m1, m2, gx2, ALPHA, THRESH, BETA, INTERVAL)
    torch.cuda.synchronize()

    n = lambda t: t.numpy()
    ivar_o, _, spike_o = c_oracle.bn_fire_forward(n(x), n(w), n(b), n(var), n(mean), EPS, ALPHA, THRESH)
    gx_o, gw_o, gb_o = c_oracle.bn_fire_backward(n(x), n(w), n(b), ivar_o, n(mean), n(g), ALPHA, THRESH, BETA, INTERVAL)
    assert np.array_equal(ivar.cpu().numpy(), ivar_o), "inverse standard deviation differs"
    assert np.array_equal(spike.cpu().numpy(), spike_o), "spikes differ from the oracle"
    # recomputed from weight * ivar instead of weight / sqrt(var + eps): a potential that sits within
    # rounding of the threshold may land on the other side
    assert (again != spike).float().mean().item() < 1e-4
    rel_close(gb.cpu().numpy(), gb_o, "bias gradient", tol=1e-11)
    rel_close(gw.cpu().numpy(), gw_o, "weight gradient", tol=1e-11)
    rel_close(gx.cpu().numpy(), gx_o, "input-current gradient", tol=1e-11)
    assert torch.equal(gx, gx2) and torch.equal(gw, gw2) and torch.equal(gb, gb2)


def test_bn_fire_layer_in_double_precision():
    """The layer with float64 parameters and input against autograd in double through batch_norm +
    the gold fire loop."""
    from oracle import gold_fire
    from snn_gpu_training_bptt_amd import snnlib_func as sf
    from snn_gpu_training_bptt_amd import snnlib_op as sop
    saved = (sf.alpha, sf.thresh, sf.beta, sf.interval)
    sf.alpha, sf.thresh, sf.beta, sf.interval = ALPHA, THRESH, BETA, INTERVAL
    try:
        shape, dim_bn, C = (6, 4, 8, 8, 8), (0, 1, 3, 4), 8
        f = lambda v: float(np.float32(v))       # hyper-parameters reach the kernels as C floats

        def draw(seed):
            torch.manual_seed(seed)
            return (torch.rand(C, dtype=torch.float64) + 0.5, torch.randn(C, dtype=torch.float64) * 0.2,
                    torch.randn(shape, dtype=torch.float64), torch.randn(shape, dtype=torch.float64))

        def potentials(seed):
            w_, b_, x_, _ = (t.cuda() for t in draw(seed))
            with torch.no_grad():
                return gold_fire.gold_bn_fire(x_, w_, b_, None, None, True, f(EPS), ALPHA, THRESH, BETA, INTERVAL)[0]

        w0, b0, x0, g0 = draw(seed_clear_of_decision_points(potentials, range(36, 4036, 100), margin=1e-9))
        layer = sop.BnFire(C, dim_bn, EPS).double().cuda()
        with torch.no_grad():
            layer.weight_bn.copy_(w0)
            layer.bias_bn.copy_(b0)
        x = x0.cuda().requires_grad_(True)
        g = g0.cuda()
        spikes = layer(x)
        assert spikes.dtype == torch.float64
        spikes.backward(g)
        xr = x.detach().clone().requires_grad_(True)
        wr = layer.weight_bn.detach().clone().requires_grad_(True)
        br = layer.bias_bn.detach().clone().requires_grad_(True)
        _, s_ref = gold_fire.gold_bn_fire(xr, wr, br, None, None, True, f(EPS), ALPHA, THRESH, BETA, INTERVAL)
        s_ref.backward(g)
        assert torch.equal(spikes, s_ref), "spikes differ from the gold layer"
        for got, want, what in ((x.grad, xr.grad, "input"), (layer.weight_bn.grad, wr.grad, "weight"),
                                (layer.bias_bn.grad, br.grad, "bias")):
            rel_close(got.cpu().numpy(), want.cpu().numpy(), what + " gradient", tol=1e-9)
    finally:
        sf.alpha, sf.thresh, sf.beta, sf.interval = saved
