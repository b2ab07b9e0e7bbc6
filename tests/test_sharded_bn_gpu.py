"""The sharded-batch ("dist") halves of the batch-norm layers, on one GPU.

What the reference runs on either side of its all-reduce (snnlib/example/snnlib_func.py:261-379,
snnlib/cuda/snn_kernel_bp.cu:348-425, 753-854, 966-1061, 1265-1340) is checked here without any
process group:

* ``dist1`` followed by ``dist2`` on one shard is the unsplit backward, bit for bit;
* two shards of one batch, handled one after the other on the same GPU with the averaging of the
  two ``[C]`` vectors done by hand where the all-reduce would be, give the gradients of the unsplit
  backward over the whole batch (which the other test files check against the CPU oracle);
* the ``*Dist`` modules, with ``torch.distributed`` replaced by a one-rank stand-in, equal the
  single-GPU modules given the same statistics.
"""
import numpy as np
import pytest
import torch

from conftest import ALPHA, BETA, INTERVAL, THRESH

pytestmark = pytest.mark.gpu
EPS = 1e-5


@pytest.fixture(scope="module")
def cabi():
    from snn_gpu_training_bptt_amd import lif_cabi
    lif_cabi.load()
    return lif_cabi


@pytest.fixture()
def hyper():
    from snn_gpu_training_bptt_amd import snnlib_func as sf
    saved = (sf.alpha, sf.thresh, sf.beta, sf.interval)
    sf.alpha, sf.thresh, sf.beta, sf.interval = ALPHA, THRESH, BETA, INTERVAL
    yield sf
    sf.alpha, sf.thresh, sf.beta, sf.interval = saved


def rel_close(a, b, what, tol=1e-5):
    a, b = a.detach().cpu().numpy(), b.detach().cpu().numpy()
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
    return [t.cuda() for t in (x, g, w, b, var, mean)]


def dims_of(shape):
    T, B, C = shape[:3]
    HW = int(np.prod(shape[3:])) if len(shape) > 3 else 1
    return T, B, C, HW


SHAPES = [(6, 4, 8), (6, 4, 8, 8, 8), (8, 6, 32, 16, 16), (4, 6, 7, 7, 7), (13, 2, 20, 5, 3), (8, 16, 1024),
          (40, 2, 6, 8, 8), (1030, 2, 4, 6, 6), (1100, 2, 12)]


@pytest.mark.parametrize("shape", SHAPES)
def test_halves_back_to_back_equal_the_unsplit_backward(cabi, shape):
    x, g, w, b, var, mean = make(shape, seed=41)
    T, B, C, HW = dims_of(shape)
    ivar, spike = torch.empty_like(var), torch.empty_like(x)
    cabi.bn_fire_s_fp_into(x, w, b, var, mean, ivar, spike, EPS, ALPHA, THRESH)
    ws = torch.empty(cabi.bn_fire_bp_workspace_bytes(cabi.DTYPE_F32, T, B, C, HW), dtype=torch.uint8, device="cuda")
    gx, gw, gb = torch.empty_like(x), torch.empty_like(w), torch.empty_like(w)
    cabi.bn_fire_bp_into(x, w, b, ivar, mean, g, gx, gw, gb, ALPHA, THRESH, BETA, INTERVAL, ws)

    m1, m2, gw2, gb2 = (torch.empty_like(w) for _ in range(4))
    cabi.bn_fire_bp_dist1_into(x, w, b, ivar, mean, g, m1, m2, gw2, gb2, ALPHA, THRESH, BETA, INTERVAL, ws)
    gx2 = torch.empty_like(x)
    cabi.bn_fire_bp_dist2_into(x, w, b, ivar, mean, g, m1, m2, gx2, ALPHA, THRESH, BETA, INTERVAL)
    torch.cuda.synchronize()
    assert torch.equal(gw, gw2) and torch.equal(gb, gb2)
    assert torch.equal(gx, gx2)
    # the two means are weight * sum / count (to the last bit or so: the device divides exactly,
    # torch may multiply by the reciprocal)
    count = float(T * B * HW)
    rel_close(m1, (gb * w) / count, "mean of gy*weight", tol=1e-6)
    rel_close(m2, (gw * w) / count, "mean of gy*weight*xhat", tol=1e-6)


@pytest.mark.parametrize("shape", SHAPES)
def test_two_shards_on_one_gpu_reproduce_the_whole_batch(cabi, shape):
    """Rank r holds x[:, r*B/2:(r+1)*B/2]; the statistics are those of the whole batch."""
    x, g, w, b, var, mean = make(shape, seed=43)
    T, B, C, HW = dims_of(shape)
    ivar, spike = torch.empty_like(var), torch.empty_like(x)
    cabi.bn_fire_s_fp_into(x, w, b, var, mean, ivar, spike, EPS, ALPHA, THRESH)
    ws = torch.empty(cabi.bn_fire_bp_workspace_bytes(cabi.DTYPE_F32, T, B, C, HW), dtype=torch.uint8, device="cuda")
    gx, gw, gb = torch.empty_like(x), torch.empty_like(w), torch.empty_like(w)
    cabi.bn_fire_bp_into(x, w, b, ivar, mean, g, gx, gw, gb, ALPHA, THRESH, BETA, INTERVAL, ws)

    half = B // 2
    shards = [(x[:, r * half:(r + 1) * half].contiguous(), g[:, r * half:(r + 1) * half].contiguous())
              for r in range(2)]
    local = []
    for xs, gs in shards:
        iv_s, sp_s = torch.empty_like(var), torch.empty_like(xs)
        cabi.bn_fire_s_fp_into(xs, w, b, var, mean, iv_s, sp_s, EPS, ALPHA, THRESH)
        assert torch.equal(iv_s, ivar)
        out = [torch.empty_like(w) for _ in range(4)]
        cabi.bn_fire_bp_dist1_into(xs, w, b, ivar, mean, gs, *out, ALPHA, THRESH, BETA, INTERVAL, ws)
        local.append((sp_s, out))
    assert torch.equal(torch.cat([l[0] for l in local], dim=1), spike)
    # where the all-reduce would be: sum over ranks, divide by the world size
    gxhat = (local[0][1][0] + local[1][1][0]) / 2
    gxhatx = (local[0][1][1] + local[1][1][1]) / 2
    parts = []
    for xs, gs in shards:
        gxs = torch.empty_like(xs)
        cabi.bn_fire_bp_dist2_into(xs, w, b, ivar, mean, gs, gxhat, gxhatx, gxs, ALPHA, THRESH, BETA, INTERVAL)
        parts.append(gxs)
    torch.cuda.synchronize()
    rel_close(torch.cat(parts, dim=1), gx, "input gradient over two shards")
    rel_close(local[0][1][2] + local[1][1][2], gw, "weight gradient summed over shards")   # what DDP would sum
    rel_close(local[0][1][3] + local[1][1][3], gb, "bias gradient summed over shards")


def test_argument_checks_of_the_halves(cabi):
    lib = cabi.load()
    f32 = cabi.DTYPE_F32
    assert lib.snnlif_bn_fire_bp_dist1(*[None] * 10, f32, 0, 2, 3, 4, 0.25, 0.5, 1.0, 0.5, None, 0, None) == cabi.OK
    assert lib.snnlif_bn_fire_bp_dist1(*[None] * 10, f32, 4, 2, 3, 4, 0.25, 0.5, 1.0, 0.5, None, 0, None) == cabi.ERR_ARG
    assert lib.snnlif_bn_fire_bp_dist2(*[None] * 9, f32, 4, 2, 3, 4, 0.25, 0.5, 1.0, 0.5, None) == cabi.ERR_ARG
    assert lib.snnlif_bn_fire_bp_dist2(*[None] * 9, f32, 1025, 2, 3, 4, 0.25, 0.5, 1.0, 0.5, None) == cabi.ERR_ARG
    assert lib.snnlif_bn_fire_bp_dist2(*[None] * 9, cabi.DTYPE_BF16, 4, 2, 3, 4, 0.25, 0.5, 1.0, 0.5, None) == cabi.ERR_UNSUPPORTED
    x, g, w, b, var, mean = make((4, 2, 3, 2, 2), seed=44)
    out = [torch.empty_like(w) for _ in range(4)]
    small = torch.empty(8, dtype=torch.uint8, device="cuda")
    with pytest.raises(ValueError, match="workspace"):     # the ctypes helper checks sizes first
        cabi.bn_fire_bp_dist1_into(x, w, b, var, mean, g, *out, ALPHA, THRESH, BETA, INTERVAL, small)
    rc = lib.snnlif_bn_fire_bp_dist1(x.data_ptr(), w.data_ptr(), b.data_ptr(), var.data_ptr(), mean.data_ptr(),
                                     g.data_ptr(), *(t.data_ptr() for t in out), f32, 4, 2, 3, 4, ALPHA, THRESH,
                                     BETA, INTERVAL, small.data_ptr(), small.numel(), None)
    assert rc == cabi.ERR_WORKSPACE


@pytest.mark.parametrize("shape,dim_bn", [((6, 4, 8), (0, 1)), ((6, 4, 8, 8, 8), (0, 1, 3, 4))])
def test_plain_bn_halves(shape, dim_bn):
    import snn_gpu_training_bptt_amd.snnlib_func  # noqa: F401  (registers the module)
    import snnlib
    x, g, w, b, var, mean = make(shape, seed=45)
    ivar, _ = snnlib.bn_fp(x, w, b, var, mean, EPS)
    gx, gw, gb = snnlib.bn_bp(x, w, b, ivar, mean, dim_bn, g)
    m1, m2, gw2, gb2 = snnlib.bn_bp_dist1(x, w, b, ivar, mean, dim_bn, g)
    gx2 = snnlib.bn_bp_dist2(x, w, b, ivar, mean, dim_bn, g, m1, m2)
    rel_close(gw2, gw, "bn weight gradient")
    rel_close(gb2, gb, "bn bias gradient")
    rel_close(gx2, gx, "bn input gradient")
    # against autograd of the textbook formula
    xa, wa, ba = x.clone().requires_grad_(True), w.clone().requires_grad_(True), b.clone().requires_grad_(True)
    view = (1, 1, -1) + (1,) * (len(shape) - 3)
    mu = xa.mean(dim=dim_bn, keepdim=True)
    va = ((xa - mu) ** 2).mean(dim=dim_bn, keepdim=True)
    y = (xa - mu) / torch.sqrt(va + EPS) * wa.view(view) + ba.view(view)
    y.backward(g)
    rel_close(gx2, xa.grad, "bn input gradient vs autograd", tol=2e-5)
    rel_close(gw2, wa.grad, "bn weight gradient vs autograd", tol=2e-5)
    rel_close(gb2, ba.grad, "bn bias gradient vs autograd", tol=2e-5)
    # two shards with the statistics of the whole batch
    half = shape[1] // 2
    loc = [snnlib.bn_bp_dist1(x[:, r * half:(r + 1) * half].contiguous(), w, b, ivar, mean, dim_bn,
                              g[:, r * half:(r + 1) * half].contiguous()) for r in range(2)]
    a1, a2 = (loc[0][0] + loc[1][0]) / 2, (loc[0][1] + loc[1][1]) / 2
    parts = [snnlib.bn_bp_dist2(x[:, r * half:(r + 1) * half].contiguous(), w, b, ivar, mean, dim_bn,
                                g[:, r * half:(r + 1) * half].contiguous(), a1, a2) for r in range(2)]
    rel_close(torch.cat(parts, dim=1), gx, "bn input gradient over two shards")


def test_fused_halves_equal_the_unsplit_ops(hyper):
    import snnlib
    gen = torch.Generator().manual_seed(46)
    # fully connected
    x, _, w, b, var, mean = make((6, 4, 32), seed=47)
    wf = (torch.randn(10, 32, generator=gen) * 0.2).cuda()
    bf = torch.zeros(10).cuda()
    gfc = torch.randn(6, 4, 10, generator=gen).cuda()
    ivar, _ = snnlib.bn_fire_fc_fp(x, w, b, var, mean, EPS, wf, bf, ALPHA, THRESH)
    whole = snnlib.bn_fire_fc_bp(x, w, b, ivar, mean, (0, 1), gfc, wf, bf, (0, 1), ALPHA, THRESH, BETA, INTERVAL)
    gs, m1, m2, gwb, gbb, gwf, gbf = snnlib.bn_fire_fc_bp_dist1(
        x, w, b, ivar, mean, (0, 1), gfc, wf, bf, (0, 1), ALPHA, THRESH, BETA, INTERVAL)
    gx = snnlib.bn_fire_bp_dist2(x, w, b, ivar, mean, gs, m1, m2, ALPHA, THRESH, BETA, INTERVAL)
    for got, want in zip((gx, gwb, gbb, gwf, gbf), whole):
        assert torch.equal(got, want)
    # convolution
    x, _, w, b, var, mean = make((4, 2, 8, 8, 8), seed=48)
    wc = (torch.randn(5, 8, 3, 3, generator=gen) * 0.2).cuda()
    bc = torch.zeros(5).cuda()
    gconv = torch.randn(4, 2, 5, 8, 8, generator=gen).cuda()
    conv_args = ((1, 1), (1, 1), (1, 1), 1, False, False)
    ivar, _ = snnlib.bn_fire_conv_fp(x, w, b, var, mean, EPS, wc, bc, *conv_args, ALPHA, THRESH)
    whole = snnlib.bn_fire_conv_bp(x, w, b, ivar, mean, (0, 1, 3, 4), gconv, wc, *conv_args, True,
                                   (0, 1, 3, 4), ALPHA, THRESH, BETA, INTERVAL)
    gs, m1, m2, gwb, gbb, gwc, gbc = snnlib.bn_fire_conv_bp_dist1(
        x, w, b, ivar, mean, (0, 1, 3, 4), gconv, wc, *conv_args, True, (0, 1, 3, 4), ALPHA, THRESH, BETA, INTERVAL)
    gx = snnlib.bn_fire_bp_dist2(x, w, b, ivar, mean, gs, m1, m2, ALPHA, THRESH, BETA, INTERVAL)
    # the convolution's own gradients come from MIOpen, whose weight gradient is not bit-reproducible
    # from call to call; everything computed by this library's kernels is
    for got, want in zip((gwb, gbb), whole[1:3]):
        assert torch.equal(got, want)
    for got, want, what in zip((gx, gwc, gbc), (whole[0], whole[3], whole[4]), ("input", "conv weight", "conv bias")):
        rel_close(got, want, what + " gradient")
    # the exported but otherwise unused bn_fire_bp_dist1 (snnlib/cuda/snn.cpp:826)
    four = snnlib.bn_fire_bp_dist1(x, w, b, ivar, mean, (0, 1, 3, 4), gs, ALPHA, THRESH, BETA, INTERVAL)
    assert torch.equal(four[0], m1) and torch.equal(four[1], m2)


class OneRank:
    """Stand-in for ``torch.distributed`` with a single rank: all-reduce is the identity."""

    def __init__(self):
        self.calls = 0

    def install(self, monkeypatch):
        def all_reduce(tensor, op=None, group=None):
            self.calls += 1
            assert tensor.is_cuda and tensor.dim() == 1
        monkeypatch.setattr(torch.distributed, "all_reduce", all_reduce)
        monkeypatch.setattr(torch.distributed, "get_world_size", lambda group=None: 1)


@pytest.mark.parametrize("kind", ["bn", "fc", "conv"])
def test_dist_modules_with_one_rank(hyper, monkeypatch, kind):
    from snn_gpu_training_bptt_amd import snnlib_op as sop
    sf = hyper
    rank = OneRank()
    rank.install(monkeypatch)
    torch.manual_seed(49)
    if kind == "bn":
        shape = (6, 4, 8, 8, 8)
        layer = sop.BnDist(8, (0, 1, 3, 4)).cuda()
    elif kind == "fc":
        shape = (6, 4, 8, 4, 4)
        layer = sop.BnFireFcDist(8 * 16, 10, dim_bn=(0, 1, 3, 4), cin_bn=8).cuda()
    else:
        shape = (6, 4, 8, 8, 8)
        layer = sop.BnFireConvDist(8, 5).cuda()
    with torch.no_grad():
        layer.weight_bn.copy_(torch.rand(8) + 0.5)
        layer.bias_bn.copy_(torch.randn(8) * 0.2)
    x = (0.5 + torch.randn(shape)).cuda().requires_grad_(True)
    out = layer(x)
    gout = torch.randn_like(out)
    out.backward(gout)
    assert rank.calls == 4            # two vectors forward (statistics), two backward (means)

    # the same layer through the single-GPU function with the statistics formed the sharded way:
    # E[x] and E[x^2] from the op the layer itself uses, var = E[x^2] - E[x]^2
    import snnlib
    dim_bn = (0, 1, 3, 4)
    mean, second = snnlib.bn_moments(x.detach())
    var = second - mean ** 2
    torch.testing.assert_close(mean, x.detach().mean(dim=dim_bn), rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(second, (x.detach() ** 2).mean(dim=dim_bn), rtol=1e-5, atol=1e-6)
    x2 = x.detach().clone().requires_grad_(True)
    params = {n: p.detach().clone().requires_grad_(True) for n, p in layer.named_parameters()
              if not n.startswith("running")}
    if kind == "bn":
        ref = sf.bn_func(x2, params["weight_bn"], params["bias_bn"], var, mean, dim_bn, layer.eps_bn)
    elif kind == "fc":
        ref = sf.bn_fire_fc_func(x2, params["weight_bn"], params["bias_bn"], var, mean, dim_bn, layer.eps_bn,
                                 params["weight_fc"], params["bias_fc"])
    else:
        ref = sf.bn_fire_conv_func(x2, params["weight_bn"], params["bias_bn"], var, mean, layer.eps_bn,
                                   params["weight_conv"], params["bias_conv"], layer.stride, layer.padding, True)
    ref.backward(gout)
    if kind == "bn":
        rel_close(out, ref, "output")
        rel_close(x.grad, x2.grad, "input gradient")
    elif kind == "fc":
        assert torch.equal(out, ref)
        assert torch.equal(x.grad, x2.grad)
    else:       # MIOpen's convolution gradients may differ in the last bits from call to call
        assert torch.equal(out, ref)
        rel_close(x.grad, x2.grad, "input gradient")
    for n, p in params.items():
        rel_close(getattr(layer, n).grad, p.grad, n)
    # running statistics: momentum 0.05, variance corrected by n/(n-1)
    n = x.numel() / 8
    rel_close(layer.running_mean, 0.05 * mean, "running mean")
    rel_close(layer.running_var, 0.95 + var * (0.05 * n / (n - 1)), "running variance")


def test_residual_and_alexnet_style_stacks_of_dist_layers_train(hyper, monkeypatch):
    """The way the reference composes the sharded layers (snnlib/example/models.py:63-105 Alexnet_BN_DIST,
    :107-127 ResidualDist, in-place residual add included), scaled down, with one rank."""
    from snn_gpu_training_bptt_amd import snnlib_op as sop
    OneRank().install(monkeypatch)
    torch.manual_seed(50)
    T, B = 4, 8

    class Residual(torch.nn.Module):
        def __init__(self, cin, cout, stride, downsample):
            super().__init__()
            self.conv1 = sop.FireConv(cin, cout, kernel_size=(3, 3), stride=stride, padding=(1, 1))
            self.conv2 = sop.BnFireConvDist(cout, cout, kernel_size=(3, 3), stride=(1, 1), padding=(1, 1))
            self.bn2 = sop.BnDist(cout, dim_bn=(0, 1, 3, 4))
            self.downsample = downsample

        def forward(self, inp):
            x = self.bn2(self.conv2(self.conv1(inp)))
            x += self.downsample(inp) if self.downsample is not None else inp
            return x

    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.pre_conv = sop.Conv(3, 8, kernel_size=(3, 3), stride=(1, 1), padding=(1, 1))
            self.pre_bn = sop.BnDist(8, dim_bn=(0, 1, 3, 4))
            down = torch.nn.Sequential(sop.FireConv(8, 16, kernel_size=(1, 1), stride=(2, 2), padding=(0, 0)),
                                       sop.BnDist(16, (0, 1, 3, 4)))
            self.block1 = Residual(8, 16, (2, 2), down)
            self.block2 = Residual(16, 16, (1, 1), None)
            self.conv = sop.BnFireConvDist(16, 16, stride=(2, 2))
            self.fc1 = sop.BnFireFcDist(4 * 4 * 16, 32, dim_bn=(0, 1, 3, 4), cin_bn=16)
            self.fc2 = sop.BnFireFcDist(32, 32, dim_bn=(0, 1))
            self.fire = sop.Fire()
            self.fc3 = torch.nn.Linear(32, 10)

        def forward(self, images):
            x = torch.stack([images] * T, dim=0)
            x = self.pre_bn(self.pre_conv(x))
            x = self.block2(self.block1(x))
            x = self.fc2(self.fc1(self.conv(x)))
            return self.fc3(self.fire(x).mean(dim=0))

    net = Net().cuda()
    images = torch.rand(B, 3, 16, 16).cuda()
    labels = torch.randint(0, 10, (B,)).cuda()
    trainable = [p for n, p in net.named_parameters() if "running" not in n]
    opt = torch.optim.SGD(trainable, lr=0.05)
    crit = torch.nn.CrossEntropyLoss()
    losses = []
    for _ in range(12):
        opt.zero_grad(set_to_none=True)
        loss = crit(net(images), labels)
        loss.backward()
        for n, p in net.named_parameters():
            if "running" not in n:
                assert p.grad is not None and torch.isfinite(p.grad).all(), n
        opt.step()
        losses.append(float(loss.detach()))
    assert losses[-1] < losses[0], losses
    # inference with the running statistics
    for m in net.modules():
        if hasattr(m, "train_bn"):
            m.train_bn = False
    with torch.no_grad():
        out = net(images)
    assert out.shape == (B, 10) and torch.isfinite(out).all()
