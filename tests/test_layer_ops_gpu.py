"""The remaining single-GPU layers of the snnlib interface -- ``Bn``, ``Fc``, ``Conv``, ``BnFireFc``,
``BnFireConv`` -- against the gold restatement of the reference's per-time-step PyTorch modules
(snnlib/example/gold_op.py:49-179), in the manner of the reference's test_bn.py, test_fc.py,
test_conv.py, test_bn_fire_fc.py and test_bn_fire_conv.py: same inputs and parameters on both sides,
outputs and every gradient compared.

Dense parts run on the same rocBLAS / MIOpen kernels on both sides, but with T*B rows per call here
and B rows per call in the gold loop, so the bar is 2e-5 of the tensor's scale, not bit equality.
The spikes feeding them are compared exactly where the test can see them.
"""
import pytest
import torch

from conftest import ALPHA, BETA, INTERVAL, THRESH, seed_clear_of_decision_points

pytestmark = pytest.mark.gpu
EPS = 1e-5


@pytest.fixture()
def mods():
    from oracle import gold_fire
    from snn_gpu_training_bptt_amd import snnlib_func as sf
    from snn_gpu_training_bptt_amd import snnlib_op as sop
    saved = (sf.alpha, sf.thresh, sf.beta, sf.interval)
    sf.alpha, sf.thresh, sf.beta, sf.interval = ALPHA, THRESH, BETA, INTERVAL
    yield sf, sop, gold_fire
    sf.alpha, sf.thresh, sf.beta, sf.interval = saved


def close(a, b, what, tol=2e-5):
    scale = b.abs().max().item() + 1e-12
    err = (a - b).abs().max().item()
    assert err <= tol * scale, f"{what}: max abs err {err:.3e} vs scale {scale:.3e}"


def clones(*tensors):
    return [t.detach().clone().requires_grad_(True) for t in tensors]


def randomise_bn(layer, gen_seed):
    g = torch.Generator().manual_seed(gen_seed)
    C = layer.weight_bn.numel()
    dev = layer.weight_bn.device
    layer.weight_bn = torch.nn.Parameter((0.5 + torch.rand(C, generator=g)).to(dev))
    layer.bias_bn = torch.nn.Parameter((0.2 * torch.randn(C, generator=g)).to(dev))
    layer.running_var = torch.nn.Parameter((0.5 + torch.rand(C, generator=g)).to(dev))
    layer.running_mean = torch.nn.Parameter((0.1 * torch.randn(C, generator=g)).to(dev))


@pytest.mark.parametrize("shape,dim_bn", [((6, 2, 8), (0, 1)), ((6, 2, 8, 8, 8), (0, 1, 3, 4)), ((4, 8, 32, 16, 16), (0, 1, 3, 4))])
@pytest.mark.parametrize("train_bn", [True, False])
def test_bn(mods, shape, dim_bn, train_bn):
    _, sop, gold = mods
    torch.manual_seed(51)
    x_cpu = 0.3 + 1.5 * torch.randn(shape)
    layer = sop.Bn(shape[2], dim_bn, EPS).cuda()
    randomise_bn(layer, 52)
    layer.train_bn = train_bn
    rm, rv = layer.running_mean.detach().clone(), layer.running_var.detach().clone()
    x = x_cpu.cuda().requires_grad_(True)
    y = layer(x)
    g = torch.randn_like(y)
    y.backward(g)
    xg, w, b = clones(x_cpu.cuda(), layer.weight_bn, layer.bias_bn)
    ref = gold.gold_bn(xg, w, b, rm, rv, train_bn, EPS)
    ref.backward(g)
    close(y.detach(), ref.detach(), "bn output")
    close(layer.weight_bn.grad, w.grad, "weight gradient")
    close(layer.bias_bn.grad, b.grad, "bias gradient")
    if train_bn:   # like the reference, the backward always treats the statistics as batch statistics
        close(x.grad, xg.grad, "input gradient")


@pytest.mark.parametrize("shape,cout", [((6, 2, 8), 8), ((6, 2, 8, 8, 8), 8), ((8, 16, 300), 17)])
def test_fc(mods, shape, cout):
    _, sop, gold = mods
    torch.manual_seed(53)
    x_cpu = torch.randn(shape)
    layer = sop.Fc(x_cpu[0, 0].numel(), cout).cuda()
    with torch.no_grad():
        layer.bias_fc.normal_()
    x = x_cpu.cuda().requires_grad_(True)
    y = layer(x)
    g = torch.randn_like(y)
    y.backward(g)
    xg, w, b = clones(x_cpu.cuda(), layer.weight_fc, layer.bias_fc)
    ref = gold.gold_fc(xg, w, b)
    ref.backward(g)
    close(y.detach(), ref.detach(), "fc output")
    close(x.grad, xg.grad, "input gradient")
    close(layer.weight_fc.grad, w.grad, "weight gradient")
    close(layer.bias_fc.grad, b.grad, "bias gradient")


@pytest.mark.parametrize("shape,cout,stride,padding,bias", [
    ((6, 2, 8, 8, 8), 8, (1, 1), (1, 1), True),
    ((4, 3, 3, 32, 32), 16, (1, 1), (1, 1), True),      # the first layer of the CIFAR model
    ((3, 2, 16, 9, 7), 12, (2, 2), (1, 1), False),
])
def test_conv(mods, shape, cout, stride, padding, bias):
    _, sop, gold = mods
    torch.manual_seed(54)
    x_cpu = torch.randn(shape)
    layer = sop.Conv(shape[2], cout, (3, 3), stride, padding, if_bias_conv=bias).cuda()
    x = x_cpu.cuda().requires_grad_(True)
    y = layer(x)
    g = torch.randn_like(y)
    y.backward(g)
    xg, w, b = clones(x_cpu.cuda(), layer.weight_conv, layer.bias_conv)
    ref = gold.gold_conv(xg, w, b, stride, padding)
    ref.backward(g)
    close(y.detach(), ref.detach(), "conv output")
    close(x.grad, xg.grad, "input gradient")
    close(layer.weight_conv.grad, w.grad, "weight gradient")
    if bias:
        close(layer.bias_conv.grad, b.grad, "bias gradient")
    else:
        assert layer.bias_conv.grad is None


@pytest.mark.parametrize("shape,dim_bn,cin_bn,cout", [
    ((6, 2, 8), (0, 1), None, 8),
    ((6, 2, 8, 8, 8), (0, 1, 3, 4), 8, 8),
    ((8, 8, 32, 4, 4), (0, 1, 3, 4), 32, 40),            # image-shaped input flattened for the linear
    ((8, 16, 256), (0, 1), None, 64),
])
@pytest.mark.parametrize("train_bn", [True, False])
def test_bn_fire_fc(mods, shape, dim_bn, cin_bn, cout, train_bn):
    _, sop, gold = mods

    def build(seed):
        torch.manual_seed(seed)
        x_cpu = 0.3 + torch.randn(shape)
        layer = sop.BnFireFc(x_cpu[0, 0].numel(), cout, dim_bn, EPS, cin_bn=cin_bn).cuda()
        randomise_bn(layer, seed + 1)
        layer.train_bn = train_bn
        return x_cpu, layer

    def potentials(seed):
        x_cpu, layer = build(seed)
        with torch.no_grad():
            return gold.gold_bn_fire(x_cpu.cuda(), layer.weight_bn, layer.bias_bn, layer.running_mean.clone(),
                                     layer.running_var.clone(), train_bn, EPS, ALPHA, THRESH, BETA, INTERVAL)[0]

    x_cpu, layer = build(seed_clear_of_decision_points(potentials, range(55, 4055, 100)))
    rm, rv = layer.running_mean.detach().clone(), layer.running_var.detach().clone()
    x = x_cpu.cuda().requires_grad_(True)
    y = layer(x)
    g = torch.randn_like(y)
    y.backward(g)
    xg, wbn, bbn, wfc, bfc = clones(x_cpu.cuda(), layer.weight_bn, layer.bias_bn, layer.weight_fc, layer.bias_fc)
    ref = gold.gold_bn_fire_fc(xg, wbn, bbn, rm, rv, train_bn, EPS, wfc, bfc, ALPHA, THRESH, BETA, INTERVAL)
    ref.backward(g)
    close(y.detach(), ref.detach(), "fc output")
    close(layer.weight_fc.grad, wfc.grad, "fc weight gradient")
    close(layer.bias_fc.grad, bfc.grad, "fc bias gradient")
    close(layer.weight_bn.grad, wbn.grad, "bn weight gradient")
    close(layer.bias_bn.grad, bbn.grad, "bn bias gradient")
    if train_bn:
        close(x.grad, xg.grad, "input gradient")


@pytest.mark.parametrize("shape,cout,stride", [((6, 2, 8, 8, 8), 8, (1, 1)), ((4, 4, 32, 16, 16), 48, (2, 2))])
@pytest.mark.parametrize("train_bn,bias", [(True, True), (False, True), (True, False)])
def test_bn_fire_conv(mods, shape, cout, stride, train_bn, bias):
    _, sop, gold = mods

    def build(seed):
        torch.manual_seed(seed)
        x_cpu = 0.3 + torch.randn(shape)
        layer = sop.BnFireConv(shape[2], cout, (3, 3), stride, (1, 1), EPS, if_bias_conv=bias).cuda()
        randomise_bn(layer, seed + 1)
        layer.train_bn = train_bn
        return x_cpu, layer

    def potentials(seed):
        x_cpu, layer = build(seed)
        with torch.no_grad():
            return gold.gold_bn_fire(x_cpu.cuda(), layer.weight_bn, layer.bias_bn, layer.running_mean.clone(),
                                     layer.running_var.clone(), train_bn, EPS, ALPHA, THRESH, BETA, INTERVAL)[0]

    x_cpu, layer = build(seed_clear_of_decision_points(potentials, range(57, 4057, 100)))
    rm, rv = layer.running_mean.detach().clone(), layer.running_var.detach().clone()
    x = x_cpu.cuda().requires_grad_(True)
    y = layer(x)
    g = torch.randn_like(y)
    y.backward(g)
    xg, wbn, bbn, wc, bc = clones(x_cpu.cuda(), layer.weight_bn, layer.bias_bn, layer.weight_conv, layer.bias_conv)
    ref = gold.gold_bn_fire_conv(xg, wbn, bbn, rm, rv, train_bn, EPS, wc, bc, stride, (1, 1), ALPHA, THRESH, BETA, INTERVAL)
    ref.backward(g)
    close(y.detach(), ref.detach(), "conv output")
    close(layer.weight_conv.grad, wc.grad, "conv weight gradient")
    if bias:
        close(layer.bias_conv.grad, bc.grad, "conv bias gradient")
    else:
        assert layer.bias_conv.grad is None
    close(layer.weight_bn.grad, wbn.grad, "bn weight gradient")
    close(layer.bias_bn.grad, bbn.grad, "bn bias gradient")
    if train_bn:
        close(x.grad, xg.grad, "input gradient")


def test_cifar_style_stack_trains(mods):
    """Conv -> BnFireConv x2 -> BnFireFc x2 -> BnFire -> Linear, the layer pattern of the reference's
    CIFAR model (snnlib/example/models.py:8-61) at reduced width: one SGD step lowers the loss on a
    fixed batch and every parameter receives a finite gradient."""
    sf, sop, _ = mods
    torch.manual_seed(59)
    T, B = 4, 8

    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.conv1 = sop.Conv(3, 16)
            self.conv2 = sop.BnFireConv(16, 32, stride=(2, 2))
            self.conv3 = sop.BnFireConv(32, 32, stride=(2, 2))
            self.fc1 = sop.BnFireFc(8 * 8 * 32, 64, dim_bn=(0, 1, 3, 4), cin_bn=32)
            self.fc2 = sop.BnFireFc(64, 32, dim_bn=(0, 1))
            self.bn = sop.BnFire(32, dim_bn=(0, 1))
            self.head = torch.nn.Linear(32, 10)

        def forward(self, img):
            x = torch.stack([img for _ in range(T)], dim=0)
            for layer in (self.conv1, self.conv2, self.conv3, self.fc1, self.fc2, self.bn):
                x = layer(x)
            return self.head(x.mean(dim=0))

    net = Net().cuda()
    img = torch.rand(B, 3, 32, 32).cuda()
    labels = torch.randint(0, 10, (B,)).cuda()
    opt = torch.optim.SGD(net.parameters(), lr=0.05)
    losses = []
    for _ in range(8):
        opt.zero_grad()
        loss = torch.nn.functional.cross_entropy(net(img), labels)
        loss.backward()
        for name, p in net.named_parameters():
            if "running" in name:
                continue
            assert p.grad is not None and torch.isfinite(p.grad).all(), name
        opt.step()
        losses.append(loss.item())
    assert losses[-1] < losses[0], losses


def test_cifar_model_at_full_width(mods):
    """The reference's CIFAR model at its real layer widths (snnlib/example/models.py:8-61: 128-128-128 /
    256-256-256 / 512-512-512 convolutions, 8192-1024-512 fully connected, T = 6), assembled from this
    build's layers: two SGD steps on a small batch, then inference with the running statistics."""
    _, sop, _ = mods
    import numpy as np
    torch.manual_seed(61)
    T, B = 6, 8

    class Cifar(torch.nn.Module):
        def __init__(self):
            super().__init__()
            s1, s2, p = (1, 1), (2, 2), (1, 1)
            self.conv1_1 = sop.Conv(3, 128, kernel_size=(3, 3), stride=s1, padding=p)
            self.conv1_2 = sop.BnFireConv(128, 128, kernel_size=(3, 3), stride=s1, padding=p)
            self.conv1_3 = sop.BnFireConv(128, 128, kernel_size=(3, 3), stride=s2, padding=p)
            self.conv2_1 = sop.BnFireConv(128, 256, kernel_size=(3, 3), stride=s1, padding=p)
            self.conv2_2 = sop.BnFireConv(256, 256, kernel_size=(3, 3), stride=s1, padding=p)
            self.conv2_3 = sop.BnFireConv(256, 256, kernel_size=(3, 3), stride=s2, padding=p)
            self.conv3_1 = sop.BnFireConv(256, 512, kernel_size=(3, 3), stride=s1, padding=p)
            self.conv3_2 = sop.BnFireConv(512, 512, kernel_size=(3, 3), stride=s1, padding=p)
            self.conv3_3 = sop.BnFireConv(512, 512, kernel_size=(3, 3), stride=s2, padding=p)
            self.fc1 = sop.BnFireFc(4 * 4 * 512, 1024, dim_bn=(0, 1, 3, 4), cin_bn=512)
            self.fc2 = sop.BnFireFc(1024, 512, dim_bn=(0, 1))
            self.bn = sop.BnFire(512, dim_bn=(0, 1))
            self.fc3 = torch.nn.Linear(512, 10)

        def forward(self, images):
            x = torch.stack([images for _ in range(T)], dim=0)
            for name in ("conv1_1", "conv1_2", "conv1_3", "conv2_1", "conv2_2", "conv2_3",
                         "conv3_1", "conv3_2", "conv3_3", "fc1", "fc2", "bn"):
                x = getattr(self, name)(x)
            return self.fc3(x.mean(dim=0))

    net = Cifar().cuda()
    images = torch.rand(B, 3, 32, 32).cuda()
    labels = torch.randint(0, 10, (B,)).cuda()
    trainable = [p for n, p in net.named_parameters() if "running" not in n]
    opt = torch.optim.SGD(trainable, lr=0.02)
    crit = torch.nn.CrossEntropyLoss()
    losses = []
    for _ in range(2):
        opt.zero_grad(set_to_none=True)
        loss = crit(net(images), labels)
        loss.backward()
        for n, p in net.named_parameters():
            if "running" not in n:
                assert p.grad is not None and bool(torch.isfinite(p.grad).all()), n
        opt.step()
        losses.append(float(loss.detach()))
    assert all(np.isfinite(losses)), losses
    spikes_seen = net.bn(torch.randn(T, B, 512, device="cuda"))
    assert bool(((spikes_seen == 0) | (spikes_seen == 1)).all())
    for m in net.modules():
        if hasattr(m, "train_bn"):
            m.train_bn = False
    with torch.no_grad():
        out = net(images)
    assert out.shape == (B, 10) and bool(torch.isfinite(out).all())
