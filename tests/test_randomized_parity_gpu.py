"""Seeded random sweep of shapes, window lengths, storage types, hyper-parameters, cache hints and base-pointer
offsets through the C ABI against the CPU oracle: the cases nobody thought of listing by hand.

fp32 / fp64: spikes, membrane potentials and gradients bit-identical.  bf16 storage: spikes exact,
potentials and gradients equal to the fp32 oracle on the bf16-rounded inputs rounded once to bf16.
Batch-norm + fire (fp32 and fp64): spikes and inverse standard deviation bit-identical, gradients to
1e-5 (fp32) / 1e-11 (fp64) of scale.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def cabi():
    from snn_gpu_training_bptt_amd import lif_cabi
    lif_cabi.load()
    return lif_cabi


@pytest.fixture(scope="module")
def oracle():
    from oracle import c_oracle
    return c_oracle


def draw_case(rng):
    T = int(rng.choice([1, 2, 3, 4, 5, 6, 7, 8, 9, 11, 12, 13, 16, 17, 23, 24, 31, 32, 33, 40, 47, 48, 64, 65, 97]))
    n = int(rng.choice([1, 2, 3, 63, 64, 65, 127, 255, 256, 257, 1000, 4097, 20000]))
    B = int(rng.integers(1, 4))
    dtype = [torch.float32, torch.float32, torch.float64, torch.bfloat16][int(rng.integers(0, 4))]
    alpha = float(rng.choice([0.0, 0.25, 0.3, 0.5, 0.9, 1.0]))
    thresh = float(rng.choice([0.25, 0.5, 1.0]))
    beta = float(rng.choice([0.7, 1.0, 2.0]))
    interval = float(rng.choice([0.3, 0.5, 1.5]))
    offset = int(rng.integers(0, 4))       # elements by which the base pointers are shifted
    keep = [None, True, False][int(rng.integers(0, 3))]   # cache hint: by size / kept / streamed
    return T, B, n, dtype, alpha, thresh, beta, interval, offset, keep


@pytest.mark.parametrize("seed", range(240))
def test_random_fire_case(cabi, oracle, seed):
    rng = np.random.default_rng(9000 + seed)
    T, B, n, dtype, alpha, thresh, beta, interval, offset, keep = draw_case(rng)
    shape = (T, B, n)
    gen = torch.Generator().manual_seed(seed)
    x = (0.4 + 0.9 * torch.randn(shape, generator=gen)).to(dtype)
    g = torch.randn(shape, generator=gen).to(dtype)
    numel = x.numel()

    def shifted(src=None):     # a dense tensor whose base pointer is `offset` elements into a buffer
        buf = torch.empty(numel + offset, dtype=dtype, device="cuda")
        view = buf[offset:].view(shape)
        if src is not None:
            view.copy_(src)
        return view

    xd, gd = shifted(x), shifted(g)
    mem, spike, gx = shifted(), shifted(), shifted()
    cabi.fire_us_fp_into(xd, mem, spike, alpha, thresh, keep_spatial=keep)
    cabi.fire_bp_into(xd, gd, gx, alpha, thresh, beta, interval, keep_spatial=keep)
    spike_only = shifted()
    cabi.fire_s_fp_into(xd, spike_only, alpha, thresh, keep_spatial=keep)
    torch.cuda.synchronize()

    what = f"T={T} B={B} n={n} {dtype} a={alpha} th={thresh} b={beta} iv={interval} off={offset} keep={keep}"
    if dtype == torch.bfloat16:
        xo, go = x.float().numpy(), g.float().numpy()
        mem_o, spike_o = oracle.fire_forward(xo, alpha, thresh)
        gx_o = oracle.fire_backward(xo, go, alpha, thresh, beta, interval)
        rounded = lambda a: torch.from_numpy(a).to(torch.bfloat16).float().numpy()
        assert np.array_equal(spike.float().cpu().numpy(), spike_o), what
        assert np.array_equal(spike_only.float().cpu().numpy(), spike_o), what
        assert np.array_equal(mem.float().cpu().numpy(), rounded(mem_o)), what
        assert np.array_equal(gx.float().cpu().numpy(), rounded(gx_o)), what
    else:
        mem_o, spike_o = oracle.fire_forward(x.numpy(), alpha, thresh)
        gx_o = oracle.fire_backward(x.numpy(), g.numpy(), alpha, thresh, beta, interval)
        assert np.array_equal(spike.cpu().numpy(), spike_o), what
        assert np.array_equal(spike_only.cpu().numpy(), spike_o), what
        assert np.array_equal(mem.cpu().numpy(), mem_o), what
        assert np.array_equal(gx.cpu().numpy(), gx_o), what


@pytest.mark.parametrize("seed", range(64))
def test_random_bn_fire_case(cabi, oracle, seed):
    rng = np.random.default_rng(9500 + seed)
    T = int(rng.choice([1, 2, 4, 6, 8, 9, 13, 16, 24, 32, 33, 50, 64]))
    B = int(rng.integers(1, 5))
    C = int(rng.choice([1, 2, 3, 8, 17, 64]))
    HW = int(rng.choice([1, 2, 9, 31, 32, 33, 49, 64, 100, 196]))
    alpha = float(rng.choice([0.25, 0.3, 0.9]))
    thresh = float(rng.choice([0.25, 0.5]))
    beta = float(rng.choice([0.7, 1.0]))
    interval = float(rng.choice([0.5, 1.5]))
    eps = 1e-5
    dtype = torch.float64 if rng.integers(0, 3) == 0 else torch.float32
    shape = (T, B, C, HW)
    gen = torch.Generator().manual_seed(seed)
    x = (0.5 + torch.randn(shape, generator=gen) * (0.5 + torch.rand((C, 1), generator=gen))).to(dtype)
    g = torch.randn(shape, generator=gen).to(dtype)
    w = (0.5 + torch.rand(C, generator=gen)).to(dtype)
    b = (0.2 * torch.randn(C, generator=gen)).to(dtype)
    var, mean = torch.var_mean(x, dim=(0, 1, 3), unbiased=False)
    var = var + 0.05          # also meaningful when T*B*HW == 1
    xd, gd, wd, bd, vd, md = (t.cuda() for t in (x, g, w, b, var, mean))
    ivar, spike = torch.empty_like(vd), torch.empty_like(xd)
    cabi.bn_fire_s_fp_into(xd, wd, bd, vd, md, ivar, spike, eps, alpha, thresh,
                           keep_spatial=(None, True, False)[seed % 3])
    gx, gw, gb = torch.empty_like(xd), torch.empty_like(wd), torch.empty_like(wd)
    code = cabi.DTYPE_F64 if dtype == torch.float64 else cabi.DTYPE_F32
    ws = torch.empty(cabi.bn_fire_bp_workspace_bytes(code, T, B, C, HW), dtype=torch.uint8, device="cuda")
    cabi.bn_fire_bp_into(xd, wd, bd, ivar, md, gd, gx, gw, gb, alpha, thresh, beta, interval, ws)
    torch.cuda.synchronize()

    what = f"T={T} B={B} C={C} HW={HW} {dtype} a={alpha} th={thresh} b={beta} iv={interval}"
    tol, floor = (1e-11, 1e-14) if dtype == torch.float64 else (1e-5, 1e-7)
    ivar_o, _, spike_o = oracle.bn_fire_forward(x.numpy(), w.numpy(), b.numpy(), var.numpy(), mean.numpy(), eps, alpha, thresh)
    gx_o, gw_o, gb_o = oracle.bn_fire_backward(x.numpy(), w.numpy(), b.numpy(), ivar_o, mean.numpy(), g.numpy(),
                                               alpha, thresh, beta, interval)
    assert np.array_equal(ivar.cpu().numpy(), ivar_o), what
    assert np.array_equal(spike.cpu().numpy(), spike_o), what
    for got, want, name in ((gb, gb_o, "bias"), (gw, gw_o, "weight"), (gx, gx_o, "input")):
        scale = np.abs(want).max() + 1e-12
        err = np.abs(got.cpu().numpy() - want).max()
        assert err <= tol * scale + floor, f"{what}: {name} gradient err {err:.3e} vs scale {scale:.3e}"
