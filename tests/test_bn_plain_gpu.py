"""Plain batch norm (no fire recurrence) on the GPU, through the C ABI.

Against the CPU oracle (``oracle/lif_oracle.c``: ``lif_oracle_plain_bn_*``, which follow the reference's
bn_fp / bn_bp kernels): the output and the per-channel inverse standard deviation bit-exact (same
operation order, one rounding per operation); gradients within 1e-5 of the tensor's scale (the
reference itself reduces the per-channel sums in no defined order).  The two halves of the backward
for a sharded batch against the unsplit one, bit for bit.
"""
import numpy as np
import pytest
import torch

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


def make(shape, seed, dtype=torch.float32):
    gen = torch.Generator().manual_seed(seed)
    C = shape[2]
    spread = 0.5 + torch.rand((C,) + (1,) * (len(shape) - 3), generator=gen)
    x = (0.5 + torch.randn(shape, generator=gen) * spread).to(dtype)
    g = torch.randn(shape, generator=gen).to(dtype)
    w = (0.5 + torch.rand(C, generator=gen)).to(dtype)
    b = (0.2 * torch.randn(C, generator=gen)).to(dtype)
    dims = (0, 1) + tuple(range(3, len(shape)))
    var, mean = torch.var_mean(x, dim=dims, unbiased=False)
    return x, g, w, b, var, mean


SHAPES = [
    (6, 2, 8),                # the reference test's fc shape (test_bn.py)
    (6, 2, 8, 8, 8),          # the reference test's conv shape
    (8, 16, 32, 16, 16),      # HW = 256
    (4, 5, 7, 7, 7),          # HW = 49: one partly idle wavefront per plane, C*HW odd: one element per lane
    (6, 3, 6, 14, 14),        # HW = 196: four wavefronts per plane, the last with 4 active lanes
    (5, 2, 3, 4, 8),          # HW = 32: the smallest plane-aligned case
    (5, 2, 9, 31),            # HW = 31: just below it, one lane per column
    (13, 3, 20, 5, 3),        # T*B = 39 rows: the last row slice partly filled
    (1, 1, 4, 8, 8),          # a single row
    (3, 1, 2, 2),             # C*HW = 4: one pack
    (100, 3, 20),             # fully connected, 300 rows
    (8, 64, 1024),            # fully connected, many channels
    (6, 200, 4, 3, 3),        # HW = 9, few channels, many rows
    (1100, 2, 6, 8, 8),       # 2200 rows
    (6, 64, 512, 7, 7),       # the reference's ResNet block shape (models.py:145)
    (8, 32, 128, 32, 32),     # 16 wavefront partials per plane
    (2, 3, 5, 6),             # C*HW = 30: two elements per lane at most
]


@pytest.mark.parametrize("shape", SHAPES)
def test_bn_against_oracle(cabi, shape):
    from oracle import c_oracle
    x, g, w, b, var, mean = make(shape, seed=61)
    T, B, C = shape[:3]
    HW = int(np.prod(shape[3:])) if len(shape) > 3 else 1
    xd, gd, wd, bd, vd, md = (t.cuda() for t in (x, g, w, b, var, mean))
    ivar, y = torch.empty_like(vd), torch.empty_like(xd)
    cabi.bn_fp_into(xd, wd, bd, vd, md, ivar, y, EPS)
    gx, gw, gb = torch.empty_like(xd), torch.empty_like(wd), torch.empty_like(wd)
    ws = torch.empty(cabi.bn_bp_workspace_bytes(cabi.DTYPE_F32, T, B, C, HW), dtype=torch.uint8, device="cuda")
    cabi.bn_bp_into(xd, wd, ivar, md, gd, gx, gw, gb, ws)
    torch.cuda.synchronize()

    ivar_o, y_o = c_oracle.bn_forward(x.numpy(), w.numpy(), b.numpy(), var.numpy(), mean.numpy(), EPS)
    gx_o, gw_o, gb_o = c_oracle.bn_backward(x.numpy(), w.numpy(), ivar_o, mean.numpy(), g.numpy())
    assert np.array_equal(ivar.cpu().numpy(), ivar_o), "inverse standard deviation differs"
    assert np.array_equal(y.cpu().numpy(), y_o), "output differs from the oracle"
    rel_close(gb.cpu().numpy(), gb_o, "bias gradient")
    rel_close(gw.cpu().numpy(), gw_o, "weight gradient")
    rel_close(gx.cpu().numpy(), gx_o, "input gradient")

    # reproducibility: the reduction order is fixed
    gx2, gw2, gb2 = torch.empty_like(xd), torch.empty_like(wd), torch.empty_like(wd)
    cabi.bn_bp_into(xd, wd, ivar, md, gd, gx2, gw2, gb2, ws)
    assert torch.equal(gx, gx2) and torch.equal(gw, gw2) and torch.equal(gb, gb2)

    # the two halves of a sharded batch: dist1 + dist2 on the same arrays is the unsplit backward
    m1, m2, gw3, gb3 = (torch.empty_like(wd) for _ in range(4))
    cabi.bn_bp_dist1_into(xd, wd, ivar, md, gd, m1, m2, gw3, gb3, ws)
    gx3 = torch.empty_like(xd)
    cabi.bn_bp_dist2_into(xd, wd, ivar, md, gd, m1, m2, gx3)
    assert torch.equal(gw3, gw) and torch.equal(gb3, gb) and torch.equal(gx3, gx)
    count = T * B * HW
    rel_close(m1.cpu().numpy(), w.numpy() * gb_o / count, "mean of the xhat gradient")
    rel_close(m2.cpu().numpy(), w.numpy() * gw_o / count, "mean of the xhat*x gradient")


@pytest.mark.parametrize("shape", [(6, 2, 8, 8, 8), (5, 2, 9, 31), (8, 4, 16, 16, 16), (6, 16, 40)])
def test_bn_double_precision(cabi, shape):
    from oracle import c_oracle
    x, g, w, b, var, mean = make(shape, seed=62, dtype=torch.float64)
    T, B, C = shape[:3]
    HW = int(np.prod(shape[3:])) if len(shape) > 3 else 1
    xd, gd, wd, bd, vd, md = (t.cuda() for t in (x, g, w, b, var, mean))
    ivar, y = torch.empty_like(vd), torch.empty_like(xd)
    cabi.bn_fp_into(xd, wd, bd, vd, md, ivar, y, EPS)
    gx, gw, gb = torch.empty_like(xd), torch.empty_like(wd), torch.empty_like(wd)
    ws = torch.empty(cabi.bn_bp_workspace_bytes(cabi.DTYPE_F64, T, B, C, HW), dtype=torch.uint8, device="cuda")
    cabi.bn_bp_into(xd, wd, ivar, md, gd, gx, gw, gb, ws)
    ivar_o, y_o = c_oracle.bn_forward(x.numpy(), w.numpy(), b.numpy(), var.numpy(), mean.numpy(), EPS)
    gx_o, gw_o, gb_o = c_oracle.bn_backward(x.numpy(), w.numpy(), ivar_o, mean.numpy(), g.numpy())
    assert ivar.dtype == torch.float64 and y.dtype == torch.float64
    assert np.array_equal(ivar.cpu().numpy(), ivar_o)
    assert np.array_equal(y.cpu().numpy(), y_o)
    rel_close(gb.cpu().numpy(), gb_o, "bias gradient", 1e-12)
    rel_close(gw.cpu().numpy(), gw_o, "weight gradient", 1e-12)
    rel_close(gx.cpu().numpy(), gx_o, "input gradient", 1e-12)


def test_bn_misaligned_bases_and_odd_rows(cabi):
    """Tensors that start 4 bytes past a 16-byte boundary (the wide-lane form does not apply) and a row
    length that is a multiple of 4 elements all the same: same bits as the aligned call."""
    from oracle import c_oracle
    shape = (5, 3, 8, 4, 4)
    x, g, w, b, var, mean = make(shape, seed=63)
    n = x.numel()
    pool = torch.empty(3 * (n + 8), device="cuda")
    xd = pool[1:1 + n].view(shape)
    gd = pool[n + 9:2 * n + 9].view(shape)
    yd = pool[2 * n + 13:3 * n + 13].view(shape)
    xd.copy_(x)
    gd.copy_(g)
    assert xd.data_ptr() % 16 == 4 and gd.data_ptr() % 16 == 4 and yd.data_ptr() % 16 == 4
    wd, bd, vd, md = (t.cuda() for t in (w, b, var, mean))
    ivar = torch.empty_like(vd)
    cabi.bn_fp_into(xd, wd, bd, vd, md, ivar, yd, EPS)
    ivar_o, y_o = c_oracle.bn_forward(x.numpy(), w.numpy(), b.numpy(), var.numpy(), mean.numpy(), EPS)
    assert np.array_equal(yd.cpu().numpy(), y_o) and np.array_equal(ivar.cpu().numpy(), ivar_o)
    gw, gb = torch.empty_like(wd), torch.empty_like(wd)
    ws = torch.empty(cabi.bn_bp_workspace_bytes(cabi.DTYPE_F32, 5, 3, 8, 16), dtype=torch.uint8, device="cuda")
    cabi.bn_bp_into(xd, wd, ivar, md, gd, yd, gw, gb, ws)           # gx into the misaligned buffer
    gx_a = torch.empty(shape, device="cuda")
    cabi.bn_bp_into(x.cuda(), wd, ivar, md, g.cuda(), gx_a, gw, gb, ws)
    assert torch.equal(yd, gx_a)


def test_bn_empty_shapes_and_errors(cabi):
    dev = "cuda"
    C = 4
    w = torch.ones(C, device=dev)
    for shape in [(0, 2, C, 3), (2, 0, C, 3), (2, 2, C, 0)]:
        x = torch.empty(shape, device=dev)
        ivar = torch.full((C,), 7.0, device=dev)
        cabi.bn_fp_into(x, w, w, w, w, ivar, torch.empty_like(x), EPS)
        gw = torch.full((C,), 7.0, device=dev)
        gb = torch.full((C,), 7.0, device=dev)
        cabi.bn_bp_into(x, w, w, w, x, torch.empty_like(x), gw, gb, None)
        assert float(ivar[0]) == 7.0 and float(gw[0]) == 7.0 and float(gb[0]) == 7.0   # untouched
    lib = cabi.load()
    x = torch.zeros((2, 2, C, 3), device=dev)
    y = torch.empty_like(x)
    p = lambda t: t.data_ptr()
    assert lib.snnlif_bn_fp(p(x), p(w), p(w), p(w), p(w), p(w), p(y), cabi.DTYPE_BF16, 2, 2, C, 3, EPS, None) == cabi.ERR_UNSUPPORTED
    assert lib.snnlif_bn_fp(p(x), p(w), p(w), p(w), p(w), p(w), p(y), 7, 2, 2, C, 3, EPS, None) == cabi.ERR_DTYPE
    assert lib.snnlif_bn_fp(p(x), None, p(w), p(w), p(w), p(w), p(y), cabi.DTYPE_F32, 2, 2, C, 3, EPS, None) == cabi.ERR_ARG
    assert lib.snnlif_bn_fp(p(x), p(w), p(w), p(w), p(w), p(w), p(y), cabi.DTYPE_F32, -1, 2, C, 3, EPS, None) == cabi.ERR_ARG
    need = cabi.bn_bp_workspace_bytes(cabi.DTYPE_F32, 2, 2, C, 3)
    assert need > 0
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    assert lib.snnlif_bn_bp(p(x), p(w), p(w), p(w), p(x), p(y), p(w), p(w), cabi.DTYPE_F32, 2, 2, C, 3,
                            p(ws), need - 1, None) == cabi.ERR_WORKSPACE
    assert lib.snnlif_bn_bp(p(x), p(w), p(w), p(w), p(x), p(y), p(w), p(w), cabi.DTYPE_F32, 2, 2, C, 3,
                            None, 0, None) == cabi.ERR_WORKSPACE
    assert lib.snnlif_bn_bp_dist2(p(x), p(w), p(w), p(w), p(x), p(w), None, p(y), cabi.DTYPE_F32, 2, 2, C, 3,
                                  None) == cabi.ERR_ARG


def test_bn_full_size_properties(cabi):
    """[8,64,128,32,32] fp32 (256 MiB tensors): sampled channels against the oracle for the forward,
    and for the backward the properties that do not need one: grad_bias / grad_weight against float64
    sums of sampled channels, and the input gradient orthogonal to 1 and to xhat per channel."""
    from oracle import c_oracle
    shape = (8, 64, 128, 32, 32)
    T, B, C, HW = 8, 64, 128, 1024
    gen = torch.Generator(device="cuda").manual_seed(64)
    x = 0.5 + torch.randn(shape, generator=gen, device="cuda")
    g = torch.randn(shape, generator=gen, device="cuda")
    w = 0.5 + torch.rand(C, generator=gen, device="cuda")
    b = 0.2 * torch.randn(C, generator=gen, device="cuda")
    var, mean = torch.var_mean(x, dim=(0, 1, 3, 4), unbiased=False)
    ivar, y = torch.empty_like(var), torch.empty_like(x)
    cabi.bn_fp_into(x, w, b, var, mean, ivar, y, EPS)
    pick = [0, 1, 63, 127]
    take = lambda t: t[:, :, pick].contiguous().cpu().numpy()
    p = lambda t: t[pick].cpu().numpy()
    ivar_o, y_o = c_oracle.bn_forward(take(x), p(w), p(b), p(var), p(mean), EPS)
    assert np.array_equal(p(ivar), ivar_o) and np.array_equal(take(y), y_o)
    gx, gw, gb = torch.empty_like(x), torch.empty_like(w), torch.empty_like(w)
    ws = torch.empty(cabi.bn_bp_workspace_bytes(cabi.DTYPE_F32, T, B, C, HW), dtype=torch.uint8, device="cuda")
    cabi.bn_bp_into(x, w, ivar, mean, g, gx, gw, gb, ws)
    gx_o, gw_o, gb_o = c_oracle.bn_backward(take(x), p(w), ivar_o, p(mean), take(g))
    rel_close(p(gb), gb_o, "bias gradient")
    rel_close(p(gw), gw_o, "weight gradient")
    rel_close(take(gx), gx_o, "input gradient")
    sh = (1, 1, C, 1, 1)
    xhat = (x.double() - mean.double().view(sh)) * ivar.double().view(sh)
    dims = (0, 1, 3, 4)
    assert float(gx.double().sum(dim=dims).abs().max()) <= 1e-3 * float(gx.abs().sum(dim=dims).max())
    assert float((gx.double() * xhat).sum(dim=dims).abs().max()) <= 1e-3 * float((gx.abs() * xhat.abs()).sum(dim=dims).max())
