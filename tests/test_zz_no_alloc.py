"""The batch-norm + fire backward that allocates nothing (``snnlif_bn_fire_bp_static``): its partial
sums live in a fixed device array inside the library instead of a caller workspace.  Checked through
the C ABI against ``snnlif_bn_fire_bp`` (same kernels, so bit for bit), on consecutive calls that
share the array -- the later ones smaller than the first, so stale partial sums of the earlier call
sit right behind the region the later call uses.
"""
import numpy as np
import pytest
import torch

from conftest import ALPHA, BETA, INTERVAL, THRESH

pytestmark = pytest.mark.gpu
EPS = 1e-5


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


@pytest.fixture(scope="module")
def cabi():
    from snn_gpu_training_bptt_amd import lif_cabi
    lif_cabi.load()
    return lif_cabi


def both_backwards(cabi, shape, seed, dtype=torch.float32):
    x, g, w, b, var, mean = (t.to(dtype).cuda() for t in make(shape, seed))
    T, B, C = shape[:3]
    HW = int(np.prod(shape[3:])) if len(shape) > 3 else 1
    ivar, spike = torch.empty_like(var), torch.empty_like(x)
    cabi.bn_fire_s_fp_into(x, w, b, var, mean, ivar, spike, EPS, ALPHA, THRESH)
    code = cabi.DTYPE_F32 if dtype == torch.float32 else cabi.DTYPE_F64
    need = cabi.bn_fire_bp_workspace_bytes(code, T, B, C, HW)
    assert 0 < need <= cabi.STATIC_SCRATCH_BYTES
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    want = [torch.empty_like(x), torch.empty_like(w), torch.empty_like(w)]
    cabi.bn_fire_bp_into(x, w, b, ivar, mean, g, *want, ALPHA, THRESH, BETA, INTERVAL, ws)
    got = [torch.full_like(x, float("nan")), torch.full_like(w, float("nan")), torch.full_like(w, float("nan"))]
    cabi.bn_fire_bp_static_into(x, w, b, ivar, mean, g, *got, ALPHA, THRESH, BETA, INTERVAL)
    torch.cuda.synchronize()
    return got, want


# each group: calls made one after the other on the same GPU; every later shape is smaller
SEQUENCES = [
    [(8, 16, 32, 16, 16), (4, 4, 8, 8, 8)],          # one partial per wavefront
    [(6, 32, 64), (3, 8, 16)],                       # fully connected: one partial per neuron
    [(8, 8, 16, 7, 7), (5, 2, 9, 31), (6, 2, 8)],    # switches between the two layouts
    [(40, 4, 8, 8, 8), (33, 2, 6, 4, 4)],            # segmented windows
    [(1030, 2, 4, 8, 8), (1025, 1, 6)],              # boundary potentials in the array as well
]


@pytest.mark.parametrize("shapes", SEQUENCES)
def test_static_scratch_backward_equals_workspace_backward(cabi, shapes):
    for k, shape in enumerate(shapes):
        got, want = both_backwards(cabi, shape, seed=70 + k)
        for a, b, what in zip(got, want, ("input-current gradient", "weight gradient", "bias gradient")):
            assert torch.equal(a, b), f"{what} differs at shape {shape} (call {k} of the sequence)"


def test_static_scratch_backward_double_precision(cabi):
    for k, shape in enumerate([(6, 4, 8, 8, 8), (4, 2, 4, 4, 8)]):
        got, want = both_backwards(cabi, shape, seed=80 + k, dtype=torch.float64)
        for a, b in zip(got, want):
            assert torch.equal(a, b)


def test_static_scratch_backward_rejects_what_does_not_fit(cabi):
    lib = cabi.load()
    x = torch.zeros(2, 1, 8, device="cuda")
    p = torch.ones(8, device="cuda")
    args = lambda T, B, C, HW: (x.data_ptr(), p.data_ptr(), p.data_ptr(), p.data_ptr(), p.data_ptr(), x.data_ptr(),
                                x.data_ptr(), p.data_ptr(), p.data_ptr(), cabi.DTYPE_F32, T, B, C, HW,
                                ALPHA, THRESH, BETA, INTERVAL, None)
    # 2 partials x 4 bytes x (3 Mi neurons) > 16 MiB: refused before anything is launched
    assert cabi.bn_fire_bp_workspace_bytes(cabi.DTYPE_F32, 2, 3 << 10, 1 << 10, 1) > cabi.STATIC_SCRATCH_BYTES
    assert lib.snnlif_bn_fire_bp_static(*args(2, 3 << 10, 1 << 10, 1)) == cabi.ERR_SCRATCH
    assert "SNNLIF_STATIC_SCRATCH_BYTES" in cabi.strerror(cabi.ERR_SCRATCH)
    assert lib.snnlif_bn_fire_bp_static(*args(0, 4, 8, 1)) == cabi.OK           # empty: no-op
    torch.cuda.synchronize()
