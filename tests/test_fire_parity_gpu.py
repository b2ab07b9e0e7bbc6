"""GPU parity of the HIP fire kernels against the CPU oracle, driven through the C ABI
(``include/snnlib_lif.h``) on seeded inputs.

Bars: spikes bit-exact; membrane potentials and input gradients compared for exact equality as
well (the kernels keep the reference's operation order and are built without FMA contraction), with
the stated tolerance of 1e-5 relative as the documented fallback bar.
"""
import numpy as np
import pytest
import torch

from conftest import ALPHA, BETA, INTERVAL, THRESH

pytestmark = pytest.mark.gpu

RTOL = 1e-5  # stated bar for membrane potentials and gradients (relative)


@pytest.fixture(scope="module")
def cabi():
    from snn_gpu_training_bptt_amd import lif_cabi
    lif_cabi.load()
    return lif_cabi


@pytest.fixture(scope="module")
def oracle():
    from oracle import c_oracle
    return c_oracle


def make_inputs(shape, mean, std, seed, dtype=torch.float32):
    gen = torch.Generator().manual_seed(seed)
    x = (mean + std * torch.randn(shape, generator=gen)).to(dtype)
    g = torch.randn(shape, generator=gen).to(dtype)
    return x, g


def run_gpu(cabi, x, g, alpha=ALPHA, thresh=THRESH, beta=BETA, interval=INTERVAL, keep=None):
    """`keep`: the cache hint (True: SNNLIF_KEEP_SPATIAL, False: SNNLIF_STREAM_SPATIAL, None: by size);
    it selects between two instantiations of every kernel, which must give the same bits."""
    xd, gd = x.cuda(), g.cuda()
    mem = torch.empty_like(xd)
    spike_a = torch.empty_like(xd)
    spike_b = torch.empty_like(xd)
    gx = torch.empty_like(xd)
    cabi.fire_s_fp_into(xd, spike_a, alpha, thresh, keep_spatial=keep)
    cabi.fire_us_fp_into(xd, mem, spike_b, alpha, thresh, keep_spatial=keep)
    code = {torch.float32: 0, torch.float64: 1, torch.bfloat16: 2}[x.dtype]
    T = x.shape[0]
    ws_bytes = cabi.fire_bp_workspace_bytes(code, T, x.numel() // T)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda") if ws_bytes else None
    cabi.fire_bp_into(xd, gd, gx, alpha, thresh, beta, interval, workspace=ws, keep_spatial=keep)
    torch.cuda.synchronize()
    return mem.cpu(), spike_a.cpu(), spike_b.cpu(), gx.cpu()


def assert_parity(oracle, x, g, outs, alpha=ALPHA, thresh=THRESH, beta=BETA, interval=INTERVAL):
    mem, spike_a, spike_b, gx = outs
    mem_o, spike_o = oracle.fire_forward(x.numpy(), alpha, thresh)
    gx_o = oracle.fire_backward(x.numpy(), g.numpy(), alpha, thresh, beta, interval)
    assert np.array_equal(spike_a.numpy(), spike_o), "spikes (fire_s_fp) differ from the oracle"
    assert np.array_equal(spike_b.numpy(), spike_o), "spikes (fire_us_fp) differ from the oracle"
    np.testing.assert_allclose(mem.numpy(), mem_o, rtol=RTOL, atol=0)
    np.testing.assert_allclose(gx.numpy(), gx_o, rtol=RTOL, atol=0)
    # stronger than the stated bar: same operation order, no contraction -> identical values
    assert np.array_equal(mem.numpy(), mem_o), "membrane potential not bit-identical"
    assert np.array_equal(gx.numpy(), gx_o), "input gradient not bit-identical"


CASES = [
    # (shape, mean, std)                                   what it covers
    ((4, 8, 16, 8, 8), 0.5, 1.0),       # configuration 1 (the reference's CPU-runnable case)
    ((6, 2, 8), 0.0, 1.0),              # the reference test's fc shape (test_utils.py:18)
    ((6, 2, 8, 8, 8), 0.0, 1.0),        # the reference test's conv shape (test_utils.py:24)
    ((8, 4, 16, 32, 32), 0.5, 1.0),     # T=8 register window, conv-like
    ((1, 3, 5), 0.5, 1.0),              # T=1, odd N -> scalar lanes
    ((3, 2, 7, 3), 0.5, 1.0),           # N=42: 2-wide lanes
    ((5, 1, 1), 0.5, 1.0),              # a single neuron
    ((7, 3, 1000), 0.5, 1.0),           # T=7 inside the T<=8 window
    ((12, 2, 64, 9), 0.3, 0.8),         # T=12 inside the T<=16 window
    ((16, 2, 32, 8, 8), 0.5, 1.0),      # T=16
    ((32, 2, 16, 16, 16), 0.3, 0.8),    # T=32 (configuration 3's window)
    ((29, 2, 300), 0.3, 0.8),           # T=29 inside the T<=32 window
    ((33, 2, 16, 8, 8), 0.3, 0.8),      # 32-step body with a one-step head
    ((70, 3, 129), 0.3, 0.8),           # 64-step body with a 6-step head, odd N
    ((64, 2, 500), 0.3, 0.8),           # a 64-step register window
    ((120, 2, 100), 0.3, 0.8),          # four segments, the last partial
    ((257, 2, 130), 0.2, 0.7),          # nine segments
    ((1024, 1, 192), 0.2, 0.7),         # the longest window kept on chip
    ((1030, 1, 64), 0.2, 0.7),          # beyond it: membrane potential staged in the workspace
]


# the cache hint: kept (what tensors this small get by themselves), streamed
HINTS = pytest.mark.parametrize("keep", [True, False], ids=["kept", "streamed"])


@HINTS
@pytest.mark.parametrize("shape,mean,std", CASES)
def test_fp32_parity(cabi, oracle, shape, mean, std, keep):
    x, g = make_inputs(shape, mean, std, seed=1234)
    assert_parity(oracle, x, g, run_gpu(cabi, x, g, keep=keep))
    if keep:   # no hint at all: by size, i.e. kept for these shapes
        assert_parity(oracle, x, g, run_gpu(cabi, x, g))


@HINTS
@pytest.mark.parametrize("T", list(range(1, 35)))
def test_fp32_every_window_length(cabi, oracle, T, keep):
    """Each window length up to 34 has a straight-line register window of its own or runs as the
    multiple of 8 below it preceded by a head of 1 to 7 steps.  Even and odd N.  The streamed forward
    requests windows of 9 to 16 and 24 to 31 steps whole, 17 to 23 in groups of 16, longer ones through
    a rolling window."""
    for n_inner in (256, 77):
        x, g = make_inputs((T, 2, n_inner), 0.4, 0.9, seed=1000 + T)
        assert_parity(oracle, x, g, run_gpu(cabi, x, g, alpha=0.3, keep=keep), alpha=0.3)


@pytest.mark.parametrize("T", [40, 48, 56, 64, 41, 47, 63, 65])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_windows_between_32_and_64(cabi, oracle, T, dtype):
    """40, 48, 56 and 64 steps run as one register window, their neighbours in two or three
    segments; both must give the oracle's bits.  Even and odd N."""
    for n_inner in (256, 77):
        x, g = make_inputs((T, 2, n_inner), 0.4, 0.9, seed=2000 + T, dtype=dtype)
        assert_parity(oracle, x, g, run_gpu(cabi, x, g, alpha=0.3), alpha=0.3)


@HINTS
@pytest.mark.parametrize("T,dtype", [(72, torch.float32), (80, torch.float32), (88, torch.float32),
                                     (96, torch.float32), (104, torch.float32), (95, torch.float32),
                                     (97, torch.float32), (112, torch.float32), (128, torch.float32),
                                     (72, torch.float64), (96, torch.float64),
                                     (40, torch.bfloat16), (64, torch.bfloat16), (72, torch.bfloat16),
                                     (96, torch.bfloat16), (104, torch.bfloat16), (100, torch.bfloat16)])
def test_windows_between_64_and_128(cabi, oracle, T, dtype, keep):
    """With 4-byte arithmetic (fp32 and bf16 storage) windows of 72, 80, 88, 96 and 104 steps still
    run as one register window; their neighbours, longer multiples of 8 and every fp64 window beyond
    64 steps run in segments.  Even N (bf16 pairs where the register budget allows) and odd N."""
    for n_inner in (256, 77):
        x32, g32 = make_inputs((T, 2, n_inner), 0.4, 0.9, seed=4000 + T)
        x, g = x32.to(dtype), g32.to(dtype)
        outs = run_gpu(cabi, x, g, alpha=0.3, keep=keep)
        if dtype == torch.bfloat16:
            mem, spike_a, spike_b, gx = outs
            mem_o, spike_o = oracle.fire_forward(x.float().numpy(), 0.3, THRESH)
            gx_o = oracle.fire_backward(x.float().numpy(), g.float().numpy(), 0.3, THRESH, BETA, INTERVAL)
            assert np.array_equal(spike_a.float().numpy(), spike_o)
            assert torch.equal(gx, torch.from_numpy(gx_o).bfloat16())
        else:
            assert_parity(oracle, x, g, outs, alpha=0.3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.bfloat16])
@pytest.mark.parametrize("T", [32, 33, 40, 47, 48, 49, 63, 64, 65, 100, 160, 161, 175, 1040, 1047])
def test_streamed_windows_from_32_steps_on(cabi, oracle, T, dtype):
    """The streamed forward of these windows is the rolling-window kernel (16 rows in flight, refilled
    row by row; lengths that are not a multiple of 16 skip the refills past the end and finish on a
    partial group of 1 to 15 rows): spikes, the membrane output and, beyond 1024 steps, the potential it
    stages in the backward's workspace (fp32 behind bf16 storage) must be the oracle's bits.  Even and
    odd N."""
    wide = torch.float64 if dtype == torch.float64 else torch.float32
    for n_inner in (256, 77):
        x32, g32 = make_inputs((T, 2, n_inner), 0.4, 0.9, seed=9000 + T)
        x, g = x32.to(dtype), g32.to(dtype)
        mem, spike_a, spike_b, gx = run_gpu(cabi, x, g, alpha=0.3, keep=False)
        mem_o, spike_o = oracle.fire_forward(x.to(wide).numpy(), 0.3, THRESH)
        gx_o = oracle.fire_backward(x.to(wide).numpy(), g.to(wide).numpy(), 0.3, THRESH, BETA, INTERVAL)
        as_stored = lambda a: torch.from_numpy(a).to(dtype)
        assert torch.equal(spike_a, as_stored(spike_o)) and torch.equal(spike_b, as_stored(spike_o))
        assert torch.equal(mem, as_stored(mem_o))
        assert torch.equal(gx, as_stored(gx_o))


@HINTS
@pytest.mark.parametrize("T", list(range(33, 114)))
def test_fp32_windows_with_a_head(cabi, oracle, T, keep):
    """Backward windows of 33 to 111 steps that are not a multiple of 8 run as a straight-line body of a
    multiple of 8 steps preceded by a head of 1-7 steps (every operand read once); multiples of 8 up to
    104 run without a head, 112 and 113 steps are the first lengths cut into segments again.  Every
    length, both instantiations, a negative threshold (a wrong spike flag or potential at the seam between
    head and body would show), odd N."""
    x, g = make_inputs((T, 3, 77), 0.1, 0.9, seed=11000 + T)
    xd, gd = x.cuda(), g.cuda()
    gx = torch.empty_like(xd)
    cabi.fire_bp_into(xd, gd, gx, 0.3, -0.25, BETA, INTERVAL, keep_spatial=keep)
    torch.cuda.synchronize()
    gx_o = oracle.fire_backward(x.numpy(), g.numpy(), 0.3, -0.25, BETA, INTERVAL)
    assert np.array_equal(gx.cpu().numpy(), gx_o)


@pytest.mark.parametrize("dtype", [torch.float64, torch.bfloat16])
@pytest.mark.parametrize("T", [33, 36, 39, 41, 47, 63, 65, 71, 73, 79, 100, 103, 105, 111])
def test_windows_with_a_head_other_storage_types(cabi, oracle, T, dtype):
    """The same in fp64 (heads up to a 64-step body, i.e. 71 steps; longer windows are segmented) and
    bf16 (two neurons per lane when N is even; bodies from 64 steps on stay segmented), with a dense gradient and with one row of gradient that
    stands for every step (row stride 0)."""
    wide = torch.float64 if dtype == torch.float64 else torch.float32
    for n_inner in (128, 77):
        x32, g32 = make_inputs((T, 2, n_inner), 0.1, 0.9, seed=12000 + T)
        x, g = x32.to(dtype), g32.to(dtype)
        for keep in (True, False):
            xd, gd = x.cuda(), g.cuda()
            gx = torch.empty_like(xd)
            cabi.fire_bp_into(xd, gd, gx, 0.3, THRESH, BETA, INTERVAL, keep_spatial=keep)
            gx1 = torch.empty_like(xd)
            cabi.fire_bp_into(xd, gd[:1].expand_as(xd), gx1, 0.3, THRESH, BETA, INTERVAL, keep_spatial=keep)
            torch.cuda.synchronize()
            xw, gw = x.to(wide).numpy(), g.to(wide).numpy()
            gx_o = oracle.fire_backward(xw, gw, 0.3, THRESH, BETA, INTERVAL)
            gx1_o = oracle.fire_backward(xw, np.ascontiguousarray(np.broadcast_to(gw[:1], gw.shape)), 0.3,
                                         THRESH, BETA, INTERVAL)
            assert torch.equal(gx.cpu(), torch.from_numpy(gx_o).to(dtype))
            assert torch.equal(gx1.cpu(), torch.from_numpy(gx1_o).to(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.bfloat16])
@pytest.mark.parametrize("T", [33, 34, 39, 57, 63, 65, 66, 71, 95, 97, 105, 112, 115, 120, 127, 129, 138, 140, 159,
                               160, 161, 191, 193, 200, 250, 1023])
def test_segmented_windows(cabi, oracle, T, dtype):
    """Windows cut into 32-step segments, the last one partial (fp64, bf16) or a long register window of
    64 + T mod 32 steps with a body of 64, 72, 80 or 88 steps (fp32): one step into a new segment (33, 65, 97,
    129, 161, 193), one short of a full one (63, 95, 127, 159, 191, 1023), whole segments only (160), many
    segments (250, 1023), every body length of the fp32 tail (129 / 138, 140 / 112, 115 / 120, 127).  A negative threshold makes a wrong spike flag at the start of the window
    visible.  Even and odd N."""
    for n_inner, thresh in ((128, THRESH), (77, -0.25)):
        x32, g32 = make_inputs((T, 2, n_inner), 0.1, 0.9, seed=7000 + T)
        x, g = x32.to(dtype), g32.to(dtype)
        xd = x.cuda()
        gx = torch.empty_like(xd)
        cabi.fire_bp_into(xd, g.cuda(), gx, 0.3, thresh, BETA, INTERVAL)
        torch.cuda.synchronize()
        wide = torch.float64 if dtype == torch.float64 else torch.float32
        gx_o = oracle.fire_backward(x.to(wide).numpy(), g.to(wide).numpy(), 0.3, thresh, BETA, INTERVAL)
        if dtype == torch.bfloat16:
            assert torch.equal(gx.cpu(), torch.from_numpy(gx_o).bfloat16())
        else:
            assert np.array_equal(gx.cpu().numpy(), gx_o)


@pytest.mark.parametrize("T", [1, 2])
@pytest.mark.parametrize("n_inner", [4096, 4098, 4097, 8])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_very_short_windows_use_wide_lanes(cabi, oracle, T, n_inner, dtype):
    """One- and two-step windows move 16 bytes per lane when N and the bases allow it (N a multiple
    of 4 for fp32), 8 or one element otherwise; every width must give the oracle's bits."""
    x, g = make_inputs((T, 3, n_inner), 0.4, 0.9, seed=3000 + T + n_inner, dtype=dtype)
    assert_parity(oracle, x, g, run_gpu(cabi, x, g, alpha=0.3), alpha=0.3)


@pytest.mark.parametrize("alpha,thresh,beta,interval", [
    (0.3, 0.5, 1.0, 0.5),      # decay that is not a power of two: exposes any FMA contraction
    (0.25, 0.25, 1.0, 0.5),    # the reference's default threshold (snnlib_func.py:14)
    (0.9, 1.0, 0.7, 0.3),
    (0.0, 0.5, 1.0, 0.5),      # no memory: per-step Heaviside
    (1.0, 0.5, 2.0, 1.5),
])
def test_fp32_parity_hyperparameters(cabi, oracle, alpha, thresh, beta, interval):
    x, g = make_inputs((8, 4, 32, 8, 8), 0.5, 1.0, seed=7)
    assert_parity(oracle, x, g, run_gpu(cabi, x, g, alpha, thresh, beta, interval),
                  alpha, thresh, beta, interval)


@HINTS
@pytest.mark.parametrize("shape", [(8, 4, 16, 8, 8), (6, 3, 7), (13, 2, 50), (16, 3, 33), (20, 2, 64), (33, 2, 10),
                                   (100, 2, 33), (1024, 1, 40), (1100, 1, 16)])
def test_fp64_parity(cabi, oracle, shape, keep):
    x, g = make_inputs(shape, 0.5, 1.0, seed=99, dtype=torch.float64)
    assert_parity(oracle, x, g, run_gpu(cabi, x, g, alpha=0.3, keep=keep), alpha=0.3)


def test_empty_shapes_are_noops(cabi):
    for shape in [(0, 4, 8), (4, 0, 8), (4, 2, 0)]:
        x = torch.empty(shape, device="cuda")
        spike = torch.empty_like(x)
        gx = torch.empty_like(x)
        cabi.fire_s_fp_into(x, spike, ALPHA, THRESH)
        cabi.fire_bp_into(x, x, gx, ALPHA, THRESH, BETA, INTERVAL)
    torch.cuda.synchronize()


def test_argument_errors(cabi):
    lib = cabi.load()
    x = torch.zeros(4, 8, device="cuda")
    assert lib.snnlif_fire_s_fp(x.data_ptr(), None, 0, 4, 8, ALPHA, THRESH, None) == cabi.ERR_ARG
    assert lib.snnlif_fire_s_fp(x.data_ptr(), x.data_ptr(), 9, 4, 8, ALPHA, THRESH, None) == cabi.ERR_DTYPE
    both = cabi.KEEP_SPATIAL | cabi.STREAM_SPATIAL       # contradictory hints, unknown flag bits
    assert lib.snnlif_fire_s_fp(x.data_ptr(), x.data_ptr(), both, 4, 8, ALPHA, THRESH, None) == cabi.ERR_DTYPE
    assert lib.snnlif_fire_s_fp(x.data_ptr(), x.data_ptr(), 0x400, 4, 8, ALPHA, THRESH, None) == cabi.ERR_DTYPE
    assert lib.snnlif_fire_bp(x.data_ptr(), x.data_ptr(), x.data_ptr(), both, 4, 8, ALPHA, THRESH, BETA, INTERVAL,
                              None, 0, None) == cabi.ERR_DTYPE
    assert lib.snnlif_fire_s_fp(x.data_ptr(), x.data_ptr(), 0, -1, 8, ALPHA, THRESH, None) == cabi.ERR_ARG
    assert lib.snnlif_fire_s_fp(x.data_ptr() + 2, x.data_ptr(), 0, 2, 4, ALPHA, THRESH, None) == cabi.ERR_ALIGN
    big = torch.zeros(1100, 8, device="cuda")
    rc = lib.snnlif_fire_bp(big.data_ptr(), big.data_ptr(), big.data_ptr(), 0, 1100, 8,
                            ALPHA, THRESH, BETA, INTERVAL, None, 0, None)
    assert rc == cabi.ERR_WORKSPACE
    torch.cuda.synchronize()


def test_misaligned_views_take_narrow_lanes(cabi, oracle):
    """A base pointer that is only 4-byte aligned must still give the oracle's bits."""
    x, g = make_inputs((8, 2, 1024), 0.5, 1.0, seed=5)
    T, N = 8, 2048
    pad = 1  # one float: 4-byte aligned, not 16
    xd = torch.empty(T * N + pad, device="cuda")[pad:].view(T, 2, 1024).copy_(x)
    gd = torch.empty(T * N + pad, device="cuda")[pad:].view(T, 2, 1024).copy_(g)
    spike = torch.empty(T * N + pad, device="cuda")[pad:].view(T, 2, 1024)
    gx = torch.empty(T * N + pad, device="cuda")[pad:].view(T, 2, 1024)
    cabi.fire_s_fp_into(xd, spike, ALPHA, THRESH)
    cabi.fire_bp_into(xd, gd, gx, ALPHA, THRESH, BETA, INTERVAL)
    torch.cuda.synchronize()
    _, spike_o = oracle.fire_forward(x.numpy(), ALPHA, THRESH)
    gx_o = oracle.fire_backward(x.numpy(), g.numpy(), ALPHA, THRESH, BETA, INTERVAL)
    assert np.array_equal(spike.cpu().numpy(), spike_o)
    assert np.array_equal(gx.cpu().numpy(), gx_o)


def test_special_values_follow_ieee_like_the_oracle(cabi, oracle):
    """Denormals (must not be flushed), signed zeros, infinities and NaNs in the input current and in
    the spike gradient: the kernels must produce the oracle's values, NaNs in the same places."""
    T, N = 6, 512
    gen = torch.Generator().manual_seed(4321)
    x = 0.5 + torch.randn((T, 1, N), generator=gen)
    g = torch.randn((T, 1, N), generator=gen)
    specials = torch.tensor([1e-40, -1e-40, 1.4e-45, 0.0, -0.0, float("inf"), -float("inf"),
                             float("nan"), 3.0e38, -3.0e38, 0.5, 1.0, 1.17549435e-38])
    for k, v in enumerate(specials):
        x[k % T, 0, 7 * k] = v            # one special per neuron, at varying time steps
        g[(k + 2) % T, 0, 7 * k + 100] = v
    x[:, 0, 300:364] *= 1e-39             # whole neurons in the denormal range
    g[:, 0, 364:428] *= 1e-41
    alpha, thresh, beta, interval = 0.5, 0.0, 1.0, 1.0e38   # wide window so denormal paths carry gradient
    outs = run_gpu(cabi, x, g, alpha, thresh, beta, interval)
    mem, spike_a, spike_b, gx = (o.numpy() for o in outs)
    mem_o, spike_o = oracle.fire_forward(x.numpy(), alpha, thresh)
    gx_o = oracle.fire_backward(x.numpy(), g.numpy(), alpha, thresh, beta, interval)
    assert np.array_equal(spike_a, spike_o) and np.array_equal(spike_b, spike_o)
    assert np.array_equal(np.isnan(mem), np.isnan(mem_o))
    assert np.array_equal(mem[~np.isnan(mem)], mem_o[~np.isnan(mem_o)])
    assert np.array_equal(np.isnan(gx), np.isnan(gx_o))
    assert np.array_equal(gx[~np.isnan(gx)], gx_o[~np.isnan(gx_o)])
    # the denormal neurons really exercised denormal arithmetic
    assert (np.abs(mem_o[:, 0, 300:364]) < 1.2e-38).all() and (mem_o[:, 0, 300:364] != 0).any()


@HINTS
@pytest.mark.parametrize("shape", [(8, 3, 255), (5, 1, 1), (16, 2, 4097), (33, 3, 77), (12, 4, 64, 4, 4),
                                   (48, 2, 130), (64, 2, 77), (64, 3, 256), (1024, 1, 128), (1040, 1, 30)])
def test_bf16_storage_parity_including_odd_sizes(cabi, oracle, shape, keep):
    """bf16 storage, fp32 arithmetic: two values per lane when N is even and the bases are 4-byte
    aligned, one otherwise.  Expected = the fp32 oracle on the bf16-rounded inputs, outputs rounded
    once to bf16 (spikes are exact either way)."""
    x32, g32 = make_inputs(shape, 0.5, 1.0, seed=2468)
    x, g = x32.bfloat16(), g32.bfloat16()
    mem, spike_a, spike_b, gx = run_gpu(cabi, x, g, keep=keep)
    mem_o, spike_o = oracle.fire_forward(x.float().numpy(), ALPHA, THRESH)
    gx_o = oracle.fire_backward(x.float().numpy(), g.float().numpy(), ALPHA, THRESH, BETA, INTERVAL)
    assert np.array_equal(spike_a.float().numpy(), spike_o)
    assert np.array_equal(spike_b.float().numpy(), spike_o)
    assert torch.equal(mem, torch.from_numpy(mem_o).bfloat16())
    assert torch.equal(gx, torch.from_numpy(gx_o).bfloat16())


def test_bf16_misaligned_base_takes_single_lanes(cabi, oracle):
    T, N = 8, 1024
    x32, g32 = make_inputs((T, 1, N), 0.5, 1.0, seed=1357)
    x, g = x32.bfloat16(), g32.bfloat16()
    off = 1  # one bf16: 2-byte aligned only
    view = lambda: torch.empty(T * N + off, dtype=torch.bfloat16, device="cuda")[off:].view(T, 1, N)
    xd, gd, spike, gx = view().copy_(x), view().copy_(g), view(), view()
    assert xd.data_ptr() % 4 == 2
    cabi.fire_s_fp_into(xd, spike, ALPHA, THRESH)
    cabi.fire_bp_into(xd, gd, gx, ALPHA, THRESH, BETA, INTERVAL)
    torch.cuda.synchronize()
    _, spike_o = oracle.fire_forward(x.float().numpy(), ALPHA, THRESH)
    gx_o = oracle.fire_backward(x.float().numpy(), g.float().numpy(), ALPHA, THRESH, BETA, INTERVAL)
    assert np.array_equal(spike.float().cpu().numpy(), spike_o)
    assert torch.equal(gx.cpu(), torch.from_numpy(gx_o).bfloat16())


def _backward_with_gradient_layout(cabi, x, g_rows, alpha, keep=None):
    """Backward through the C ABI with ``g_rows`` (a device tensor of x's shape, any time-axis layout)."""
    xd = x.cuda()
    gx = torch.empty_like(xd)
    code = {torch.float32: 0, torch.float64: 1, torch.bfloat16: 2}[x.dtype]
    T = x.shape[0]
    ws_bytes = cabi.fire_bp_workspace_bytes(code, T, x.numel() // T)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda") if ws_bytes else None
    cabi.fire_bp_into(xd, g_rows, gx, alpha, THRESH, BETA, INTERVAL, workspace=ws, keep_spatial=keep)
    torch.cuda.synchronize()
    return gx.cpu()


@HINTS
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.bfloat16])
@pytest.mark.parametrize("T", [1, 2, 8, 9, 16, 31, 32, 50, 64, 96, 130, 1030])
def test_gradient_expanded_over_time_is_read_in_place(cabi, oracle, T, dtype, keep):
    """A gradient that is one [N] row for every time step (stride 0 on the time axis, what autograd
    hands over after ``spike.sum(dim=0)``) goes to ``snnlif_fire_bp_strided`` as it is.  The result
    must be the oracle's on the gradient made dense, and the bits of the dense call: every kernel
    form of the backward (register windows with and without a head, wide windows, segments, workspace
    stream) takes the row stride.  Even N (pairs of bf16 per lane) and odd N."""
    for n_inner in (256, 77):
        x32, g32 = make_inputs((T, 2, n_inner), 0.4, 0.9, seed=5000 + T)
        x = x32.to(dtype)
        row = g32[0].to(dtype)
        g_dense = row.unsqueeze(0).expand(T, 2, n_inner).contiguous()
        g_view = row.cuda().unsqueeze(0).expand(T, 2, n_inner)
        assert T == 1 or g_view.stride(0) == 0
        gx = _backward_with_gradient_layout(cabi, x, g_view, 0.3, keep)
        gx_dense = _backward_with_gradient_layout(cabi, x, g_dense.cuda(), 0.3, keep)
        assert torch.equal(gx, gx_dense)
        wide = torch.float64 if dtype == torch.float64 else torch.float32
        gx_o = oracle.fire_backward(x.to(wide).numpy(), g_dense.to(wide).numpy(), 0.3, THRESH, BETA, INTERVAL)
        if dtype == torch.bfloat16:
            assert torch.equal(gx, torch.from_numpy(gx_o).bfloat16())
        else:
            np.testing.assert_allclose(gx.numpy(), gx_o, rtol=RTOL, atol=0)
            assert np.array_equal(gx.numpy(), gx_o)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,pad", [(8, 1), (8, 64), (20, 3), (96, 2), (50, 5)])
def test_gradient_rows_of_a_wider_tensor(cabi, oracle, T, pad, dtype):
    """Time rows further apart than N (a slice of a wider tensor).  An odd pitch forces single bf16
    lanes even for even N."""
    n_inner = 128
    x32, g32 = make_inputs((T, 2, n_inner), 0.4, 0.9, seed=6000 + T)
    x, g = x32.to(dtype), g32.to(dtype)
    N = 2 * n_inner
    backing = torch.full((T, N + pad), float("nan"), dtype=dtype, device="cuda")
    backing[:, :N] = g.reshape(T, N).cuda()
    g_view = backing[:, :N].unflatten(1, (2, n_inner))
    assert g_view.stride(0) == N + pad and not g_view.is_contiguous()
    gx = _backward_with_gradient_layout(cabi, x, g_view, 0.3)
    gx_dense = _backward_with_gradient_layout(cabi, x, g.cuda(), 0.3)
    assert torch.equal(gx, gx_dense)
    assert not torch.isnan(gx.float()).any()


def test_gradient_row_stride_is_validated(cabi):
    lib = cabi.load()
    x = torch.zeros(4, 64, device="cuda")
    g = torch.zeros(4, 64, device="cuda")
    gx = torch.empty(4, 64, device="cuda")
    args = (x.data_ptr(), g.data_ptr(), gx.data_ptr(), 0, 4, 64)
    tail = (0.25, 0.5, 1.0, 0.5, None, 0, None)
    assert lib.snnlif_fire_bp_strided(*args, -1, *tail) == cabi.ERR_ARG
    assert lib.snnlif_fire_bp_strided(*args, 63, *tail) == cabi.ERR_ARG      # rows would overlap
    assert lib.snnlif_fire_bp_strided(*args, 1, *tail) == cabi.ERR_ARG
    assert lib.snnlif_fire_bp_strided(*args, 64, *tail) == cabi.OK
    assert lib.snnlif_fire_bp_strided(*args, 0, *tail) == cabi.OK
    torch.cuda.synchronize()
    with pytest.raises(ValueError):   # rows that are not dense themselves
        cabi.fire_bp_into(x, torch.zeros(4, 128, device="cuda")[:, ::2], gx, 0.25, 0.5, 1.0, 0.5)
