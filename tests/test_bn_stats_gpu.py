"""Per-channel batch statistics (``snnlif_bn_stats``) and sums (``snnlif_channel_sum``) on the GPU, through
the C ABI.

What it replaces is a library routine -- ``torch.var_mean(x, dim_bn, unbiased=False)`` in the
reference's layers (snnlib/example/snnlib_op.py:78) and ``torch.mean(x)``, ``torch.mean(x**2)`` in the
sharded ones (:265-266) -- so that routine, evaluated in float64 on the same values, is the checker:
fp32 results within 1e-6 of it (relative to the statistic's scale), fp64 within 1e-13.  The per-channel sum
replaces ``at::sum(grad_conv, dim_conv)``, the bias gradient of the layers that end in a convolution
(snnlib/cuda/snn_kernel_bp.cu:1261, 1338, 1401, 1435): checked against the float64 sum of the same
values (the result is that sum rounded once, up to 1e-12 of sum|x| of accumulation error) and exactly on
integer-valued inputs.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

SHAPES = [
    (6, 2, 8),                # the reference test's fc shape: one position per channel
    (6, 2, 8, 8, 8),          # the reference test's conv shape
    (8, 16, 32, 16, 16),      # HW = 256: four wavefronts per plane
    (4, 5, 7, 7, 7),          # HW = 49: one partly idle wavefront per plane
    (6, 3, 6, 14, 14),        # HW = 196
    (5, 2, 3, 4, 8),          # HW = 32: the smallest plane-aligned case
    (5, 2, 9, 31),            # HW = 31: column layout
    (13, 3, 20, 5, 3),        # 13 steps: two groups of rows, the second partial
    (32, 2, 16, 4, 4),
    (33, 2, 6, 8, 8),
    (100, 3, 20),
    (1024, 1, 4, 6, 6),
    (1, 1, 5, 1),             # a single value per channel: variance 0
    (8, 64, 1024),            # fully connected, many channels
    (8, 256, 16),             # fully connected, few channels: many row slices
    (3, 7, 300, 3, 3),        # HW = 9, more columns than one workgroup holds
    (8, 32, 128, 32, 32),     # few channels, many positions
    (4, 64, 16, 8, 8),        # 4 steps: a lane sums four batch entries' worth (16 row slices)
    (2, 6, 5, 8, 8),          # 12 rows: one slice, one partial group
    (1, 64, 8, 16, 16),       # a single step: sixteen batch entries per lane
    (3, 5, 4, 6, 6),          # 15 rows in one slice
    (6, 64, 8, 8, 8),         # 384 rows in 24 slices of exactly 16
    (7, 9, 4, 8, 8),          # 63 rows in 3 slices of 21: one whole group and a five-row tail
    (8, 64, 8, 8, 8),         # the headline window: 32 slices, two batch entries per lane
    (16, 4, 8, 8, 8),         # 16 steps: one slice per batch entry, one whole group
    (40, 3, 4, 8, 8),         # 40 steps: two whole groups and an eight-row tail per batch entry
]


@pytest.fixture(scope="module")
def cabi():
    from snn_gpu_training_bptt_amd import lif_cabi
    lif_cabi.load()
    return lif_cabi


def dims_of(shape):
    T, B, C = shape[:3]
    HW = int(np.prod(shape[3:])) if len(shape) > 3 else 1
    return T, B, C, HW


def run_stats(cabi, x, raw_moments=False):
    T, B, C, HW = dims_of(tuple(x.shape))
    code = cabi.DTYPE_F32 if x.dtype == torch.float32 else cabi.DTYPE_F64
    ws = torch.empty(cabi.bn_stats_workspace_bytes(code, T, B, C, HW), dtype=torch.uint8, device="cuda")
    mean = torch.full((C,), float("nan"), dtype=x.dtype, device="cuda")
    second = torch.full((C,), float("nan"), dtype=x.dtype, device="cuda")
    cabi.bn_stats_into(x, mean, second, ws, raw_moments=raw_moments)
    torch.cuda.synchronize()
    return mean.cpu(), second.cpu()


def make(shape, seed, dtype=torch.float32, offset=0.5):
    gen = torch.Generator().manual_seed(seed)
    C = shape[2]
    per_channel = (C,) + (1,) * (len(shape) - 3)
    x = offset + torch.randn(per_channel, generator=gen) + torch.randn(shape, generator=gen) * (
        0.5 + torch.rand(per_channel, generator=gen))
    return x.to(dtype)


def reference(x):
    dims = tuple(d for d in range(x.dim()) if d != 2)
    var, mean = torch.var_mean(x.double(), dim=dims, unbiased=False)
    return mean, var, torch.mean(x.double() ** 2, dim=dims)


def assert_close(got, want, scale, tol, what):
    err = (got.double() - want).abs()
    assert bool((err <= tol * scale + 1e-300).all()), \
        f"{what}: max error {err.max().item():.3e} against scale {scale.max().item():.3e} (tolerance {tol})"


@pytest.mark.parametrize("shape", SHAPES)
def test_fp32_statistics_against_float64_var_mean(cabi, shape):
    x = make(shape, seed=51)
    mean_ref, var_ref, second_ref = reference(x)
    spread = var_ref.sqrt() + mean_ref.abs() + 1e-30
    mean, var = run_stats(cabi, x.cuda())
    assert_close(mean, mean_ref, spread, 1e-6, "mean")
    assert_close(var, var_ref, var_ref + 1e-30, 1e-6, "biased variance")
    first, second = run_stats(cabi, x.cuda(), raw_moments=True)
    assert torch.equal(first, mean)
    assert_close(second, second_ref, second_ref + 1e-30, 1e-6, "second raw moment")
    # fixed summation order: the same bits on every call
    again = run_stats(cabi, x.cuda())
    assert torch.equal(again[0], mean) and torch.equal(again[1], var)


@pytest.mark.parametrize("shape", [(6, 2, 8), (6, 2, 8, 8, 8), (8, 16, 32, 16, 16), (4, 5, 7, 7, 7), (5, 2, 9, 31),
                                   (13, 3, 20, 5, 3), (8, 64, 256)])
def test_fp64_statistics(cabi, shape):
    x = make(shape, seed=52, dtype=torch.float64)
    mean_ref, var_ref, second_ref = reference(x)
    mean, var = run_stats(cabi, x.cuda())
    assert_close(mean, mean_ref, var_ref.sqrt() + mean_ref.abs() + 1e-300, 1e-13, "mean")
    assert_close(var, var_ref, var_ref + 1e-300, 1e-13, "biased variance")
    _, second = run_stats(cabi, x.cuda(), raw_moments=True)
    assert_close(second, second_ref, second_ref + 1e-300, 1e-13, "second raw moment")


@pytest.mark.parametrize("shape", [(8, 16, 8, 16, 16), (8, 64, 32)])
def test_variance_survives_a_mean_far_from_zero(cabi, shape):
    """|mean| = 1000 standard deviations: E[x^2] - E[x]^2 in float32 would keep no correct digit; the
    shifted sums still resolve the variance of the float32 values to 1e-6."""
    x = make(shape, seed=53, offset=1000.0)
    mean_ref, var_ref, _ = reference(x)
    assert float((mean_ref.abs() / var_ref.sqrt()).min()) > 300
    mean, var = run_stats(cabi, x.cuda())
    assert_close(mean, mean_ref, mean_ref.abs(), 1e-7, "mean")
    assert_close(var, var_ref, var_ref, 1e-6, "biased variance")


@pytest.mark.parametrize("shape", [(8, 16, 8, 16, 16), (8, 64, 32), (5, 2, 9, 31)])
@pytest.mark.parametrize("distance", [100.0, 1000.0])
def test_variance_survives_an_outlier_as_the_shift(cabi, shape, distance):
    """The sums are shifted by each channel's first element (t = 0, b = 0, position 0).  Make that element
    an outlier, `distance` standard deviations from the channel's mean: the shift is then a poor guess of
    the mean, the shifted squares are `distance`^2 times the variance, and sums of squares taken in
    float32 would lose 6e-8 * distance^2 of it (6e-4 and 6e-2 here).  Formed in double they must still
    meet the 1e-6 bar."""
    x = make(shape, seed=54)
    C = shape[2]
    flat = x.reshape(shape[0], shape[1], C, -1)
    sigma = flat.double().std(dim=(0, 1, 3))
    flat[0, 0, :, 0] += (distance * sigma).float()
    mean_ref, var_ref, second_ref = reference(x)
    mean, var = run_stats(cabi, x.cuda())
    assert_close(mean, mean_ref, var_ref.sqrt() + mean_ref.abs(), 1e-6, "mean")
    assert_close(var, var_ref, var_ref, 1e-6, "biased variance")
    _, second = run_stats(cabi, x.cuda(), raw_moments=True)
    assert_close(second, second_ref, second_ref, 1e-6, "second raw moment")


def test_constant_channels_have_zero_variance(cabi):
    x = torch.full((4, 3, 5, 6, 6), 0.75)
    x[:, :, 2] = -3.0
    mean, var = run_stats(cabi, x.cuda())
    assert torch.equal(var, torch.zeros(5))
    assert torch.equal(mean, torch.tensor([0.75, 0.75, -3.0, 0.75, 0.75]))


def test_full_size_headline_shape(cabi):
    """[8, 64, 128, 32, 32]: 524 288 values per channel, generated on the device."""
    gen = torch.Generator(device="cuda").manual_seed(54)
    x = 0.5 + torch.randn((8, 64, 128, 32, 32), generator=gen, device="cuda")
    var_ref, mean_ref = torch.var_mean(x.double(), dim=(0, 1, 3, 4), unbiased=False)
    mean, var = run_stats(cabi, x)
    assert_close(mean, mean_ref.cpu(), (var_ref.sqrt() + mean_ref.abs()).cpu(), 1e-6, "mean")
    assert_close(var, var_ref.cpu(), var_ref.cpu(), 1e-6, "biased variance")


def run_sum(cabi, g):
    T, B, C, HW = dims_of(tuple(g.shape))
    code = cabi.DTYPE_F32 if g.dtype == torch.float32 else cabi.DTYPE_F64
    ws = torch.empty(cabi.bn_stats_workspace_bytes(code, T, B, C, HW), dtype=torch.uint8, device="cuda")
    total = torch.full((C,), float("nan"), dtype=g.dtype, device="cuda")
    cabi.channel_sum_into(g, total, ws)
    torch.cuda.synchronize()
    return total.cpu()


@pytest.mark.parametrize("shape", SHAPES)
def test_fp32_channel_sums_against_float64_sum(cabi, shape):
    g = make(shape, seed=56, offset=0.0)
    dims = tuple(d for d in range(g.dim()) if d != 2)
    want = g.double().sum(dim=dims)
    mass = g.double().abs().sum(dim=dims)
    got = run_sum(cabi, g.cuda())
    err = (got.double() - want).abs()
    # the double-precision sum rounded once to float32 (2^-24 relative) + accumulation error
    assert bool((err <= 6.1e-8 * want.abs() + 1e-12 * mass).all()), f"max error {err.max().item():.3e}"
    assert torch.equal(run_sum(cabi, g.cuda()), got)   # fixed summation order


@pytest.mark.parametrize("shape", [(6, 2, 8), (6, 2, 8, 8, 8), (8, 16, 32, 16, 16), (4, 5, 7, 7, 7), (5, 2, 9, 31),
                                   (13, 3, 20, 5, 3)])
def test_fp64_channel_sums(cabi, shape):
    g = make(shape, seed=57, dtype=torch.float64, offset=0.0)
    dims = tuple(d for d in range(g.dim()) if d != 2)
    want, mass = g.sum(dim=dims), g.abs().sum(dim=dims)
    err = (run_sum(cabi, g.cuda()) - want).abs()
    assert bool((err <= 1e-13 * mass).all()), f"max error {err.max().item():.3e}"


@pytest.mark.parametrize("shape", [(6, 2, 8, 8, 8), (4, 5, 7, 7, 7), (13, 3, 20, 5, 3), (8, 16, 32, 16, 16),
                                   (3, 7, 300, 3, 3), (7, 9, 4, 8, 8), (40, 3, 4, 8, 8), (8, 64, 32)])
def test_channel_sums_of_small_integers_are_exact(cabi, shape):
    """Every element a small integer that depends on its step, batch entry, channel and position: all
    sums are exact in any order, so an element left out, read twice or credited to another channel shows."""
    T, B, C, HW = dims_of(shape)
    t = torch.arange(T).view(T, 1, 1, 1)
    b = torch.arange(B).view(1, B, 1, 1)
    c = torch.arange(C).view(1, 1, C, 1)
    i = torch.arange(HW).view(1, 1, 1, HW)
    g = ((3 * t + 5 * b + 7 * c + 11 * i) % 13 - 6 + (c % 3)).to(torch.float32)   # |g| <= 8
    want = g.sum(dim=(0, 1, 3))
    assert int(want.abs().max()) < 2 ** 24
    got = run_sum(cabi, g.reshape(shape).cuda())
    assert torch.equal(got, want)


def test_channel_sum_argument_errors(cabi):
    lib = cabi.load()
    g = torch.zeros(4, 2, 8, device="cuda")
    p = torch.zeros(8, device="cuda")
    ws = torch.zeros(1 << 16, dtype=torch.uint8, device="cuda")
    f32 = cabi.DTYPE_F32
    call = lambda dtype, T, B, C, HW, w, n: lib.snnlif_channel_sum(g.data_ptr(), p.data_ptr(), dtype, T, B, C, HW,
                                                                    w, n, None)
    assert call(cabi.DTYPE_BF16, 4, 2, 8, 1, ws.data_ptr(), ws.numel()) == cabi.ERR_UNSUPPORTED
    assert call(9, 4, 2, 8, 1, ws.data_ptr(), ws.numel()) == cabi.ERR_DTYPE
    assert call(f32, 0, 2, 8, 1, ws.data_ptr(), ws.numel()) == cabi.ERR_ARG
    assert call(f32, 4, 2, 0, 1, ws.data_ptr(), ws.numel()) == cabi.OK
    assert call(f32, 4, 2, 8, 1, None, 0) == cabi.ERR_WORKSPACE
    assert call(f32, 4, 2, 8, 1, ws.data_ptr(), 8) == cabi.ERR_WORKSPACE
    assert call(f32, 4, 2, 8, 1, ws.data_ptr() + 4, ws.numel() - 4) == cabi.ERR_ALIGN
    assert lib.snnlif_channel_sum(None, p.data_ptr(), f32, 4, 2, 8, 1, ws.data_ptr(), ws.numel(),
                                  None) == cabi.ERR_ARG
    torch.cuda.synchronize()


def test_convolution_bias_gradient_takes_the_channel_sum():
    """``snnlib.conv_bp`` / ``fire_conv_bp``: the bias gradient for the layers' dim_conv = (0, 1, 3, 4)
    (snnlib/example/snnlib_func.py:215, 247) comes from the hand-written reduction -- reproducible and the
    float64 sum rounded once, which a float32 reduction tree is not held to -- and any other dim_conv
    still gives what ``torch.sum`` gives."""
    import snn_gpu_training_bptt_amd.snnlib_func  # noqa: F401
    import snnlib
    gen = torch.Generator().manual_seed(58)
    x = torch.randn((4, 3, 5, 12, 12), generator=gen).cuda()
    w = (0.2 * torch.randn((6, 5, 3, 3), generator=gen)).cuda()
    g = torch.randn((4, 3, 6, 12, 12), generator=gen).cuda()
    conv_args = (w, (1, 1), (1, 1), (1, 1), 1, False, False, True)
    want = g.double().sum(dim=(0, 1, 3, 4))
    mass = g.double().abs().sum(dim=(0, 1, 3, 4))
    for dims in ((0, 1, 3, 4), (4, 3, 1, 0), (-5, 1, -2, -1)):
        for grads in (snnlib.conv_bp(x, g, *conv_args, dims),
                      snnlib.fire_conv_bp(x, g, *conv_args, dims, 0.25, 0.5, 1.0, 0.5)):
            gb = grads[2]
            assert gb.shape == (6,) and gb.dtype == torch.float32
            err = (gb.double().cpu() - want.cpu()).abs()
            assert bool((err <= 6.1e-8 * want.abs().cpu() + 1e-12 * mass.cpu()).all())
    strided = g.transpose(3, 4)                                     # made dense inside the op
    xs = x.transpose(3, 4).contiguous()
    gb = snnlib.conv_bp(xs, strided, *conv_args, (0, 1, 3, 4))[2]
    torch.testing.assert_close(gb.double().cpu(), want.cpu(), rtol=1e-6, atol=1e-6)
    partial = snnlib.conv_bp(x, g, *conv_args, (0, 3, 4))[2]        # not the layers' reduction: ATen's
    assert partial.shape == (3, 6)
    torch.testing.assert_close(partial, g.sum(dim=(0, 3, 4)))
    small = snnlib.conv_bp(x[..., :4, :4].contiguous(), g[..., :4, :4].contiguous(), *conv_args, (0, 1, 3, 4))[2]
    torch.testing.assert_close(small, g[..., :4, :4].sum(dim=(0, 1, 3, 4)))   # planes of 16 positions: ATen's


RUNNING_SHAPES = [(6, 2, 8), (6, 2, 8, 8, 8), (8, 16, 32, 16, 16), (4, 5, 7, 7, 7), (5, 2, 9, 31), (13, 3, 20, 5, 3),
                  (8, 64, 1024), (6, 64, 8, 8, 8)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("shape", RUNNING_SHAPES)
def test_running_statistics_carry_the_bits_of_the_layer_expressions(cabi, shape, dtype):
    """``snnlif_bn_stats_running`` = ``snnlif_bn_stats`` + what the reference's layers do next in Python
    (snnlib/example/snnlib_op.py:79-80): ``running * 0.9 + statistic * gain`` as the framework's
    element-wise ops evaluate it on the same device -- the same bits, also when written in place."""
    x = make(shape, seed=60, dtype=dtype).cuda()
    T, B, C, HW = dims_of(shape)
    gen = torch.Generator().manual_seed(61)
    running_var = (0.5 + torch.rand(C, generator=gen)).to(dtype).cuda()
    running_mean = torch.randn(C, generator=gen).to(dtype).cuda()
    n = T * B * HW
    factor = n / (n - 1) if n > 1 else 1.0
    mean_ref, var_ref = (t.cuda() for t in run_stats(cabi, x))
    want_var = running_var * 0.9 + var_ref * (0.1 * factor)
    want_mean = running_mean * 0.9 + mean_ref * 0.1
    code = cabi.DTYPE_F32 if dtype == torch.float32 else cabi.DTYPE_F64
    ws = torch.empty(cabi.bn_stats_workspace_bytes(code, T, B, C, HW), dtype=torch.uint8, device="cuda")
    mean, var, new_mean, new_var = (torch.full((C,), float("nan"), dtype=dtype, device="cuda") for _ in range(4))
    cabi.bn_stats_running_into(x, mean, var, running_mean, running_var, new_mean, new_var, ws,
                               0.9, 0.1, 0.1 * factor)
    torch.cuda.synchronize()
    assert torch.equal(mean, mean_ref) and torch.equal(var, var_ref)
    assert torch.equal(new_var, want_var) and torch.equal(new_mean, want_mean)
    assert torch.equal(running_var, (0.5 + torch.rand(C, generator=torch.Generator().manual_seed(61))).to(dtype).cuda())
    # in place
    rm, rv = running_mean.clone(), running_var.clone()
    cabi.bn_stats_running_into(x, mean, var, rm, rv, rm, rv, ws, 0.9, 0.1, 0.1 * factor)
    torch.cuda.synchronize()
    assert torch.equal(rv, want_var) and torch.equal(rm, want_mean)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("world", [1, 2, 3, 6, 7, 8])
def test_moments_finish_carries_the_bits_of_the_sharded_layers_expressions(cabi, world, dtype):
    """``snnlif_bn_moments_finish`` against snnlib/example/snnlib_op.py:271-275 evaluated by the framework on
    the same device: ``mean = first / world``, ``var = second / world - mean ** 2`` and the running pair with
    momentum 0.05; world sizes that are not powers of two show whether the division is the framework's."""
    C = 1000
    gen = torch.Generator().manual_seed(62 + world)
    first = (world * (0.3 + torch.randn(C, generator=gen))).to(dtype).cuda()
    second = (world * (1.5 + torch.rand(C, generator=gen) * 3)).to(dtype).cuda()
    running_var = (0.5 + torch.rand(C, generator=gen)).to(dtype).cuda()
    running_mean = torch.randn(C, generator=gen).to(dtype).cuda()
    factor = 98304 / 98303
    want_mean = first / world
    want_var = second / world - want_mean ** 2
    want_rv = running_var * 0.95 + want_var * (0.05 * factor)
    want_rm = running_mean * 0.95 + want_mean * 0.05
    mean, var, new_mean, new_var = (torch.full((C,), float("nan"), dtype=dtype, device="cuda") for _ in range(4))
    cabi.bn_moments_finish_into(first, second, mean, var, world,
                                running=(running_mean, running_var, new_mean, new_var, 0.95, 0.05, 0.05 * factor))
    torch.cuda.synchronize()
    assert torch.equal(mean, want_mean) and torch.equal(var, want_var)
    assert torch.equal(new_var, want_rv) and torch.equal(new_mean, want_rm)
    # without a running pair
    mean2, var2 = torch.empty_like(mean), torch.empty_like(var)
    cabi.bn_moments_finish_into(first, second, mean2, var2, world)
    torch.cuda.synchronize()
    assert torch.equal(mean2, want_mean) and torch.equal(var2, want_var)


def test_running_and_moments_argument_errors(cabi):
    lib = cabi.load()
    x = torch.zeros(4, 2, 8, device="cuda")
    p = [torch.zeros(8, device="cuda") for _ in range(6)]
    ws = torch.zeros(1 << 16, dtype=torch.uint8, device="cuda")
    f32 = cabi.DTYPE_F32
    ptr = [t.data_ptr() for t in p]
    run = lambda dtype, T, w, n, rm=ptr[2]: lib.snnlif_bn_stats_running(
        x.data_ptr(), ptr[0], ptr[1], rm, ptr[3], ptr[4], ptr[5], 0.9, 0.1, 0.1, dtype, T, 2, 8, 1, w, n, None)
    assert run(f32, 4, ws.data_ptr(), ws.numel()) == cabi.OK
    assert run(cabi.DTYPE_BF16, 4, ws.data_ptr(), ws.numel()) == cabi.ERR_UNSUPPORTED
    assert run(f32, 0, ws.data_ptr(), ws.numel()) == cabi.ERR_ARG
    assert run(f32, 4, None, 0) == cabi.ERR_WORKSPACE
    assert run(f32, 4, ws.data_ptr(), ws.numel(), rm=None) == cabi.ERR_ARG
    fin = lambda world, rm, rv, nm, nv, C=8, dtype=f32: lib.snnlif_bn_moments_finish(
        ptr[0], ptr[1], ptr[2], ptr[3], rm, rv, nm, nv, world, 0.95, 0.05, 0.05, dtype, C, None)
    assert fin(2.0, None, None, None, None) == cabi.OK
    assert fin(2.0, ptr[4], ptr[5], ptr[4], ptr[5]) == cabi.OK
    assert fin(2.0, ptr[4], None, ptr[4], ptr[5]) == cabi.ERR_ARG        # the running pair goes together
    assert fin(0.0, None, None, None, None) == cabi.ERR_ARG
    assert fin(2.0, None, None, None, None, C=-1) == cabi.ERR_ARG
    assert fin(2.0, None, None, None, None, C=0) == cabi.OK
    assert fin(2.0, None, None, None, None, dtype=cabi.DTYPE_BF16) == cabi.ERR_UNSUPPORTED
    torch.cuda.synchronize()


def test_argument_errors(cabi):
    lib = cabi.load()
    x = torch.zeros(4, 2, 8, device="cuda")
    p = torch.zeros(8, device="cuda")
    ws = torch.zeros(1 << 16, dtype=torch.uint8, device="cuda")
    f32 = cabi.DTYPE_F32
    call = lambda dtype, T, B, C, HW, w, n: lib.snnlif_bn_stats(x.data_ptr(), p.data_ptr(), p.data_ptr(), dtype,
                                                                 T, B, C, HW, 0, w, n, None)
    assert call(cabi.DTYPE_BF16, 4, 2, 8, 1, ws.data_ptr(), ws.numel()) == cabi.ERR_UNSUPPORTED
    assert call(9, 4, 2, 8, 1, ws.data_ptr(), ws.numel()) == cabi.ERR_DTYPE
    assert call(f32, 0, 2, 8, 1, ws.data_ptr(), ws.numel()) == cabi.ERR_ARG       # no elements per channel
    assert call(f32, 4, 2, 0, 1, ws.data_ptr(), ws.numel()) == cabi.OK            # no channels: nothing to do
    assert call(f32, 4, 2, 8, 1, None, 0) == cabi.ERR_WORKSPACE
    assert call(f32, 4, 2, 8, 1, ws.data_ptr(), 8) == cabi.ERR_WORKSPACE
    assert call(f32, 4, 2, 8, 1, ws.data_ptr() + 4, ws.numel() - 4) == cabi.ERR_ALIGN
    assert lib.snnlif_bn_stats(None, p.data_ptr(), p.data_ptr(), f32, 4, 2, 8, 1, 0, ws.data_ptr(), ws.numel(),
                               None) == cabi.ERR_ARG
    torch.cuda.synchronize()


def test_module_ops_and_layer_statistics():
    """``snnlib.bn_stats`` / ``snnlib.bn_moments`` and the running statistics of a layer that uses them."""
    import snn_gpu_training_bptt_amd.snnlib_func  # noqa: F401  (registers the module)
    import snnlib
    from snn_gpu_training_bptt_amd import snnlib_op as sop
    x = make((6, 4, 8, 8, 8), seed=55).cuda()
    mean_ref, var_ref, second_ref = reference(x.cpu())
    var, mean = snnlib.bn_stats(x)                       # the order of torch.var_mean
    first, second = snnlib.bn_moments(x)
    torch.testing.assert_close(mean.cpu().double(), mean_ref, rtol=1e-6, atol=1e-7)
    torch.testing.assert_close(var.cpu().double(), var_ref, rtol=1e-6, atol=0)
    torch.testing.assert_close(second.cpu().double(), second_ref, rtol=1e-6, atol=0)
    assert torch.equal(first, mean)
    strided = x.transpose(3, 4)                          # made dense inside the op
    v2, m2 = snnlib.bn_stats(strided)
    torch.testing.assert_close(m2, mean, rtol=1e-6, atol=1e-7)
    with pytest.raises(RuntimeError, match="float32 and float64"):
        snnlib.bn_stats(x.bfloat16())
    with pytest.raises(RuntimeError, match="ROCm GPU"):
        snnlib.bn_stats(x.cpu())
    with pytest.raises(RuntimeError, match="no elements per channel"):
        snnlib.bn_stats(torch.zeros(0, 2, 3, device="cuda"))
    rv, rm = torch.rand(8, device="cuda") + 0.5, torch.randn(8, device="cuda")
    n = x.numel() / 8
    v3, m3, rv3, rm3 = snnlib.bn_stats_running(x, rv, rm, 0.9, 0.1 * n / (n - 1), 0.1)
    assert torch.equal(v3, var) and torch.equal(m3, mean)
    assert torch.equal(rv3, rv * 0.9 + var * (0.1 * n / (n - 1))) and torch.equal(rm3, rm * 0.9 + mean * 0.1)
    v4, m4, rv4, rm4 = snnlib.bn_moments_finish(first * 3, second * 3, 3, rv, rm, 0.95, 0.05 * n / (n - 1), 0.05)
    want_m = (first * 3) / 3
    want_v = (second * 3) / 3 - want_m ** 2
    assert torch.equal(m4, want_m) and torch.equal(v4, want_v)
    assert torch.equal(rv4, rv * 0.95 + want_v * (0.05 * n / (n - 1))) and torch.equal(rm4, rm * 0.95 + want_m * 0.05)
    layer = sop.Bn(8, (0, 1, 3, 4)).cuda()
    layer(x.requires_grad_(True))
    assert isinstance(layer.running_var, torch.nn.Parameter) and layer.running_var.is_leaf
    n = x.numel() / 8
    torch.testing.assert_close(layer.running_mean.detach().cpu().double(), 0.1 * mean_ref, rtol=1e-5, atol=1e-7)
    torch.testing.assert_close(layer.running_var.detach().cpu().double(), 0.9 + 0.1 * var_ref * n / (n - 1),
                               rtol=1e-5, atol=0)
    with pytest.raises(ValueError, match="dim_bn"):
        sop.Bn(8, (0, 1)).cuda()(x)
