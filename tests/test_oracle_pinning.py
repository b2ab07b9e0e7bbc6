"""Pins the CPU oracle (``oracle/lif_oracle.c`` through ``oracle/c_oracle.py``, and the pure-PyTorch
restatement ``oracle/gold_fire.py``) without the reference's help: the reference's own tests hold no
stored vectors for this path (snnlib/example/test_fire.py + test_utils.py draw unseeded inputs on a
GPU and print differences), so every check here is something the mathematics fixes.

Each check is chosen so that a plausible transcription mistake fails it:
  dropped reset term / wrong sign of the reset gradient  -> T=2 and always-spiking closed forms
  decay applied to the wrong operand or missing          -> dyadic geometric sums, alpha=0 case
  '>' vs '>=' or '<' vs '<=' at the threshold / window   -> boundary inputs placed exactly on them
  transposed / mis-strided indexing over [T, B, CHW]     -> permutation and reshape invariance
  time loop running the wrong way or off by one          -> prefix property, T=1 reduction
  any arithmetic-order slip                              -> bit equality with the fp32 tape
"""
import json
import os
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import c_oracle, gold_fire

HERE = os.path.dirname(os.path.abspath(__file__))


def fwd(x, alpha, thresh):
    return c_oracle.fire_forward(np.asarray(x, dtype=np.float32), alpha, thresh)


def bwd(x, g, alpha, thresh, beta, interval):
    return c_oracle.fire_backward(np.asarray(x, dtype=np.float32), np.asarray(g, dtype=np.float32),
                                  alpha, thresh, beta, interval)


def col(values):
    """[T] list -> array shaped [T, 1, 1] (one neuron)."""
    return np.asarray(values, dtype=np.float32).reshape(-1, 1, 1)


# ---- closed forms ---------------------------------------------------------------------------

def test_single_step_reduces_to_heaviside_and_window():
    rng = np.random.default_rng(0)
    x = rng.normal(0.5, 1.0, size=(1, 3, 50)).astype(np.float32)
    g = rng.normal(size=x.shape).astype(np.float32)
    mem, spike = fwd(x, 0.25, 0.5)
    assert np.array_equal(mem, x + np.float32(0))
    assert np.array_equal(spike, (x > np.float32(0.5)).astype(np.float32))
    gx = bwd(x, g, 0.25, 0.5, 0.75, 0.5)
    window = (np.abs(x - np.float32(0.5)) < np.float32(0.5)).astype(np.float32)
    assert np.array_equal(gx, g * window * np.float32(0.75))


def test_zero_decay_makes_steps_independent():
    rng = np.random.default_rng(1)
    x = rng.normal(0.5, 1.0, size=(5, 2, 40)).astype(np.float32)
    g = rng.normal(size=x.shape).astype(np.float32)
    mem, spike = fwd(x, 0.0, 0.5)
    assert np.array_equal(mem, x + np.float32(0))
    assert np.array_equal(spike, (x > np.float32(0.5)).astype(np.float32))
    gx = bwd(x, g, 0.0, 0.5, 1.0, 0.5)
    window = (np.abs(x - np.float32(0.5)) < np.float32(0.5)).astype(np.float32)
    assert np.array_equal(gx, g * window)


def test_subthreshold_dyadic_input_gives_exact_geometric_sums():
    """No spikes (threshold far above): u[t] = sum_k alpha^(t-k) x[k], exact in fp32 for dyadic data."""
    alpha = Fraction(1, 4)
    xs = [Fraction(1, 2), Fraction(1, 8), Fraction(3, 4), Fraction(1, 16), Fraction(1, 2), Fraction(1, 4)]
    mem, spike = fwd(col([float(v) for v in xs]), float(alpha), 100.0)
    expect, u = [], Fraction(0)
    for v in xs:
        u = alpha * u + v
        expect.append(float(u))
    assert mem.reshape(-1).tolist() == expect
    assert not spike.any()


def test_subthreshold_in_window_gradient_closed_form():
    """No spikes, every step inside the window:
    gx[t] = beta*(g[t] - gx[t+1]*alpha*u[t]) + gx[t+1]*alpha, evaluated exactly with fractions."""
    alpha, beta, thresh, interval = Fraction(1, 4), Fraction(1, 2), Fraction(1), Fraction(2)
    xs = [Fraction(1, 4), Fraction(1, 8), Fraction(1, 2), Fraction(1, 4)]
    gs = [Fraction(1), Fraction(-1, 2), Fraction(2), Fraction(1, 4)]
    u, us = Fraction(0), []
    for v in xs:
        u = alpha * u + v
        us.append(u)
    assert all(v <= thresh and abs(v - thresh) < interval for v in us)
    expect, carry = [None] * 4, Fraction(0)
    for t in range(3, -1, -1):
        carry = beta * (gs[t] - carry * alpha * us[t]) + carry * alpha
        expect[t] = carry
    gx = bwd(col([float(v) for v in xs]), col([float(v) for v in gs]),
             float(alpha), float(thresh), float(beta), float(interval))
    # dyadic inputs, four steps: every intermediate fits fp32 exactly
    assert gx.reshape(-1).tolist() == [float(v) for v in expect]


def test_always_spiking_neuron_resets_every_step():
    """Every step fires: the carried potential is multiplied by (1 - 1) = 0, so u[t] = x[t]; the
    decay path is closed ((u <= thresh) = 0) and only the reset path -gx[t+1]*alpha*u[t] remains."""
    alpha, beta, thresh, interval = Fraction(1, 4), Fraction(1), Fraction(1, 2), Fraction(1, 2)
    xs = [Fraction(3, 4), Fraction(5, 8), Fraction(7, 8), Fraction(3, 4), Fraction(9, 16)]   # all in (0.5, 1.0)
    gs = [Fraction(1), Fraction(1, 2), Fraction(-1), Fraction(2), Fraction(1)]
    mem, spike = fwd(col([float(v) for v in xs]), float(alpha), float(thresh))
    assert mem.reshape(-1).tolist() == [float(v) for v in xs]
    assert spike.all()
    expect, carry = [None] * 5, Fraction(0)
    for t in range(4, -1, -1):
        carry = beta * (gs[t] - carry * alpha * xs[t])
        expect[t] = carry
    gx = bwd(col([float(v) for v in xs]), col([float(v) for v in gs]),
             float(alpha), float(thresh), float(beta), float(interval))
    assert gx.reshape(-1).tolist() == [float(v) for v in expect]


@pytest.mark.parametrize("x0,x1", [
    (0.25, 0.25),    # no spike, no spike; both inside the window
    (0.75, 0.25),    # spike then none: the reset kills the carry
    (0.25, 0.75),    # none then spike
    (2.0, 0.25),     # step 0 spikes outside the window: its spike gradient is cut
    (-1.0, 0.75),    # step 0 silent outside the window: only the decay path reaches x0
])
def test_two_step_gradient_by_hand(x0, x1):
    """T = 2 chain rule written out: L = g0*s0 + g1*s1, ds/du = beta*W(u),
    u1 = x1 + alpha*u0*(1 - s0)."""
    alpha, beta, thresh, interval = 0.5, 0.5, 0.5, 1.0
    g0, g1 = 1.0, -2.0
    u0 = x0
    s0 = 1.0 if u0 > thresh else 0.0
    u1 = x1 + alpha * u0 * (1 - s0)
    W = lambda u: 1.0 if abs(u - thresh) < interval else 0.0
    d_u1 = g1 * beta * W(u1)
    d_s0 = g0 + d_u1 * (-alpha * u0)            # through the reset factor (1 - s0)
    d_u0 = d_s0 * beta * W(u0) + d_u1 * alpha * (1 - s0)
    mem, spike = fwd(col([x0, x1]), alpha, thresh)
    assert mem.reshape(-1).tolist() == [u0, u1]
    assert spike.reshape(-1).tolist() == [s0, 1.0 if u1 > thresh else 0.0]
    gx = bwd(col([x0, x1]), col([g0, g1]), alpha, thresh, beta, interval)
    assert gx.reshape(-1).tolist() == [d_u0, d_u1]


def test_comparisons_are_strict_at_the_boundaries():
    thresh, interval = 0.5, 0.5
    # u == thresh does not fire; u just above does
    _, spike = fwd(col([0.5]), 0.25, thresh)
    assert spike.item() == 0.0
    _, spike = fwd(col([np.nextafter(np.float32(0.5), np.float32(1))]), 0.25, thresh)
    assert spike.item() == 1.0
    # |u - thresh| == interval is outside the window on both sides; one ulp inside is inside
    for u_edge in (0.0, 1.0):
        assert bwd(col([u_edge]), col([1.0]), 0.25, thresh, 1.0, interval).item() == 0.0
    assert bwd(col([np.nextafter(np.float32(1.0), np.float32(0))]), col([1.0]), 0.25, thresh, 1.0, interval).item() == 1.0
    # (below 0.5 the spacing of fp32 halves, so 'just inside' from the low side is 2**-24, the
    # smallest value whose distance to 0.5 is representable)
    assert bwd(col([2.0 ** -24]), col([1.0]), 0.25, thresh, 1.0, interval).item() == 1.0
    # u == thresh counts as "not fired" for the decay path: (u <= thresh) = 1
    gx = bwd(col([0.5, 0.25]), col([0.0, 1.0]), 0.5, thresh, 1.0, interval)
    # step 1: u1 = 0.25 + 0.5*0.5 = 0.5 (in window) -> d_u1 = 1; step 0: u0 = 0.5, in window:
    # d_u0 = (0 - 1*0.5*0.5)*1 + 1*0.5*1 = 0.25
    assert gx.reshape(-1).tolist() == [0.25, 1.0]


# ---- invariants ------------------------------------------------------------------------------

def test_spikes_are_binary_and_neurons_independent():
    rng = np.random.default_rng(2)
    x = rng.normal(0.5, 1.0, size=(6, 4, 3, 5, 2)).astype(np.float32)
    g = rng.normal(size=x.shape).astype(np.float32)
    mem, spike = fwd(x, 0.3, 0.5)
    gx = bwd(x, g, 0.3, 0.5, 1.0, 0.5)
    assert set(np.unique(spike)) <= {0.0, 1.0}
    # any reshape of the neuron axes, and any permutation of neurons, gives the same bits
    flat = x.reshape(6, 1, -1)
    mem_f, spike_f = fwd(flat, 0.3, 0.5)
    assert np.array_equal(mem_f.reshape(x.shape), mem) and np.array_equal(spike_f.reshape(x.shape), spike)
    perm = rng.permutation(flat.shape[2])
    gx_p = bwd(flat[:, :, perm], g.reshape(6, 1, -1)[:, :, perm], 0.3, 0.5, 1.0, 0.5)
    assert np.array_equal(gx_p, gx.reshape(6, 1, -1)[:, :, perm])
    # batch-major vs position-major storage of the same neurons ([T,B,CHW] vs [T,CHW,B] transposed)
    xt = np.ascontiguousarray(x.reshape(6, 4, 30).transpose(0, 2, 1))
    _, spike_t = fwd(xt, 0.3, 0.5)
    assert np.array_equal(spike_t.transpose(0, 2, 1).reshape(x.shape), spike)


def test_prefix_property_and_causality():
    rng = np.random.default_rng(3)
    x = rng.normal(0.5, 1.0, size=(9, 2, 33)).astype(np.float32)
    mem, spike = fwd(x, 0.25, 0.5)
    for t_cut in (1, 4, 8):
        mem_c, spike_c = fwd(x[:t_cut], 0.25, 0.5)
        assert np.array_equal(mem_c, mem[:t_cut]) and np.array_equal(spike_c, spike[:t_cut])
    # the gradient at step t depends only on spike gradients at steps >= t
    g = rng.normal(size=x.shape).astype(np.float32)
    gx = bwd(x, g, 0.25, 0.5, 1.0, 0.5)
    g2 = g.copy()
    g2[:3] = 0
    gx2 = bwd(x, g2, 0.25, 0.5, 1.0, 0.5)
    assert np.array_equal(gx2[3:], gx[3:])


def test_backward_is_linear_in_the_spike_gradient():
    rng = np.random.default_rng(4)
    x = rng.normal(0.5, 1.0, size=(7, 2, 20)).astype(np.float32)
    g = rng.normal(size=x.shape).astype(np.float32)
    gx = bwd(x, g, 0.25, 0.5, 1.0, 0.5)
    assert not bwd(x, np.zeros_like(g), 0.25, 0.5, 1.0, 0.5).any()
    # scaling by a power of two commutes with every rounding
    assert np.array_equal(bwd(x, g * np.float32(4), 0.25, 0.5, 1.0, 0.5), gx * np.float32(4))
    assert np.array_equal(bwd(x, -g, 0.25, 0.5, 1.0, 0.5), -gx)


# ---- independent implementations ---------------------------------------------------------------

def _load_vectors():
    with open(os.path.join(HERE, "golden", "fire_vectors.json")) as f:
        data = json.load(f)

    def unpack(rows, shape):
        flat = [int(r[i:i + 8], 16) for r in rows for i in range(0, len(r), 8)]
        return np.array(flat, dtype=np.uint32).view(np.float32).reshape(shape)

    for case in data["cases"]:
        shape = case["shape"]
        yield case["name"], case["hyper"], {k: unpack(case[k], shape)
                                            for k in ("x", "grad_spike", "mem", "spike", "grad_x")}


@pytest.mark.parametrize("name,hyper,arrays", list(_load_vectors()), ids=lambda v: v if isinstance(v, str) else "")
def test_stored_vectors_from_the_fp32_tape(name, hyper, arrays):
    """Vectors written by tests/golden/make_fire_vectors.py with the pure-Python fp32 autodiff tape
    (a transcription of the gold path's graph, not of the kernels)."""
    mem, spike = fwd(arrays["x"], hyper["alpha"], hyper["thresh"])
    gx = bwd(arrays["x"], arrays["grad_spike"], **hyper)
    assert np.array_equal(spike, arrays["spike"])
    assert np.array_equal(mem, arrays["mem"])
    assert np.array_equal(gx, arrays["grad_x"])
    u_t, s_t, gx_t = gold_fire.gold_fire_fwd_bwd(torch.from_numpy(arrays["x"]), torch.from_numpy(arrays["grad_spike"]), **hyper)
    assert np.array_equal(s_t.numpy(), arrays["spike"])
    assert np.array_equal(u_t.numpy(), arrays["mem"])
    assert np.array_equal(gx_t.numpy(), arrays["grad_x"])


def test_fp32_tape_agrees_on_fresh_random_neurons():
    import sys
    sys.path.insert(0, os.path.join(HERE, "golden"))
    import fp32_tape

    rng = np.random.default_rng(5)
    hyper = dict(alpha=0.3, thresh=0.5, beta=0.9, interval=0.45)
    T, n = 9, 24
    x = rng.normal(0.5, 1.0, size=(T, 1, n)).astype(np.float32)
    g = rng.normal(size=x.shape).astype(np.float32)
    mem, spike = fwd(x, hyper["alpha"], hyper["thresh"])
    gx = bwd(x, g, **hyper)
    for i in range(n):
        u_i, s_i, gx_i = fp32_tape.gold_fire_neuron(x[:, 0, i].tolist(), g[:, 0, i].tolist(), **hyper)
        assert mem[:, 0, i].tolist() == u_i
        assert spike[:, 0, i].tolist() == s_i
        assert gx[:, 0, i].tolist() == gx_i


@pytest.mark.parametrize("shape,mean,std", [((4, 8, 16, 8, 8), 0.5, 1.0), ((32, 2, 16, 4, 4), 0.3, 0.8), ((6, 2, 8), 0.0, 1.0)])
@pytest.mark.parametrize("alpha,thresh,beta,interval", [(0.25, 0.5, 1.0, 0.5), (0.3, 0.25, 0.7, 0.8)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_scalar_loops_match_autograd_of_the_gold_graph(shape, mean, std, alpha, thresh, beta, interval, dtype):
    """The C loops follow the kernels' order; gold_fire.py follows the PyTorch graph and lets autograd
    derive the backward.  Two derivations, one result, bit for bit."""
    gen = torch.Generator().manual_seed(6)
    x = (mean + std * torch.randn(shape, generator=gen)).to(dtype)
    g = torch.randn(shape, generator=gen).to(dtype)
    if dtype == torch.float64:
        # the C ABI narrows hyper-parameters to fp32 (as the reference's binding does); give the
        # PyTorch side the same values
        alpha, thresh, beta, interval = (float(np.float32(v)) for v in (alpha, thresh, beta, interval))
    u, s, gx = gold_fire.gold_fire_fwd_bwd(x, g, alpha, thresh, beta, interval)
    mem_c, spike_c = c_oracle.fire_forward(x.numpy(), alpha, thresh)
    gx_c = c_oracle.fire_backward(x.numpy(), g.numpy(), alpha, thresh, beta, interval)
    assert np.array_equal(spike_c, s.numpy())
    assert np.array_equal(mem_c, u.numpy())
    assert np.array_equal(gx_c, gx.numpy())


# ---- batch-norm + fire ---------------------------------------------------------------------------

def _bn_case(shape, seed):
    gen = torch.Generator().manual_seed(seed)
    C = shape[2]
    x = 0.5 + torch.randn(shape, generator=gen)
    g = torch.randn(shape, generator=gen)
    w = 0.5 + torch.rand(C, generator=gen)
    b = 0.2 * torch.randn(C, generator=gen)
    dims = (0, 1) + tuple(range(3, len(shape)))
    var, mean = torch.var_mean(x, dim=dims, unbiased=False)
    return x, g, w, b, var, mean


def test_bn_fire_with_identity_statistics_is_plain_fire():
    """mean 0, var + eps == 1, weight 1, bias 0: the affine is exactly the identity, so spikes and
    potentials equal the plain fire op's and the input gradient is the plain one minus the two
    batch-norm projection terms computed from it."""
    eps = 1e-5
    x, g, _, _, _, _ = _bn_case((5, 3, 4, 6), 40)
    C = 4
    one, zero = np.ones(C, np.float32), np.zeros(C, np.float32)
    var = np.full(C, np.float32(1.0) - np.float32(eps), np.float32)
    assert np.float32(var[0] + np.float32(eps)) == np.float32(1.0)
    ivar, mem, spike = c_oracle.bn_fire_forward(x.numpy(), one, zero, var, zero, eps, 0.25, 0.5)
    mem_p, spike_p = c_oracle.fire_forward(x.numpy(), 0.25, 0.5)
    assert np.array_equal(ivar, one) and np.array_equal(mem, mem_p) and np.array_equal(spike, spike_p)
    gx, gw, gb = c_oracle.bn_fire_backward(x.numpy(), one, zero, one, zero, g.numpy(), 0.25, 0.5, 1.0, 0.5)
    gy = c_oracle.fire_backward(x.numpy(), g.numpy(), 0.25, 0.5, 1.0, 0.5).astype(np.float64)
    xs = x.numpy().astype(np.float64)
    axes = (0, 1, 3)
    np.testing.assert_allclose(gb, gy.sum(axis=axes), rtol=1e-5)
    np.testing.assert_allclose(gw, (gy * xs).sum(axis=axes), rtol=1e-5, atol=1e-5)
    expect = gy - gy.mean(axis=axes, keepdims=True) - xs * (gy * xs).mean(axis=axes, keepdims=True)
    np.testing.assert_allclose(gx, expect, rtol=1e-5, atol=1e-5)


def test_bn_fire_single_step_is_textbook_batch_norm_backward():
    """T = 1: no recurrence; spikes = (bn(x) > thresh) and the backward is batch-norm's with the
    upstream gradient g * window(bn(x)) * beta (closed form evaluated in float64)."""
    eps, thresh, beta, interval = 1e-5, 0.5, 0.8, 0.6
    x, g, w, b, var, mean = _bn_case((1, 6, 3, 5), 41)
    ivar, mem, spike = c_oracle.bn_fire_forward(x.numpy(), w.numpy(), b.numpy(), var.numpy(), mean.numpy(), eps, 0.25, thresh)
    xs, gs = x.numpy().astype(np.float64), g.numpy().astype(np.float64)
    sh = (1, 1, 3, 1)
    m64, v64 = mean.numpy().astype(np.float64).reshape(sh), var.numpy().astype(np.float64).reshape(sh)
    w64, b64 = w.numpy().astype(np.float64).reshape(sh), b.numpy().astype(np.float64).reshape(sh)
    iv64 = 1.0 / np.sqrt(v64 + eps)
    xhat = (xs - m64) * iv64
    y = xhat * w64 + b64
    np.testing.assert_allclose(mem, y, rtol=1e-5, atol=1e-6)
    safe = np.abs(y - thresh) > 1e-4            # away from the threshold the spike is unambiguous
    assert np.array_equal(spike[safe], (y > thresh)[safe].astype(np.float32))
    gy = gs * (np.abs(y - thresh) < interval) * beta
    axes = (0, 1, 3)
    gx, gw, gb = c_oracle.bn_fire_backward(x.numpy(), w.numpy(), b.numpy(), ivar, mean.numpy(), g.numpy(),
                                           0.25, thresh, beta, interval)
    np.testing.assert_allclose(gb, gy.sum(axis=axes), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(gw, (gy * xhat).sum(axis=axes), rtol=1e-5, atol=1e-6)
    gxhat = gy * w64
    expect = iv64 * (gxhat - gxhat.mean(axis=axes, keepdims=True) - xhat * (gxhat * xhat).mean(axis=axes, keepdims=True))
    np.testing.assert_allclose(gx, expect, rtol=1e-4, atol=1e-6)


@pytest.mark.parametrize("shape", [(6, 4, 8, 8, 8), (6, 16, 8), (3, 2, 5, 7)])
def test_bn_fire_loops_match_autograd_through_batch_norm(shape):
    """The C loops (the reference kernels' formulae) against autograd of
    torch.nn.functional.batch_norm + the gold fire loop: two derivations of the same backward."""
    eps = 1e-5
    x, g, w, b, var, mean = _bn_case(shape, 42)
    ivar, mem, spike = c_oracle.bn_fire_forward(x.numpy(), w.numpy(), b.numpy(), var.numpy(), mean.numpy(), eps, 0.25, 0.5)
    gx, gw, gb = c_oracle.bn_fire_backward(x.numpy(), w.numpy(), b.numpy(), ivar, mean.numpy(), g.numpy(), 0.25, 0.5, 1.0, 0.5)
    xr, wr, br = x.clone().requires_grad_(True), w.clone().requires_grad_(True), b.clone().requires_grad_(True)
    u, s = gold_fire.gold_bn_fire(xr, wr, br, None, None, True, eps, 0.25, 0.5, 1.0, 0.5)
    s.backward(g)
    assert np.array_equal(spike, s.detach().numpy())
    np.testing.assert_allclose(mem, u.detach().numpy(), rtol=1e-5, atol=1e-6)
    scale = lambda a: np.abs(a).max()
    assert np.abs(gx - xr.grad.numpy()).max() <= 1e-5 * scale(gx)
    assert np.abs(gw - wr.grad.numpy()).max() <= 1e-5 * scale(gw)
    assert np.abs(gb - br.grad.numpy()).max() <= 1e-5 * scale(gb)


@pytest.mark.parametrize("shape", [(6, 4, 8, 8, 8), (6, 16, 8), (3, 2, 5, 7), (1, 6, 3, 5)])
def test_bn_fire_double_precision_loops(shape):
    """The fp64 instantiation of the same loops: against autograd in double through batch_norm + the
    gold fire loop (errors at double rounding level), against the textbook closed form when T = 1, and
    against the fp32 loops on the same inputs."""
    eps = 1e-5
    x, g, w, b, var, mean = (t.double() for t in _bn_case(shape, 43))
    dims = (0, 1) + tuple(range(3, len(shape)))
    var, mean = torch.var_mean(x, dim=dims, unbiased=False)
    n = lambda t: t.numpy()
    ivar, mem, spike = c_oracle.bn_fire_forward(n(x), n(w), n(b), n(var), n(mean), eps, 0.25, 0.5)
    gx, gw, gb = c_oracle.bn_fire_backward(n(x), n(w), n(b), ivar, n(mean), n(g), 0.25, 0.5, 0.8, 0.6)
    assert ivar.dtype == mem.dtype == gx.dtype == gw.dtype == np.float64

    xr, wr, br = x.clone().requires_grad_(True), w.clone().requires_grad_(True), b.clone().requires_grad_(True)
    # hyper-parameters reach the loops as C floats (as in the reference's kernels): give the double
    # graph the same values
    f = lambda v: float(np.float32(v))
    u, s = gold_fire.gold_bn_fire(xr, wr, br, None, None, True, f(eps), 0.25, 0.5, f(0.8), f(0.6))
    s.backward(g)
    assert np.array_equal(spike, n(s.detach()))
    np.testing.assert_allclose(mem, n(u.detach()), rtol=1e-12, atol=1e-13)
    for got, want in ((gx, xr.grad), (gw, wr.grad), (gb, br.grad)):
        assert np.abs(got - n(want)).max() <= 1e-11 * (np.abs(got).max() + 1e-300)

    if shape[0] == 1:
        sh = (1, 1, shape[2]) + (1,) * (len(shape) - 3)
        iv = 1.0 / np.sqrt(n(var).reshape(sh) + np.float64(np.float32(eps)))
        xhat = (n(x) - n(mean).reshape(sh)) * iv
        y = xhat * n(w).reshape(sh) + n(b).reshape(sh)
        gy = n(g) * (np.abs(y - 0.5) < np.float64(np.float32(0.6))) * np.float64(np.float32(0.8))
        gxhat = gy * n(w).reshape(sh)
        expect = iv * (gxhat - gxhat.mean(axis=dims, keepdims=True) - xhat * (gxhat * xhat).mean(axis=dims, keepdims=True))
        np.testing.assert_allclose(gx, expect, rtol=1e-9, atol=1e-12)

    # the fp32 loops on the same (fp32-representable) inputs
    x32 = x.float()
    var32, mean32 = torch.var_mean(x32, dim=dims, unbiased=False)
    iv32, mem32, spike32 = c_oracle.bn_fire_forward(n(x32), n(w.float()), n(b.float()), n(var32), n(mean32), eps, 0.25, 0.5)
    assert iv32.dtype == np.float32
    np.testing.assert_allclose(iv32, c_oracle.bn_fire_forward(n(x32.double()), n(w.float().double()), n(b.float().double()),
                                                               n(var32.double()), n(mean32.double()), eps, 0.25, 0.5)[0], rtol=1e-6)


# ---- plain batch norm (no fire): lif_oracle_plain_bn_* ----------------------------------------------

@pytest.mark.parametrize("shape", [(6, 4, 8, 8, 8), (6, 16, 8), (3, 2, 5, 7), (1, 6, 3, 5)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_plain_bn_loops_match_the_library_batch_norm_and_its_autograd(shape, dtype):
    """Forward: torch.nn.functional.batch_norm with given statistics (the textbook affine).  Backward:
    autograd through the training-mode batch norm evaluated in float64, i.e. the statistics as
    functions of x -- a derivation independent of the reference kernels' formulae."""
    eps = 1e-5
    x, g, w, b, var, mean = (t.to(dtype) for t in _bn_case(shape, 50))
    dims = (0, 1) + tuple(range(3, len(shape)))
    var, mean = torch.var_mean(x, dim=dims, unbiased=False)
    n = lambda t: t.numpy()
    ivar, y = c_oracle.bn_forward(n(x), n(w), n(b), n(var), n(mean), eps)
    assert ivar.dtype == y.dtype == n(x).dtype
    fold = lambda t: t.reshape((shape[0] * shape[1],) + tuple(shape[2:]))
    y_lib = torch.nn.functional.batch_norm(fold(x.double()), mean.double(), var.double(), w.double(), b.double(),
                                           False, 0.0, float(np.float32(eps)) if dtype == torch.float64 else eps)
    tol = 1e-5 if dtype == torch.float32 else 1e-12
    np.testing.assert_allclose(y.reshape(y_lib.shape), n(y_lib), rtol=tol, atol=tol)
    np.testing.assert_allclose(ivar, 1.0 / np.sqrt(n(var).astype(np.float64) + np.float64(np.float32(eps))), rtol=tol)

    gx, gw, gb = c_oracle.bn_backward(n(x), n(w), ivar, n(mean), n(g))
    xr = x.double().clone().requires_grad_(True)
    wr, br = w.double().clone().requires_grad_(True), b.double().clone().requires_grad_(True)
    out = torch.nn.functional.batch_norm(fold(xr), None, None, wr, br, True, 0.0, float(np.float32(eps)))
    out.backward(fold(g.double()))
    scale = lambda a: np.abs(a).max() + 1e-300
    btol = 2e-5 if dtype == torch.float32 else 1e-11
    assert np.abs(gx - n(xr.grad)).max() <= btol * scale(gx)
    assert np.abs(gw - n(wr.grad)).max() <= btol * scale(gw)
    assert np.abs(gb - n(br.grad)).max() <= btol * scale(gb)


def test_plain_bn_loops_on_a_hand_computed_case():
    """Two channels, dyadic values, everything exact: channel 0 holds x = (1, 3) with g = (1, 0),
    channel 1 holds x = (0, 4) with g = (2, 2); statistics given, not derived.
    Channel 0: mean 2, ivar 1, weight 2 -> xhat = (-1, 1); grad_bias 1, grad_weight -1,
    gxhat = 2*1/2 = 1, gxhatx = 2*(-1)/2 = -1, gx = g*2 - (xhat*(-1) + 1) = (2 - 2, 0 - 0) = (0, 0).
    Channel 1: mean 2, ivar 0.5, weight 1 -> xhat = (-1, 1); grad_bias 4, grad_weight 0,
    gxhat = 2, gxhatx = 0, gx = g*0.5 - 0.5*(0 + 2) = (0, 0)."""
    x = np.array([[[1.0, 0.0]], [[3.0, 4.0]]], np.float32)        # [T=2, B=1, C=2]
    g = np.array([[[1.0, 2.0]], [[0.0, 2.0]]], np.float32)
    w = np.array([2.0, 1.0], np.float32)
    mean = np.array([2.0, 2.0], np.float32)
    ivar = np.array([1.0, 0.5], np.float32)
    gx, gw, gb = c_oracle.bn_backward(x, w, ivar, mean, g)
    assert np.array_equal(gb, np.array([1.0, 4.0], np.float32))
    assert np.array_equal(gw, np.array([-1.0, 0.0], np.float32))
    assert np.array_equal(gx, np.zeros_like(x))
    # a gradient that is not orthogonal to the projections: g' = g + (1, 0) on channel 1's first element
    g2 = g.copy()
    g2[0, 0, 1] = 3.0      # channel 1: g = (3, 2): grad_bias 5, grad_weight -3+2 = -1, gxhat 2.5, gxhatx -0.5
    gx2, gw2, gb2 = c_oracle.bn_backward(x, w, ivar, mean, g2)
    assert gb2[1] == 5.0 and gw2[1] == -1.0
    # gx = g*0.5 - 0.5*(xhat*(-0.5) + 2.5) -> (1.5 - 0.5*3.0, 1.0 - 0.5*2.0) = (0.0, 0.0)
    assert np.array_equal(gx2[:, 0, 1], np.array([0.0, 0.0], np.float32))
    # forward with var chosen so that var + eps is exactly 4 (scale = weight / 2)
    eps = np.float32(1e-5)
    var = np.full(2, np.float32(4.0) - eps, np.float32)
    assert np.float32(var[0] + eps) == np.float32(4.0)
    iv, y = c_oracle.bn_forward(x, w, np.array([0.5, -1.0], np.float32), var, mean, float(eps))
    assert np.array_equal(iv, np.array([0.5, 0.5], np.float32))
    assert np.array_equal(y, np.array([[[-0.5, -2.0]], [[1.5, 0.0]]], np.float32))
