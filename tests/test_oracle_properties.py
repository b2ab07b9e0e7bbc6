"""Property tests of the CPU oracle over generated shapes and hyper-parameters (hypothesis): the
invariants the mathematics of the fire recurrence fixes, checked where test_oracle_pinning.py checks
them on hand-picked cases.  A dropped term, a wrong comparison or a transposed index in the scalar
loops breaks at least one of them.
"""
import numpy as np
import torch
from hypothesis import given, settings, strategies as st

from oracle import c_oracle, gold_fire

SETTINGS = dict(max_examples=60, deadline=None)
hyper = st.tuples(st.sampled_from([0.0, 0.25, 0.3, 0.5, 0.9, 1.0]),      # alpha
                  st.sampled_from([0.25, 0.5, 1.0]),                      # thresh
                  st.sampled_from([0.5, 1.0, 2.0]),                       # beta
                  st.sampled_from([0.25, 0.5, 1.5]))                      # interval
dims = st.tuples(st.integers(1, 40), st.integers(1, 3), st.integers(1, 50))
seeds = st.integers(0, 2**31 - 1)


def draw(shape, seed, dtype=np.float32):
    rng = np.random.default_rng(seed)
    return (rng.normal(0.4, 0.9, size=shape).astype(dtype), rng.normal(0.0, 1.0, size=shape).astype(dtype))


@settings(**SETTINGS)
@given(dims, hyper, seeds)
def test_scalar_loops_equal_autograd_of_the_gold_graph(shape, h, seed):
    alpha, thresh, beta, interval = h
    x, g = draw(shape, seed)
    mem, spike = c_oracle.fire_forward(x, alpha, thresh)
    gx = c_oracle.fire_backward(x, g, alpha, thresh, beta, interval)
    xt = torch.from_numpy(x).requires_grad_(True)
    u, s = gold_fire.gold_fire(xt, alpha, thresh, beta, interval)
    s.backward(torch.from_numpy(g))
    assert np.array_equal(mem, u.detach().numpy())
    assert np.array_equal(spike, s.detach().numpy())
    assert np.array_equal(gx, xt.grad.numpy())


@settings(**SETTINGS)
@given(dims, hyper, seeds, st.integers(1, 40))
def test_prefix_and_causality(shape, h, seed, cut):
    alpha, thresh, beta, interval = h
    T = shape[0]
    cut = min(cut, T)
    x, g = draw(shape, seed)
    mem, spike = c_oracle.fire_forward(x, alpha, thresh)
    mem_p, spike_p = c_oracle.fire_forward(np.ascontiguousarray(x[:cut]), alpha, thresh)
    assert np.array_equal(mem[:cut], mem_p) and np.array_equal(spike[:cut], spike_p)
    # the gradient at steps >= cut does not depend on spike gradients before cut
    g2 = g.copy()
    g2[:cut] = 0
    gx = c_oracle.fire_backward(x, g, alpha, thresh, beta, interval)
    gx2 = c_oracle.fire_backward(x, g2, alpha, thresh, beta, interval)
    assert np.array_equal(gx[cut:], gx2[cut:])


@settings(**SETTINGS)
@given(dims, hyper, seeds)
def test_neurons_are_independent_and_the_gradient_is_linear(shape, h, seed):
    alpha, thresh, beta, interval = h
    x, g = draw(shape, seed)
    T = shape[0]
    n = x[0].size
    perm = np.random.default_rng(seed + 1).permutation(n)
    flat = lambda a: a.reshape(T, 1, n)
    xs, gs = flat(x), flat(g)
    mem, spike = c_oracle.fire_forward(xs, alpha, thresh)
    gx = c_oracle.fire_backward(xs, gs, alpha, thresh, beta, interval)
    xp, gp = np.ascontiguousarray(xs[:, :, perm]), np.ascontiguousarray(gs[:, :, perm])
    mem_p, spike_p = c_oracle.fire_forward(xp, alpha, thresh)
    gx_p = c_oracle.fire_backward(xp, gp, alpha, thresh, beta, interval)
    assert np.array_equal(mem[:, :, perm], mem_p) and np.array_equal(spike[:, :, perm], spike_p)
    assert np.array_equal(gx[:, :, perm], gx_p)
    assert set(np.unique(spike)) <= {0.0, 1.0}
    # scaling by a power of two commutes with every rounding
    gx4 = c_oracle.fire_backward(xs, gs * 4, alpha, thresh, beta, interval)
    assert np.array_equal(gx4, gx * 4)
    assert not c_oracle.fire_backward(xs, np.zeros_like(gs), alpha, thresh, beta, interval).any()


@settings(**SETTINGS)
@given(st.tuples(st.integers(1, 3), st.integers(1, 60)), hyper, seeds)
def test_single_step_closed_form(bn, h, seed):
    alpha, thresh, beta, interval = h
    x, g = draw((1,) + bn, seed)
    mem, spike = c_oracle.fire_forward(x, alpha, thresh)
    gx = c_oracle.fire_backward(x, g, alpha, thresh, beta, interval)
    assert np.array_equal(mem, x)
    assert np.array_equal(spike, (x > np.float32(thresh)).astype(np.float32))
    window = ((x - np.float32(thresh)) < np.float32(interval)) & ((np.float32(thresh) - x) < np.float32(interval))
    assert np.array_equal(gx, np.where(window, g * np.float32(beta), np.float32(0)))


@settings(max_examples=30, deadline=None)
@given(dims, hyper, seeds)
def test_double_precision_loops_track_the_single_precision_ones(shape, h, seed):
    """Same inputs widened to fp64: spikes may differ only where a potential sits within rounding of
    the threshold; where they agree everywhere, potentials agree to fp32 accuracy."""
    alpha, thresh, beta, interval = h
    x, _ = draw(shape, seed)
    mem32, spike32 = c_oracle.fire_forward(x, alpha, thresh)
    mem64, spike64 = c_oracle.fire_forward(x.astype(np.float64), alpha, thresh)
    if np.array_equal(spike32, spike64):
        np.testing.assert_allclose(mem32, mem64, rtol=0, atol=1e-4)
