"""The benchmark configurations at their full sizes on the GPU, checked through properties that do
not need a full-size CPU run:

* neuron independence -- a random sample of neuron columns, gathered from the full-size device
  tensors, must equal the oracle run on just those columns (exact for fp32; spikes exact and
  gradients equal to the fp32 result rounded once for bf16 storage), for the spikes, the membrane
  potential of snnlif_fire_us_fp and the input gradient, in both the streamed instantiations of the
  kernels (what tensors of this size get without a hint) and the kept ones;
* prefix property     -- the first T' steps of the full window equal a run over a T'-step window;
* linearity           -- scaling the spike gradient by 4 scales the input gradient by 4, bit for bit;
* the stored golden vectors (tests/golden/fire_vectors.json) are reproduced exactly.
"""
import json
import os

import numpy as np
import pytest
import torch

from conftest import ALPHA, BETA, INTERVAL, THRESH

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))

FULL = {
    # name: (shape, mean, std, dtype)
    "cfg2": ((8, 64, 128, 32, 32), 0.5, 1.0, torch.float32),
    "cfg3": ((32, 32, 256, 16, 16), 0.3, 0.8, torch.float32),
    "cfg5": ((16, 128, 512, 16, 16), 0.5, 1.0, torch.float32),
    "cfg5_bf16": ((16, 128, 512, 16, 16), 0.5, 1.0, torch.bfloat16),
    # the fire layers of the synthetic training step (configuration 4) that differ from cfg2
    "cfg4_conv2": ((8, 64, 256, 32, 32), 0.5, 1.0, torch.float32),
    "cfg4_conv3": ((8, 64, 256, 16, 16), 0.5, 1.0, torch.float32),
    "cfg4_fc": ((8, 64, 1024), 0.5, 1.0, torch.float32),
}


@pytest.fixture(scope="module")
def cabi():
    from snn_gpu_training_bptt_amd import lif_cabi
    lif_cabi.load()
    return lif_cabi


@pytest.fixture(scope="module")
def oracle():
    from oracle import c_oracle
    return c_oracle


@pytest.mark.parametrize("keep", [None, True], ids=["by-size", "kept"])
@pytest.mark.parametrize("name", list(FULL))
def test_full_size_configuration(cabi, oracle, name, keep):
    shape, mean, std, dtype = FULL[name]
    T = shape[0]
    N = int(np.prod(shape[1:]))
    gen = torch.Generator(device="cuda").manual_seed(2024)
    x = (mean + std * torch.randn(shape, generator=gen, device="cuda")).to(dtype)
    g = torch.randn(shape, generator=gen, device="cuda").to(dtype)
    spike = torch.empty_like(x)
    gx = torch.empty_like(x)
    cabi.fire_s_fp_into(x, spike, ALPHA, THRESH, keep_spatial=keep)
    cabi.fire_bp_into(x, g, gx, ALPHA, THRESH, BETA, INTERVAL, keep_spatial=keep)
    torch.cuda.synchronize()

    # -- sampled neurons against the oracle
    idx = torch.randint(0, N, (min(N, 200_000),), generator=torch.Generator().manual_seed(1)).cuda()
    idx[:4] = torch.tensor([0, 1, N - 2, N - 1])        # both ends of the tensor
    take = lambda t: t.view(T, N)[:, idx].float().cpu().numpy().reshape(T, 1, -1)
    xs, gs = take(x), take(g)
    mem_o, spike_o = oracle.fire_forward(xs, ALPHA, THRESH)
    gx_o = oracle.fire_backward(xs, gs, ALPHA, THRESH, BETA, INTERVAL)
    assert np.array_equal(take(spike), spike_o), "sampled spikes differ from the oracle"
    # the membrane potential of the (u, spike) forward, and its spikes, on the same sample
    mem, spike_b = torch.empty_like(x), torch.empty_like(x)
    cabi.fire_us_fp_into(x, mem, spike_b, ALPHA, THRESH, keep_spatial=keep)
    assert torch.equal(spike_b, spike)
    mem_expect = mem_o if dtype == torch.float32 else torch.from_numpy(mem_o).to(dtype).float().numpy()
    assert np.array_equal(take(mem), mem_expect), "sampled membrane potentials differ from the oracle"
    del mem, spike_b
    if dtype == torch.float32:
        assert np.array_equal(take(gx), gx_o), "sampled gradients differ from the oracle"
    else:
        expect = torch.from_numpy(gx_o).to(dtype).float().numpy()
        assert np.array_equal(take(gx), expect), "sampled gradients differ from the rounded oracle"
        np.testing.assert_allclose(take(gx), gx_o, rtol=1e-2, atol=1e-3)
    rate = spike.float().mean().item()
    assert 0.05 < rate < 0.95
    assert bool(((spike == 0) | (spike == 1)).all())

    # -- prefix property on the device
    Tp = T // 2
    spike_p = torch.empty_like(x[:Tp])
    cabi.fire_s_fp_into(x[:Tp], spike_p, ALPHA, THRESH, keep_spatial=keep)
    assert torch.equal(spike_p, spike[:Tp])
    del spike_p

    # -- linearity in the spike gradient (power-of-two scale commutes with rounding)
    g4 = g * 4
    gx4 = torch.empty_like(x)
    cabi.fire_bp_into(x, g4, gx4, ALPHA, THRESH, BETA, INTERVAL, keep_spatial=keep)
    assert torch.equal(gx4, gx * 4)


def test_golden_vectors_on_gpu(cabi):
    with open(os.path.join(HERE, "golden", "fire_vectors.json")) as f:
        data = json.load(f)

    def unpack(rows, shape):
        flat = [int(r[i:i + 8], 16) for r in rows for i in range(0, len(r), 8)]
        return torch.from_numpy(np.array(flat, dtype=np.uint32).view(np.float32).reshape(shape).copy())

    for case in data["cases"]:
        shape, h = case["shape"], case["hyper"]
        x = unpack(case["x"], shape).cuda()
        g = unpack(case["grad_spike"], shape).cuda()
        mem, spike, gx = torch.empty_like(x), torch.empty_like(x), torch.empty_like(x)
        cabi.fire_us_fp_into(x, mem, spike, h["alpha"], h["thresh"])
        cabi.fire_bp_into(x, g, gx, h["alpha"], h["thresh"], h["beta"], h["interval"])
        torch.cuda.synchronize()
        assert torch.equal(spike.cpu(), unpack(case["spike"], shape)), case["name"]
        assert torch.equal(mem.cpu(), unpack(case["mem"], shape)), case["name"]
        assert torch.equal(gx.cpu(), unpack(case["grad_x"], shape)), case["name"]
