"""Autograd function of the LIF fire layer and the hyper-parameters it reads.

Same surface as the reference's ``snnlib_func.py`` for the fire path
(snnlib/example/snnlib_func.py:10-15 for the module-level hyper-parameters, :22-36 for ``FireFunc``
and ``fire_func``): the forward saves only the input current and calls
``snnlib.fire_s_fp(spatial, alpha, thresh)``; the backward calls
``snnlib.fire_bp(spatial, grad_spike, alpha, thresh, beta, interval)``.  The hyper-parameters are
module globals read at call time, so ``snnlib_func.thresh = 0.5`` takes effect on the next call,
as it does in the reference.
"""
import torch

from ._loader import load_snnlib

snnlib = load_snnlib()

# hyper parameter setting (defaults of snnlib/example/snnlib_func.py:10-15)
alpha = 0.25
beta = 1.0
interval = 0.5
thresh = 0.25
time_step = 6


class FireFunc(torch.autograd.Function):
    """spike = fire(spatial); only ``spatial`` is kept for the backward."""

    @staticmethod
    def forward(ctx, spatial):
        ctx.save_for_backward(spatial)
        return snnlib.fire_s_fp(spatial, alpha, thresh)

    @staticmethod
    def backward(ctx, grad_spike):
        (spatial,) = ctx.saved_tensors
        # the native op makes both operands dense itself (the upstream gradient is often a
        # stride-0 expansion, e.g. after a mean over time)
        return snnlib.fire_bp(spatial, grad_spike, alpha, thresh, beta, interval)


fire_func = FireFunc.apply
