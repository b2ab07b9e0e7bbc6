"""Autograd functions of the LIF fire layers and the hyper-parameters they read.

Same surface as the reference's ``snnlib_func.py`` for the fire path
(snnlib/example/snnlib_func.py:10-17 for the module-level settings, :22-36 for ``FireFunc`` /
``fire_func``, :67-85 for ``BnFireFunc`` / ``bn_fire_func``, :116-132 for ``FireFcFunc`` / ``fire_fc_func``, :197-223 for ``FireConvFunc`` /
``fire_conv_func``): every forward saves only its inputs (never spikes or membrane potentials) and
calls the native ``snnlib.<op>_fp``; every backward calls ``snnlib.<op>_bp``, which recomputes what
it needs.  The hyper-parameters are module globals read at call time, so
``snnlib_func.thresh = 0.5`` takes effect on the next call, as it does in the reference.
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

conv_benchmark = False  # accepted for interface parity; MIOpen's search follows torch.backends.cudnn


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


class BnFireFunc(torch.autograd.Function):
    """spike = fire(batch_norm(spatial)) with the given per-channel statistics
    (snnlib/example/snnlib_func.py:67-85).  Saves the input current, the affine parameters, the
    inverse standard deviation returned by the forward, and the mean."""

    @staticmethod
    def forward(ctx, spatial, weight_bn, bias_bn, var, mean, dim_bn, eps_bn):
        ivar, spike = snnlib.bn_fire_s_fp(spatial, weight_bn, bias_bn, var, mean, eps_bn, alpha, thresh)
        ctx.save_for_backward(spatial, weight_bn, bias_bn, ivar, mean)
        ctx.dim_bn = dim_bn
        return spike

    @staticmethod
    def backward(ctx, grad_spike):
        spatial, weight_bn, bias_bn, ivar, mean = ctx.saved_tensors
        grad_spatial, grad_weight_bn, grad_bias_bn = snnlib.bn_fire_bp(
            spatial, weight_bn, bias_bn, ivar, mean, ctx.dim_bn, grad_spike, alpha, thresh, beta, interval)
        return grad_spatial, grad_weight_bn, grad_bias_bn, None, None, None, None


bn_fire_func = BnFireFunc.apply


class FireFcFunc(torch.autograd.Function):
    """fc = linear(fire(spatial)) per time step; gradients for the input current, weight and bias."""

    @staticmethod
    def forward(ctx, spatial, weight_fc, bias_fc):
        fc = snnlib.fire_fc_fp(spatial, weight_fc, bias_fc, alpha, thresh)
        ctx.save_for_backward(spatial, weight_fc, bias_fc)
        return fc

    @staticmethod
    def backward(ctx, grad_fc):
        spatial, weight_fc, bias_fc = ctx.saved_tensors
        grad_spatial, grad_weight_fc, grad_bias_fc = snnlib.fire_fc_bp(
            spatial, grad_fc, weight_fc, bias_fc, (0, 1), alpha, thresh, beta, interval)
        return grad_spatial, grad_weight_fc, grad_bias_fc


fire_fc_func = FireFcFunc.apply


class FireConvFunc(torch.autograd.Function):
    """conv = conv2d(fire(spatial)) per time step (dilation 1, groups 1, as in the reference)."""

    @staticmethod
    def forward(ctx, spatial, weight_conv, bias_conv, stride, padding, if_bias_conv):
        conv = snnlib.fire_conv_fp(spatial, weight_conv, bias_conv, stride, padding, (1, 1), 1,
                                   conv_benchmark, False, alpha, thresh)
        ctx.save_for_backward(spatial, weight_conv, bias_conv)
        ctx.stride, ctx.padding, ctx.if_bias_conv = stride, padding, if_bias_conv
        return conv

    @staticmethod
    def backward(ctx, grad_conv):
        spatial, weight_conv, bias_conv = ctx.saved_tensors
        grad_spatial, grad_weight_conv, grad_bias_conv = snnlib.fire_conv_bp(
            spatial, grad_conv, weight_conv, ctx.stride, ctx.padding, (1, 1), 1, conv_benchmark,
            False, True, (0, 1, 3, 4), alpha, thresh, beta, interval)
        if ctx.if_bias_conv:
            return grad_spatial, grad_weight_conv, grad_bias_conv, None, None, None
        return grad_spatial, grad_weight_conv, None, None, None, None


fire_conv_func = FireConvFunc.apply
