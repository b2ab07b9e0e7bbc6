"""Autograd functions of the snnlib layers and the hyper-parameters they read.

Same surface as the reference's ``snnlib_func.py`` for every single-GPU layer
(snnlib/example/snnlib_func.py:10-17 module-level settings; ``BnFunc`` :42-59, ``BnFireFunc`` :67-85,
``BnFireFcFunc`` :91-110, ``FireFcFunc`` :116-132, ``FcFunc`` :138-154, ``BnFireConvFunc`` :162-191,
``FireConvFunc`` :197-223, ``ConvFunc`` :229-253, ``FireFunc`` :22-36, each with its
``<name>_func = <Class>.apply`` alias), and for the sharded-batch forms ``BnDistFunc`` :261-288,
``BnFireFcDistFunc`` :297-327, ``BnFireConvDistFunc`` :336-377, whose backward runs the native op in
two halves with ``torch.distributed.all_reduce`` of two ``[C]`` vectors between them.

Contract shared by all of them, as in the reference: a forward saves only its *inputs* (plus the
per-channel inverse standard deviation a batch-norm forward returns) -- never spikes or membrane
potentials -- and calls the native ``snnlib.<op>_fp``; the backward calls ``snnlib.<op>_bp``, which
recomputes what it needs.  Hyper-parameters are module globals read at call time, so
``snnlib_func.thresh = 0.5`` takes effect on the next call.
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

# True: MIOpen searches for the fastest algorithm of each convolution shape the first time it sees it
# (slower first step, often a faster steady state); handed to the native convolution ops with every
# call, as the reference does (snnlib_func.py:17), and applied there for the duration of the call.
conv_benchmark = False

_DIM_FC = (0, 1)            # axes a fully connected bias gradient sums over
_DIM_CONV = (0, 1, 3, 4)    # axes a convolution bias gradient / conv-shaped batch norm sums over
_DILATION, _GROUPS = (1, 1), 1


def _dynamics():
    """Hyper-parameters of the forward recurrence, read from the module globals at call time."""
    return alpha, thresh


def _surrogate():
    """Those plus the surrogate-gradient parameters the backward ops take."""
    return alpha, thresh, beta, interval


def _pad(grads, n):
    """Gradients for the first inputs, ``None`` for the remaining non-tensor ones."""
    return tuple(grads) + (None,) * (n - len(grads))


class FireFunc(torch.autograd.Function):
    """spike = fire(spatial)."""

    @staticmethod
    def forward(ctx, spatial):
        ctx.save_for_backward(spatial)
        return snnlib.fire_s_fp(spatial, *_dynamics())

    @staticmethod
    def backward(ctx, grad_spike):
        (spatial,) = ctx.saved_tensors
        # the native op reads a gradient that is one row expanded over time (stride 0 on axis 0, as
        # after ``spike.sum(dim=0)``) in place and makes any other non-dense operand dense itself
        return snnlib.fire_bp(spatial, grad_spike, *_surrogate())


class BnFunc(torch.autograd.Function):
    """y = batch_norm(x) with the per-channel statistics handed in (no fire)."""

    @staticmethod
    def forward(ctx, x_bn, weight_bn, bias_bn, var, mean, dim_bn, eps_bn):
        ivar, y_bn = snnlib.bn_fp(x_bn, weight_bn, bias_bn, var, mean, eps_bn)
        ctx.save_for_backward(x_bn, weight_bn, bias_bn, ivar, mean)
        ctx.dim_bn = dim_bn
        return y_bn

    @staticmethod
    def backward(ctx, grad_y_bn):
        # saved: x_bn, weight_bn, bias_bn, ivar, mean
        return _pad(snnlib.bn_bp(*ctx.saved_tensors, ctx.dim_bn, grad_y_bn), 7)


class BnFireFunc(torch.autograd.Function):
    """spike = fire(batch_norm(spatial))."""

    @staticmethod
    def forward(ctx, spatial, weight_bn, bias_bn, var, mean, dim_bn, eps_bn):
        ivar, spike = snnlib.bn_fire_s_fp(spatial, weight_bn, bias_bn, var, mean, eps_bn, *_dynamics())
        ctx.save_for_backward(spatial, weight_bn, bias_bn, ivar, mean)
        ctx.dim_bn = dim_bn
        return spike

    @staticmethod
    def backward(ctx, grad_spike):
        # saved: spatial, weight_bn, bias_bn, ivar, mean
        return _pad(snnlib.bn_fire_bp(*ctx.saved_tensors, ctx.dim_bn, grad_spike, *_surrogate()), 7)


class BnFireFcFunc(torch.autograd.Function):
    """fc = linear(fire(batch_norm(spatial)))."""

    @staticmethod
    def forward(ctx, spatial, weight_bn, bias_bn, var, mean, dim_bn, eps_bn, weight_fc, bias_fc):
        ivar, fc = snnlib.bn_fire_fc_fp(spatial, weight_bn, bias_bn, var, mean, eps_bn,
                                        weight_fc, bias_fc, *_dynamics())
        ctx.save_for_backward(spatial, weight_bn, bias_bn, ivar, mean, weight_fc, bias_fc)
        ctx.dim_bn = dim_bn
        return fc

    @staticmethod
    def backward(ctx, grad_fc):
        *bn_saved, weight_fc, bias_fc = ctx.saved_tensors
        grads = snnlib.bn_fire_fc_bp(*bn_saved, ctx.dim_bn, grad_fc, weight_fc, bias_fc, _DIM_FC,
                                     *_surrogate())
        # spatial and the two batch-norm parameters, then var / mean / dim_bn / eps_bn, then the fc pair
        return (*grads[:3], None, None, None, None, *grads[3:])


class FireFcFunc(torch.autograd.Function):
    """fc = linear(fire(spatial))."""

    @staticmethod
    def forward(ctx, spatial, weight_fc, bias_fc):
        ctx.save_for_backward(spatial, weight_fc, bias_fc)
        return snnlib.fire_fc_fp(spatial, weight_fc, bias_fc, *_dynamics())

    @staticmethod
    def backward(ctx, grad_fc):
        spatial, *fc_params = ctx.saved_tensors
        return tuple(snnlib.fire_fc_bp(spatial, grad_fc, *fc_params, _DIM_FC, *_surrogate()))


class FcFunc(torch.autograd.Function):
    """fc = linear(spatial) per time step (no fire)."""

    @staticmethod
    def forward(ctx, spatial, weight_fc, bias_fc):
        ctx.save_for_backward(spatial, weight_fc, bias_fc)
        return snnlib.fc_fp(spatial, weight_fc, bias_fc)

    @staticmethod
    def backward(ctx, grad_fc):
        spatial, *fc_params = ctx.saved_tensors
        return tuple(snnlib.fc_bp(spatial, grad_fc, *fc_params, _DIM_FC))


def _conv_grads(ctx, g_spatial, g_weight, g_bias, leading=()):
    """Order the convolution-layer gradients the way ``forward``'s arguments are ordered; the bias
    gradient is dropped when the layer was built with ``if_bias_conv=False``."""
    return leading + (g_weight, g_bias if ctx.if_bias_conv else None, None, None, None)


class BnFireConvFunc(torch.autograd.Function):
    """conv = conv2d(fire(batch_norm(spatial))) (dilation 1, groups 1, as in the reference)."""

    @staticmethod
    def forward(ctx, spatial, weight_bn, bias_bn, var, mean, eps_bn,
                weight_conv, bias_conv, stride, padding, if_bias_conv):
        ivar, conv = snnlib.bn_fire_conv_fp(spatial, weight_bn, bias_bn, var, mean, eps_bn,
                                            weight_conv, bias_conv, stride, padding, _DILATION, _GROUPS,
                                            conv_benchmark, False, *_dynamics())
        ctx.save_for_backward(spatial, weight_bn, bias_bn, ivar, mean, weight_conv, bias_conv)
        ctx.stride, ctx.padding, ctx.if_bias_conv = stride, padding, if_bias_conv
        return conv

    @staticmethod
    def backward(ctx, grad_conv):
        *bn_saved, weight_conv, _ = ctx.saved_tensors
        g_spatial, g_weight_bn, g_bias_bn, g_weight_conv, g_bias_conv = snnlib.bn_fire_conv_bp(
            *bn_saved, _DIM_CONV, grad_conv, weight_conv, ctx.stride, ctx.padding, _DILATION, _GROUPS,
            conv_benchmark, False, True, _DIM_CONV, *_surrogate())
        return _conv_grads(ctx, g_spatial, g_weight_conv, g_bias_conv,
                           leading=(g_spatial, g_weight_bn, g_bias_bn, None, None, None))


class FireConvFunc(torch.autograd.Function):
    """conv = conv2d(fire(spatial))."""

    @staticmethod
    def forward(ctx, spatial, weight_conv, bias_conv, stride, padding, if_bias_conv):
        ctx.save_for_backward(spatial, weight_conv, bias_conv)
        ctx.stride, ctx.padding, ctx.if_bias_conv = stride, padding, if_bias_conv
        return snnlib.fire_conv_fp(spatial, weight_conv, bias_conv, stride, padding, _DILATION, _GROUPS,
                                   conv_benchmark, False, *_dynamics())

    @staticmethod
    def backward(ctx, grad_conv):
        spatial, weight_conv, bias_conv = ctx.saved_tensors
        g_spatial, g_weight_conv, g_bias_conv = snnlib.fire_conv_bp(
            spatial, grad_conv, weight_conv, ctx.stride, ctx.padding, _DILATION, _GROUPS,
            conv_benchmark, False, True, _DIM_CONV, *_surrogate())
        return _conv_grads(ctx, g_spatial, g_weight_conv, g_bias_conv, leading=(g_spatial,))


class ConvFunc(torch.autograd.Function):
    """conv = conv2d(spatial) per time step (no fire)."""

    @staticmethod
    def forward(ctx, spatial, weight_conv, bias_conv, stride, padding, if_bias_conv):
        ctx.save_for_backward(spatial, weight_conv, bias_conv)
        ctx.stride, ctx.padding, ctx.if_bias_conv = stride, padding, if_bias_conv
        return snnlib.conv_fp(spatial, weight_conv, bias_conv, stride, padding, _DILATION, _GROUPS,
                              conv_benchmark, False)

    @staticmethod
    def backward(ctx, grad_conv):
        spatial, weight_conv, bias_conv = ctx.saved_tensors
        g_spatial, g_weight_conv, g_bias_conv = snnlib.conv_bp(
            spatial, grad_conv, weight_conv, ctx.stride, ctx.padding, _DILATION, _GROUPS,
            conv_benchmark, False, True, _DIM_CONV)
        return _conv_grads(ctx, g_spatial, g_weight_conv, g_bias_conv, leading=(g_spatial,))


def _mean_over_ranks(local_xhat, local_xhatx, reduce_op):
    """All-reduce the two per-channel means of a sharded batch and average them.
    ``reduce_op`` is the reference's triple ``[ReduceOp, process_group, world_size]``."""
    kinds, group, world_size = reduce_op
    torch.distributed.all_reduce(local_xhat, kinds.SUM, group)
    torch.distributed.all_reduce(local_xhatx, kinds.SUM, group)
    return local_xhat / world_size, local_xhatx / world_size


class BnDistFunc(BnFunc):
    """``BnFunc`` for a batch sharded over the ranks of a process group; one more argument, the
    ``[ReduceOp, process_group, world_size]`` triple, follows ``BnFunc``'s."""

    @staticmethod
    def forward(ctx, *args):
        ctx.reduce_op = args[-1]
        return BnFunc.forward(ctx, *args[:-1])

    @staticmethod
    def backward(ctx, grad_y_bn):
        saved = ctx.saved_tensors          # x_bn, weight_bn, bias_bn, ivar, mean
        local_xhat, local_xhatx, g_weight_bn, g_bias_bn = snnlib.bn_bp_dist1(
            *saved, ctx.dim_bn, grad_y_bn)
        g_x_bn = snnlib.bn_bp_dist2(*saved, ctx.dim_bn, grad_y_bn,
                                    *_mean_over_ranks(local_xhat, local_xhatx, ctx.reduce_op))
        return _pad((g_x_bn, g_weight_bn, g_bias_bn), 8)


def _sharded_bn_fire_input_grad(ctx, bn_saved, g_spike, local_xhat, local_xhatx):
    """Second half of a sharded bn + fire backward: average the means, then the input gradient."""
    g_xhat, g_xhatx = _mean_over_ranks(local_xhat, local_xhatx, ctx.reduce_op)
    return snnlib.bn_fire_bp_dist2(*bn_saved, g_spike, g_xhat, g_xhatx, *_surrogate())


class BnFireFcDistFunc(BnFireFcFunc):
    """``BnFireFcFunc`` for a sharded batch (same arguments plus the reduce triple)."""

    @staticmethod
    def forward(ctx, *args):
        ctx.reduce_op = args[-1]
        return BnFireFcFunc.forward(ctx, *args[:-1])

    @staticmethod
    def backward(ctx, grad_fc):
        *bn_saved, weight_fc, bias_fc = ctx.saved_tensors
        g_spike, local_xhat, local_xhatx, *param_grads = snnlib.bn_fire_fc_bp_dist1(
            *bn_saved, ctx.dim_bn, grad_fc, weight_fc, bias_fc, _DIM_FC, *_surrogate())
        g_weight_bn, g_bias_bn, g_weight_fc, g_bias_fc = param_grads
        g_spatial = _sharded_bn_fire_input_grad(ctx, bn_saved, g_spike, local_xhat, local_xhatx)
        return (g_spatial, g_weight_bn, g_bias_bn, None, None, None, None, g_weight_fc, g_bias_fc,
                None)


class BnFireConvDistFunc(BnFireConvFunc):
    """``BnFireConvFunc`` for a sharded batch (same arguments plus the reduce triple)."""

    @staticmethod
    def forward(ctx, *args):
        ctx.reduce_op = args[-1]
        return BnFireConvFunc.forward(ctx, *args[:-1])

    @staticmethod
    def backward(ctx, grad_conv):
        *bn_saved, weight_conv, _ = ctx.saved_tensors
        g_spike, local_xhat, local_xhatx, *param_grads = snnlib.bn_fire_conv_bp_dist1(
            *bn_saved, _DIM_CONV, grad_conv, weight_conv, ctx.stride, ctx.padding, _DILATION, _GROUPS,
            conv_benchmark, False, True, _DIM_CONV, *_surrogate())
        g_weight_bn, g_bias_bn, g_weight_conv, g_bias_conv = param_grads
        g_spatial = _sharded_bn_fire_input_grad(ctx, bn_saved, g_spike, local_xhat, local_xhatx)
        return _conv_grads(ctx, g_spatial, g_weight_conv, g_bias_conv,
                           leading=(g_spatial, g_weight_bn, g_bias_bn, None, None, None)) + (None,)


fire_func = FireFunc.apply
bn_func = BnFunc.apply
bn_fire_func = BnFireFunc.apply
bn_fire_fc_func = BnFireFcFunc.apply
fire_fc_func = FireFcFunc.apply
fc_func = FcFunc.apply
bn_fire_conv_func = BnFireConvFunc.apply
fire_conv_func = FireConvFunc.apply
conv_func = ConvFunc.apply
bn_dist_func = BnDistFunc.apply
bn_fire_fc_dist_func = BnFireFcDistFunc.apply
bn_fire_conv_dist_func = BnFireConvDistFunc.apply
