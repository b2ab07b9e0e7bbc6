"""Layer modules of the snnlib interface (single GPU).

Class names, constructor arguments, parameter names and initialisation are the reference's
(snnlib/example/snnlib_op.py): ``Fire`` :11-16, ``Bn`` :19-50, ``BnFire`` :53-84, ``BnFireFc`` :87-128,
``FireFc`` :131-139, ``Fc`` :141-149, ``BnFireConv`` :152-192, ``FireConv`` :195-210, ``Conv`` :214-228.
Inputs are ``[T, B, C, H, W]`` or ``[T, B, C]`` tensors; each module forwards to the matching
``snnlib_func.<name>_func``.  ``BnDist`` :231-281, ``BnFireFcDist`` :284-344 and ``BnFireConvDist``
:347-405 are the same layers for a batch sharded over the ranks of ``torch.distributed``'s default
process group (one rank per GPU): the batch statistics and, in the backward, two per-channel means
are all-reduced, so every rank normalises with the statistics of the whole batch.

Batch-norm behaviour shared by the ``Bn*`` modules, as in the reference: ``train_bn`` (not
``nn.Module.training``) selects batch statistics (biased variance and mean over ``dim_bn``, which the
reference takes from ``torch.var_mean(..., unbiased=False)`` and this build from its own reduction
kernel, ``snnlib.bn_stats``) or the running ones; the running statistics are ``nn.Parameter`` objects that are
*replaced* on every training-mode call (momentum 0.1, variance corrected by n/(n-1), n = elements
per channel of the first input seen).
"""
import math

import torch
import torch.nn as nn

from . import snnlib_func as sf


def _channel_major_input(x, dim_bn):
    """``x`` detached, after checking that ``dim_bn`` names every axis but the channel's (axis 2):
    the native batch-norm ops, like the reference's, take the channel from axis 2 and reduce over
    all others, so no other ``dim_bn`` is meaningful for a ``[T, B, C, ...]`` input."""
    wanted = tuple(d for d in range(x.dim()) if d != 2)
    if tuple(sorted(d % x.dim() for d in dim_bn)) != wanted:
        raise ValueError(f"dim_bn={tuple(dim_bn)} must name every axis of a {x.dim()}-d input except "
                         f"the channel axis 2, i.e. {wanted}")
    return x.detach()


class _BatchStatistics(nn.Module):
    """Affine parameters and running statistics of a per-channel batch norm over ``channels``."""

    def _init_batch_norm(self, channels, dim_bn, eps_bn):
        self.dim_bn = dim_bn
        self.eps_bn = eps_bn
        self._bn_channels = channels
        self.weight_bn = nn.Parameter(torch.ones(channels))
        self.bias_bn = nn.Parameter(torch.zeros(channels))
        self.running_var = nn.Parameter(torch.ones(channels))
        self.running_mean = nn.Parameter(torch.zeros(channels))
        self.factor = None
        self.train_bn = True

    def _statistics(self, x):
        """(var, mean) to normalise ``x`` with; updates the running pair in training mode."""
        if self.factor is None:
            per_channel = x.numel() / self._bn_channels
            self.factor = per_channel / (per_channel - 1)
            self.running_var = self.running_var.to(x.device)
            self.running_mean = self.running_mean.to(x.device)
        if not self.train_bn:
            return self.running_var, self.running_mean
        # one native call: the statistics and running * 0.9 + statistic * 0.1 (the variance's gain
        # carries the unbiasing factor), the bits of the reference's element-wise expressions
        var, mean, running_var, running_mean = sf.snnlib.bn_stats_running(
            _channel_major_input(x, self.dim_bn), self.running_var, self.running_mean, 0.9, 0.1 * self.factor, 0.1)
        self.running_var = nn.Parameter(running_var)
        self.running_mean = nn.Parameter(running_mean)
        return var, mean


class _ShardedBatchStatistics(_BatchStatistics):
    """Batch statistics of a batch that is sharded over the default process group: each rank
    contributes E[x] and E[x^2] of its shard (shards of equal size), var = E[x^2] - E[x]^2.
    Running statistics move with momentum 0.05."""

    def _init_batch_norm(self, channels, dim_bn, eps_bn):
        super()._init_batch_norm(channels, dim_bn, eps_bn)
        self.ReduceOp = torch.distributed.ReduceOp

    def _statistics(self, x):
        if self.factor is None:
            per_channel = x.numel() / self._bn_channels
            self.factor = per_channel / (per_channel - 1)
            self.running_var = nn.Parameter(self.running_var.to(x.device))
            self.running_mean = nn.Parameter(self.running_mean.to(x.device))
            self.process_group = torch.distributed.group.WORLD
            self.world_size = torch.distributed.get_world_size(self.process_group)
        if not self.train_bn:
            return self.running_var, self.running_mean
        first, second = sf.snnlib.bn_moments(_channel_major_input(x, self.dim_bn))
        torch.distributed.all_reduce(first, self.ReduceOp.SUM, self.process_group)
        torch.distributed.all_reduce(second, self.ReduceOp.SUM, self.process_group)
        # mean = first / world, var = second / world - mean ** 2 and the running pair (momentum 0.05), the
        # bits of the reference's element-wise expressions, in one native call
        var, mean, running_var, running_mean = sf.snnlib.bn_moments_finish(
            first, second, self.world_size, self.running_var, self.running_mean, 0.95, 0.05 * self.factor, 0.05)
        self.running_var = nn.Parameter(running_var)
        self.running_mean = nn.Parameter(running_mean)
        return var, mean

    def _reduce_op(self):
        """What the ``*_dist_func`` functions take as their last argument."""
        return [self.ReduceOp, self.process_group, self.world_size]


def _fc_parameters(module, cin, cout, like_linear):
    if like_linear:   # nn.Linear's default initialisation
        fc = nn.Linear(cin, cout, bias=True)
        module.weight_fc, module.bias_fc = nn.Parameter(fc.weight), nn.Parameter(fc.bias)
    else:             # N(0, 0.75/sqrt(cin)) weights, zero bias
        module.weight_fc = nn.Parameter(nn.init.normal_(torch.zeros(cout, cin), 0, 0.75 / math.sqrt(cin)))
        module.bias_fc = nn.Parameter(torch.zeros(cout))


def _conv_attributes(module, cin, stride, padding, if_bias_conv):
    module.cin = cin
    module.stride = stride
    module.padding = padding
    module.if_bias_conv = if_bias_conv


class Fire(nn.Module):
    def __init__(self):
        super(Fire, self).__init__()

    def forward(self, x):
        return sf.fire_func(x)


class Bn(_BatchStatistics):
    def __init__(self, cin, dim_bn, eps_bn=1e-5):
        super(Bn, self).__init__()
        self.cin = cin
        self._init_batch_norm(cin, dim_bn, eps_bn)

    def forward(self, x):
        var, mean = self._statistics(x)
        return sf.bn_func(x, self.weight_bn, self.bias_bn, var, mean, self.dim_bn, self.eps_bn)


class BnFire(_BatchStatistics):
    def __init__(self, cin, dim_bn, eps_bn=1e-5):
        super(BnFire, self).__init__()
        self.cin = cin
        self._init_batch_norm(cin, dim_bn, eps_bn)

    def forward(self, x):
        var, mean = self._statistics(x)
        return sf.bn_fire_func(x, self.weight_bn, self.bias_bn, var, mean, self.dim_bn, self.eps_bn)


class BnFireFc(_BatchStatistics):
    """``cin_bn`` is the channel count of the batch norm when the input is still an image
    (``[T, B, cin_bn, H, W]`` with ``cin = cin_bn*H*W`` features for the linear layer)."""

    def __init__(self, cin, cout, dim_bn, eps_bn=1e-5, cin_bn=None):
        super(BnFireFc, self).__init__()
        self.cin = cin
        self.cin_bn = cin if cin_bn is None else cin_bn
        self._init_batch_norm(self.cin_bn, dim_bn, eps_bn)
        _fc_parameters(self, cin, cout, like_linear=True)

    def forward(self, x):
        var, mean = self._statistics(x)
        return sf.bn_fire_fc_func(x, self.weight_bn, self.bias_bn, var, mean, self.dim_bn, self.eps_bn,
                                  self.weight_fc, self.bias_fc)


class FireFc(nn.Module):
    def __init__(self, cin, cout):
        super(FireFc, self).__init__()
        _fc_parameters(self, cin, cout, like_linear=False)

    def forward(self, x):
        return sf.fire_fc_func(x, self.weight_fc, self.bias_fc)


class Fc(nn.Module):
    def __init__(self, cin, cout):
        super(Fc, self).__init__()
        _fc_parameters(self, cin, cout, like_linear=False)

    def forward(self, x):
        return sf.fc_func(x, self.weight_fc, self.bias_fc)


class BnFireConv(_BatchStatistics):
    def __init__(self, cin, cout, kernel_size=(3, 3), stride=(1, 1), padding=(1, 1), eps_bn=1e-5,
                 if_bias_conv=True):
        super(BnFireConv, self).__init__()
        _conv_attributes(self, cin, stride, padding, if_bias_conv)
        self._init_batch_norm(cin, (0, 1, 3, 4), eps_bn)
        conv = nn.Conv2d(cin, cout, kernel_size, stride, padding)
        self.weight_conv = nn.Parameter(conv.weight)
        self.bias_conv = nn.Parameter(conv.bias)

    def forward(self, x):
        var, mean = self._statistics(x)
        return sf.bn_fire_conv_func(x, self.weight_bn, self.bias_bn, var, mean, self.eps_bn,
                                    self.weight_conv, self.bias_conv, self.stride, self.padding,
                                    self.if_bias_conv)


class FireConv(nn.Module):
    def __init__(self, cin, cout, kernel_size=(3, 3), stride=(1, 1), padding=(1, 1), if_bias_conv=True):
        super(FireConv, self).__init__()
        _conv_attributes(self, cin, stride, padding, if_bias_conv)
        conv = nn.Conv2d(cin, cout, kernel_size, stride, padding)
        self.weight_conv = nn.Parameter(conv.weight)
        self.bias_conv = nn.Parameter(conv.bias)

    def forward(self, x):
        return sf.fire_conv_func(x, self.weight_conv, self.bias_conv, self.stride, self.padding,
                                 self.if_bias_conv)


class Conv(nn.Module):
    def __init__(self, cin, cout, kernel_size=(3, 3), stride=(1, 1), padding=(1, 1), if_bias_conv=True):
        super(Conv, self).__init__()
        _conv_attributes(self, cin, stride, padding, if_bias_conv)
        self.weight_conv = nn.Parameter(nn.init.normal_(
            torch.zeros(cout, cin, kernel_size[0], kernel_size[1]), 0, 0.75 / math.sqrt(cin)))
        self.bias_conv = nn.Parameter(torch.zeros(cout))

    def forward(self, x):
        return sf.conv_func(x, self.weight_conv, self.bias_conv, self.stride, self.padding,
                            self.if_bias_conv)


class BnDist(_ShardedBatchStatistics):
    def __init__(self, cin, dim_bn, eps_bn=1e-5):
        super(BnDist, self).__init__()
        self.cin = cin
        self._init_batch_norm(cin, dim_bn, eps_bn)

    def forward(self, x):
        var, mean = self._statistics(x)
        return sf.bn_dist_func(x, self.weight_bn, self.bias_bn, var, mean, self.dim_bn, self.eps_bn,
                               self._reduce_op())


class BnFireFcDist(_ShardedBatchStatistics):
    def __init__(self, cin, cout, dim_bn, eps_bn=1e-5, cin_bn=None):
        super(BnFireFcDist, self).__init__()
        self.cin = cin
        self.cin_bn = cin if cin_bn is None else cin_bn
        self._init_batch_norm(self.cin_bn, dim_bn, eps_bn)
        _fc_parameters(self, cin, cout, like_linear=True)

    def forward(self, x):
        var, mean = self._statistics(x)
        return sf.bn_fire_fc_dist_func(x, self.weight_bn, self.bias_bn, var, mean, self.dim_bn,
                                       self.eps_bn, self.weight_fc, self.bias_fc, self._reduce_op())


class BnFireConvDist(_ShardedBatchStatistics):
    def __init__(self, cin, cout, kernel_size=(3, 3), stride=(1, 1), padding=(1, 1), eps_bn=1e-5,
                 if_bias_conv=True):
        super(BnFireConvDist, self).__init__()
        _conv_attributes(self, cin, stride, padding, if_bias_conv)
        self._init_batch_norm(cin, (0, 1, 3, 4), eps_bn)
        conv = nn.Conv2d(cin, cout, kernel_size, stride, padding)
        self.weight_conv = nn.Parameter(conv.weight)
        self.bias_conv = nn.Parameter(conv.bias)

    def forward(self, x):
        var, mean = self._statistics(x)
        return sf.bn_fire_conv_dist_func(x, self.weight_bn, self.bias_bn, var, mean, self.eps_bn,
                                         self.weight_conv, self.bias_conv, self.stride, self.padding,
                                         self.if_bias_conv, self._reduce_op())
