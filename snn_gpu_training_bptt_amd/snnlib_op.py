"""Layer modules built on the fire operator.

``Fire`` has the reference's surface (snnlib/example/snnlib_op.py:11-16): no constructor
arguments, no parameters or buffers, ``forward(x) = fire_func(x)`` on a tensor shaped
``[T, B, C, H, W]`` or ``[T, B, C]``, returning 0.0 / 1.0 spikes of the same shape and dtype.
``BnFire`` (snnlib/example/snnlib_op.py:53-84) applies a batch norm inside the recurrence.
``FireFc`` (snnlib/example/snnlib_op.py:131-139) and ``FireConv`` (:195-210) feed those spikes to a
fully connected / 3x3-style convolution layer; constructor arguments, parameter names and
initialisation are the reference's.
"""
import math

import torch
import torch.nn as nn

from . import snnlib_func as sf


class Fire(nn.Module):
    def __init__(self):
        super(Fire, self).__init__()

    def forward(self, x):
        return sf.fire_func(x)


class BnFire(nn.Module):
    """Batch norm folded into the fire recurrence (snnlib/example/snnlib_op.py:53-84).

    ``dim_bn`` names the axes the statistics run over: ``(0, 1)`` for ``[T, B, C]`` inputs,
    ``(0, 1, 3, 4)`` for ``[T, B, C, H, W]``.  As in the reference, the running statistics are held
    as ``nn.Parameter`` objects that are *replaced* on every training-mode call (momentum 0.1, the
    variance corrected by n/(n-1)), and ``train_bn`` -- not ``nn.Module.training`` -- selects between
    batch and running statistics.
    """

    def __init__(self, cin, dim_bn, eps_bn=1e-5):
        super(BnFire, self).__init__()
        self.cin = cin
        self.dim_bn = dim_bn
        self.eps_bn = eps_bn
        self.weight_bn = nn.Parameter(torch.ones(cin))
        self.bias_bn = nn.Parameter(torch.zeros(cin))
        self.running_var = nn.Parameter(torch.ones(cin))
        self.running_mean = nn.Parameter(torch.zeros(cin))
        self.factor = None
        self.train_bn = True

    def forward(self, x):
        if self.factor is None:
            factor = x.numel() / self.cin
            self.factor = factor / (factor - 1)
            self.running_var = self.running_var.to(x.device)
            self.running_mean = self.running_mean.to(x.device)

        if self.train_bn:
            var, mean = torch.var_mean(x, dim=self.dim_bn, unbiased=False)
            self.running_var = nn.Parameter(self.running_var * 0.9 + var * (0.1 * self.factor))
            self.running_mean = nn.Parameter(self.running_mean * 0.9 + mean * 0.1)
        else:
            var, mean = self.running_var, self.running_mean

        return sf.bn_fire_func(x, self.weight_bn, self.bias_bn, var, mean, self.dim_bn, self.eps_bn)


class FireFc(nn.Module):
    def __init__(self, cin, cout):
        super(FireFc, self).__init__()
        self.weight_fc = nn.Parameter(nn.init.normal_(torch.zeros(cout, cin), 0, 0.75 / math.sqrt(cin)))
        self.bias_fc = nn.Parameter(torch.zeros(cout))

    def forward(self, x):
        return sf.fire_fc_func(x, self.weight_fc, self.bias_fc)


class FireConv(nn.Module):
    def __init__(self, cin, cout, kernel_size=(3, 3), stride=(1, 1), padding=(1, 1), if_bias_conv=True):
        super(FireConv, self).__init__()
        self.cin = cin
        self.stride = stride
        self.padding = padding
        self.if_bias_conv = if_bias_conv
        conv = nn.Conv2d(cin, cout, kernel_size, stride, padding)
        self.weight_conv = nn.Parameter(conv.weight)
        self.bias_conv = nn.Parameter(conv.bias)

    def forward(self, x):
        return sf.fire_conv_func(x, self.weight_conv, self.bias_conv, self.stride, self.padding,
                                 self.if_bias_conv)
