"""Layer modules built on the fire operator.

``Fire`` has the reference's surface (snnlib/example/snnlib_op.py:11-16): no constructor
arguments, no parameters or buffers, ``forward(x) = fire_func(x)`` on a tensor shaped
``[T, B, C, H, W]`` or ``[T, B, C]``, returning 0.0 / 1.0 spikes of the same shape and dtype.
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
