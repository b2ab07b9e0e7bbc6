"""Layer modules built on the fire operator.

``Fire`` has the reference's surface (snnlib/example/snnlib_op.py:11-16): no constructor
arguments, no parameters or buffers, ``forward(x) = fire_func(x)`` on a tensor shaped
``[T, B, C, H, W]`` or ``[T, B, C]``, returning 0.0 / 1.0 spikes of the same shape and dtype.
"""
import torch.nn as nn

from . import snnlib_func as sf


class Fire(nn.Module):
    def __init__(self):
        super(Fire, self).__init__()

    def forward(self, x):
        return sf.fire_func(x)
