"""Pure-PyTorch restatement of the reference's gold LIF fire path (TEST INFRASTRUCTURE ONLY).

Follows snnlib/example/gold_op.py:17-44 operation for operation -- Heaviside forward with the
rectangular surrogate gradient (:17-29), and the time loop ``u[t] = x[t] + 0``,
``u[t] += u[t-1] * (1 - s[t-1]) * alpha`` for t > 0, ``s[t] = fire(u[t])`` (:34-44) -- with two
deliberate differences: the window length is ``x.shape[0]`` instead of the module constant
``time_step`` (:12, :37), and the hyper-parameters are arguments instead of module constants (:8-11).
The spike is not detached, so autograd carries the reset-path gradient exactly as the reference's
graph does.  This is the parity target of the HIP kernels and the path ``bench.py`` times on the
host CPU as ``cpu_baseline``.
"""
import torch


class _Heaviside(torch.autograd.Function):
    """``u > thresh`` forward; ``grad * 1[|u - thresh| < interval] * beta`` backward."""

    @staticmethod
    def forward(ctx, u, thresh, beta, interval):
        ctx.save_for_backward(u)
        ctx.hyper = (thresh, beta, interval)
        return u.gt(thresh).to(u.dtype)

    @staticmethod
    def backward(ctx, grad_out):
        (u,) = ctx.saved_tensors
        thresh, beta, interval = ctx.hyper
        window = (abs(u - thresh) < interval).to(u.dtype)
        return grad_out.clone() * window * beta, None, None, None


def gold_fire(x, alpha, thresh, beta=1.0, interval=0.5):
    """Return ``(u, s)`` stacked over time for input current ``x`` shaped ``[T, ...]``."""
    u, s = [], []
    for t in range(x.shape[0]):
        u.append(x[t] + 0)
        if t > 0:
            u[t] += u[t - 1] * (1 - s[t - 1]) * alpha
        s.append(_Heaviside.apply(u[t], thresh, beta, interval))
    return torch.stack(u, dim=0), torch.stack(s, dim=0)


def gold_fire_fwd_bwd(x, grad_spike, alpha, thresh, beta=1.0, interval=0.5):
    """Forward plus ``s.backward(grad_spike)``; returns ``(u, s, grad_x)`` (all detached)."""
    xr = x.detach().clone().requires_grad_(True)
    u, s = gold_fire(xr, alpha, thresh, beta, interval)
    s.backward(grad_spike)
    return u.detach(), s.detach(), xr.grad.detach()


def gold_fire_fc(x, weight, bias, alpha, thresh, beta=1.0, interval=0.5):
    """Fire, then one ``linear`` per time step on the flattened spikes
    (snnlib/example/gold_op.py:113-145 with ``fire=True``).  Returns ``[T, B, cout]``."""
    _, s = gold_fire(x, alpha, thresh, beta, interval)
    if s.dim() == 5:
        s = s.view(s.shape[0], s.shape[1], -1)
    return torch.stack([torch.nn.functional.linear(s[t], weight, bias) for t in range(s.shape[0])], dim=0)


def gold_fire_conv(x, weight, bias, stride, padding, alpha, thresh, beta=1.0, interval=0.5):
    """Fire, then one ``conv2d`` per time step (snnlib/example/gold_op.py:148-179 with
    ``fire=True``).  Returns ``[T, B, cout, Hout, Wout]``."""
    _, s = gold_fire(x, alpha, thresh, beta, interval)
    return torch.stack([torch.nn.functional.conv2d(s[t], weight, bias, stride, padding)
                        for t in range(s.shape[0])], dim=0)


def gold_bn_fire(x, weight, bias, running_mean, running_var, training, eps, alpha, thresh,
                 beta=1.0, interval=0.5):
    """Batch norm over the folded (T*B) batch, then the fire loop (snnlib/example/gold_op.py:67-87,
    whose ``bn`` is ``nn.BatchNorm1d`` / ``nn.BatchNorm2d``).  Returns ``(u, s)``.  With
    ``training=True`` the statistics are those of ``x`` itself, as in the reference layer's training
    mode (snnlib/example/snnlib_op.py:78 computes them with ``torch.var_mean(..., unbiased=False)``)."""
    shape = x.shape
    y = torch.nn.functional.batch_norm(x.reshape(shape[0] * shape[1], *shape[2:]), running_mean,
                                       running_var, weight, bias, training, 0.1, eps).reshape(shape)
    return gold_fire(y, alpha, thresh, beta, interval)


def _per_step(fn, x):
    return torch.stack([fn(x[t]) for t in range(x.shape[0])], dim=0)


def gold_bn(x, weight, bias, running_mean, running_var, training, eps):
    """Batch norm over the folded (T*B) batch (snnlib/example/gold_op.py:49-62)."""
    shape = x.shape
    return torch.nn.functional.batch_norm(x.reshape(shape[0] * shape[1], *shape[2:]), running_mean,
                                          running_var, weight, bias, training, 0.1, eps).reshape(shape)


def gold_fc(x, weight, bias):
    """One ``linear`` per time step on the flattened input (snnlib/example/gold_op.py:113-145 with
    neither ``bn_fire`` nor ``fire``)."""
    if x.dim() == 5:
        x = x.view(x.shape[0], x.shape[1], -1)
    return _per_step(lambda xt: torch.nn.functional.linear(xt, weight, bias), x)


def gold_conv(x, weight, bias, stride, padding):
    """One ``conv2d`` per time step (snnlib/example/gold_op.py:148-179 with neither flag)."""
    return _per_step(lambda xt: torch.nn.functional.conv2d(xt, weight, bias, stride, padding), x)


def gold_bn_fire_fc(x, weight_bn, bias_bn, running_mean, running_var, training, eps, weight_fc, bias_fc,
                    alpha, thresh, beta=1.0, interval=0.5):
    """snnlib/example/gold_op.py:113-145 with ``bn_fire=True``."""
    _, s = gold_bn_fire(x, weight_bn, bias_bn, running_mean, running_var, training, eps, alpha, thresh,
                        beta, interval)
    return gold_fc(s, weight_fc, bias_fc)


def gold_bn_fire_conv(x, weight_bn, bias_bn, running_mean, running_var, training, eps, weight_conv,
                      bias_conv, stride, padding, alpha, thresh, beta=1.0, interval=0.5):
    """snnlib/example/gold_op.py:148-179 with ``bn_fire=True``."""
    _, s = gold_bn_fire(x, weight_bn, bias_bn, running_mean, running_var, training, eps, alpha, thresh,
                        beta, interval)
    return gold_conv(s, weight_conv, bias_conv, stride, padding)
