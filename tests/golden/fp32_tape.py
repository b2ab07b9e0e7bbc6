"""A tiny scalar reverse-mode autodiff with IEEE fp32 rounding after every elementary operation,
in pure Python.  It exists to pin the CPU oracle from a direction that shares no code with it:

* values are Python floats forced through ``struct.pack('f')`` after each +, -, * (double
  arithmetic followed by one rounding to fp32 is exact fp32 arithmetic for these operations,
  because a double holds the exact product of two fp32 values and 53 >= 2*24 + 2 bits make the
  double-rounded sum innocuous);
* the forward graph is the one the reference's pure-PyTorch gold path builds
  (snnlib/example/gold_op.py:34-44): ``u[t] = x[t] + 0``; for t > 0
  ``u[t] = u[t] + ((u[t-1] * (1 - s[t-1])) * alpha)``; ``s[t] = fire(u[t])``;
* the fire node's derivative is the rectangular surrogate of snnlib/example/gold_op.py:25-29:
  ``grad_in = (grad_out * 1[|u - thresh| < interval]) * beta``;
* adjoints are accumulated per node in the order PyTorch's engine would add them (fp32 addition is
  commutative, so the order of the two contributions to a node does not matter; no node here
  receives more than two).

Nothing here is used by the shipped package; the GPU kernels are never checked against this module
directly, only through the oracle it pins and through the vectors it generated.
"""
import struct


def f32(v):
    """Round a Python float to the nearest fp32 (ties to even) and return it as a float."""
    return struct.unpack("f", struct.pack("f", v))[0]


class Node:
    __slots__ = ("value", "grad", "parents")

    def __init__(self, value, parents=()):
        self.value = f32(value)
        self.grad = 0.0
        self.parents = parents  # tuple of (node, function mapping this node's grad to the parent's share)


def leaf(v):
    return Node(v)


def add(a, b):
    return Node(a.value + b.value, ((a, lambda g: g), (b, lambda g: g)))


def add_const(a, c):
    return Node(a.value + c, ((a, lambda g: g),))


def mul(a, b):
    av, bv = a.value, b.value
    return Node(av * bv, ((a, lambda g: f32(g * bv)), (b, lambda g: f32(g * av))))


def mul_const(a, c):
    c = f32(c)
    return Node(a.value * c, ((a, lambda g: f32(g * c)),))


def one_minus(a):
    return Node(1.0 - a.value, ((a, lambda g: -g),))


def fire(u, thresh, beta, interval):
    thresh, beta, interval = f32(thresh), f32(beta), f32(interval)
    uv = u.value
    window = 1.0 if abs(f32(uv - thresh)) < interval else 0.0
    return Node(1.0 if uv > thresh else 0.0, ((u, lambda g: f32(f32(g * window) * beta)),))


def backward(order, seeds):
    """``order``: nodes in creation order; ``seeds``: {node: upstream gradient}."""
    for node, g in seeds.items():
        node.grad = f32(node.grad + g)
    for node in reversed(order):
        for parent, share in node.parents:
            parent.grad = f32(parent.grad + share(node.grad))


def gold_fire_neuron(x, g, alpha, thresh, beta, interval):
    """One neuron: currents ``x[0..T-1]``, spike gradients ``g[0..T-1]`` ->
    ``(u, s, grad_x)`` as lists of Python floats holding fp32 values."""
    T = len(x)
    order = []

    def track(n):
        order.append(n)
        return n

    xs = [track(leaf(v)) for v in x]
    u, s = [], []
    for t in range(T):
        ut = track(add_const(xs[t], 0.0))
        if t > 0:
            keep = track(one_minus(s[t - 1]))
            carried = track(mul_const(track(mul(u[t - 1], keep)), alpha))
            ut = track(add(ut, carried))
        u.append(ut)
        s.append(track(fire(ut, thresh, beta, interval)))
    backward(order, {s[t]: f32(g[t]) for t in range(T)})
    return [n.value for n in u], [n.value for n in s], [n.grad for n in xs]
