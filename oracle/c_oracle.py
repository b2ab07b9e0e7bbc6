"""ctypes binding of ``oracle/lif_oracle.c`` (TEST INFRASTRUCTURE ONLY).

The C file restates the reference's fire kernels as scalar CPU loops
(snnlib/cuda/snn_kernel_fp.cu:37-52, snnlib/cuda/snn_kernel_bp.cu:34-51 and :117-138).  Arrays are numpy,
C-contiguous, shaped ``[T, B, ...]`` like the reference's tensors (``T = shape[0]``,
``B = shape[1]``, snnlib/cuda/snn_kernel_fp.cu:60-63).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liblif_oracle.so")
_lib = None


def build(force=False):
    """Compile ``lif_oracle.c`` into ``liblif_oracle.so`` next to it (needs gcc and make)."""
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)
    return _LIB_PATH


def _load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        build()
    lib = ctypes.CDLL(_LIB_PATH)
    i64, f32, ptr = ctypes.c_int64, ctypes.c_float, ctypes.c_void_p
    for sfx in ("f32", "f64"):
        getattr(lib, f"lif_oracle_forward_{sfx}").argtypes = [ptr, ptr, ptr, i64, i64, i64, f32, f32]
        getattr(lib, f"lif_oracle_forward_{sfx}").restype = None
        getattr(lib, f"lif_oracle_reverse_{sfx}").argtypes = [ptr, ptr, ptr, i64, i64, i64, f32, f32, f32, f32]
        getattr(lib, f"lif_oracle_reverse_{sfx}").restype = None
        getattr(lib, f"lif_oracle_backward_{sfx}").argtypes = [ptr, ptr, ptr, ptr, i64, i64, i64, f32, f32, f32, f32]
        getattr(lib, f"lif_oracle_backward_{sfx}").restype = None
        getattr(lib, f"lif_oracle_bn_forward_{sfx}").argtypes = [ptr] * 8 + [i64] * 4 + [f32] * 3
        getattr(lib, f"lif_oracle_bn_forward_{sfx}").restype = None
        getattr(lib, f"lif_oracle_bn_backward_{sfx}").argtypes = [ptr] * 9 + [i64] * 4 + [f32] * 4
        getattr(lib, f"lif_oracle_bn_backward_{sfx}").restype = None
        getattr(lib, f"lif_oracle_plain_bn_forward_{sfx}").argtypes = [ptr] * 7 + [i64] * 4 + [f32]
        getattr(lib, f"lif_oracle_plain_bn_forward_{sfx}").restype = None
        getattr(lib, f"lif_oracle_plain_bn_backward_{sfx}").argtypes = [ptr] * 8 + [i64] * 4
        getattr(lib, f"lif_oracle_plain_bn_backward_{sfx}").restype = None
    _lib = lib
    return lib


def _suffix(a):
    if a.dtype == np.float32:
        return "f32"
    if a.dtype == np.float64:
        return "f64"
    raise TypeError(f"oracle supports float32/float64 arrays, got {a.dtype}")


def _dims(a):
    if a.ndim < 2:
        raise ValueError("expected an array shaped [T, B, ...]")
    T, B = a.shape[0], a.shape[1]
    chw = int(np.prod(a.shape[2:], dtype=np.int64)) if a.ndim > 2 else 1
    return T, B, chw


def _p(a):
    return ctypes.c_void_p(a.ctypes.data) if a is not None else ctypes.c_void_p(0)


def fire_forward(x, alpha, thresh):
    """Return ``(mem, spike)``, both shaped and typed like ``x``."""
    x = np.ascontiguousarray(x)
    sfx = _suffix(x)
    T, B, chw = _dims(x)
    mem = np.empty_like(x)
    spike = np.empty_like(x)
    getattr(_load(), f"lif_oracle_forward_{sfx}")(_p(x), _p(mem), _p(spike), T, B, chw, alpha, thresh)
    return mem, spike


def fire_backward(x, grad_spike, alpha, thresh, beta, interval):
    """Return ``grad_x`` for the input current ``x`` and upstream spike gradient ``grad_spike``."""
    x = np.ascontiguousarray(x)
    g = np.ascontiguousarray(grad_spike, dtype=x.dtype)
    if g.shape != x.shape:
        raise ValueError("grad_spike must have the shape of x")
    sfx = _suffix(x)
    T, B, chw = _dims(x)
    gx = np.empty_like(x)
    scratch = np.empty_like(x)
    getattr(_load(), f"lif_oracle_backward_{sfx}")(_p(x), _p(g), _p(gx), _p(scratch), T, B, chw,
                                                  alpha, thresh, beta, interval)
    return gx


def _bn_dims(a):
    if a.ndim < 3:
        raise ValueError("expected an array shaped [T, B, C, ...]")
    T, B, C = a.shape[:3]
    hw = int(np.prod(a.shape[3:], dtype=np.int64)) if a.ndim > 3 else 1
    return T, B, C, hw


def _bn_real(x):
    """dtype the batch-norm loops run in: float64 for float64 input, float32 otherwise."""
    return np.float64 if np.asarray(x).dtype == np.float64 else np.float32


def bn_fire_forward(x, weight, bias, var, mean, eps, alpha, thresh):
    """Return ``(ivar, mem, spike)`` for fp32 or fp64 ``x`` shaped ``[T, B, C, ...]`` and ``[C]``
    parameters (converted to the dtype of ``x``)."""
    real = _bn_real(x)
    x, weight, bias, var, mean = (np.ascontiguousarray(a, dtype=real) for a in (x, weight, bias, var, mean))
    T, B, C, hw = _bn_dims(x)
    ivar = np.empty(C, dtype=real)
    mem, spike = np.empty_like(x), np.empty_like(x)
    fn = getattr(_load(), "lif_oracle_bn_forward_" + _suffix(x))
    fn(_p(x), _p(weight), _p(bias), _p(var), _p(mean), _p(ivar), _p(mem), _p(spike), T, B, C, hw,
       eps, alpha, thresh)
    return ivar, mem, spike


def bn_fire_backward(x, weight, bias, ivar, mean, grad_spike, alpha, thresh, beta, interval):
    """Return ``(grad_x, grad_weight, grad_bias)``."""
    real = _bn_real(x)
    x, weight, bias, ivar, mean, g = (np.ascontiguousarray(a, dtype=real)
                                      for a in (x, weight, bias, ivar, mean, grad_spike))
    T, B, C, hw = _bn_dims(x)
    gx = np.empty_like(x)
    gw, gb = np.empty(C, dtype=real), np.empty(C, dtype=real)
    fn = getattr(_load(), "lif_oracle_bn_backward_" + _suffix(x))
    fn(_p(x), _p(weight), _p(bias), _p(ivar), _p(mean), _p(g), _p(gx), _p(gw), _p(gb), T, B, C, hw,
       alpha, thresh, beta, interval)
    return gx, gw, gb


def bn_forward(x, weight, bias, var, mean, eps):
    """Plain batch norm with given statistics: return ``(ivar, y)`` for fp32 or fp64 ``x`` shaped
    ``[T, B, C, ...]`` (loops of snnlib/cuda/snn_kernel_fp.cu:102-121)."""
    real = _bn_real(x)
    x, weight, bias, var, mean = (np.ascontiguousarray(a, dtype=real) for a in (x, weight, bias, var, mean))
    T, B, C, hw = _bn_dims(x)
    ivar = np.empty(C, dtype=real)
    y = np.empty_like(x)
    fn = getattr(_load(), "lif_oracle_plain_bn_forward_" + _suffix(x))
    fn(_p(x), _p(weight), _p(bias), _p(var), _p(mean), _p(ivar), _p(y), T, B, C, hw, eps)
    return ivar, y


def bn_backward(x, weight, ivar, mean, grad_y):
    """Plain batch-norm backward: return ``(grad_x, grad_weight, grad_bias)`` (loops of
    snnlib/cuda/snn_kernel_bp.cu:202-234, 263-283)."""
    real = _bn_real(x)
    x, weight, ivar, mean, g = (np.ascontiguousarray(a, dtype=real) for a in (x, weight, ivar, mean, grad_y))
    T, B, C, hw = _bn_dims(x)
    gx = np.empty_like(x)
    gw, gb = np.empty(C, dtype=real), np.empty(C, dtype=real)
    fn = getattr(_load(), "lif_oracle_plain_bn_backward_" + _suffix(x))
    fn(_p(x), _p(weight), _p(ivar), _p(mean), _p(g), _p(gx), _p(gw), _p(gb), T, B, C, hw)
    return gx, gw, gb
