"""ctypes view of the C ABI in ``include/snnlib_lif.h`` (``libsnnlif_gfx950.so``).

This is the boundary the parity tests and the benchmark drive directly: raw device pointers, sizes
and a stream handle, no torch types in any signature.  The helpers at the bottom only unwrap
``torch.Tensor`` arguments into those pointers; they allocate nothing except the outputs the caller
asks for and never fall back to another implementation -- if the library is missing, loading raises.
"""
import ctypes
import os

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG_DIR, "lib", "libsnnlif_gfx950.so")

DTYPE_F32, DTYPE_F64, DTYPE_BF16 = 0, 1, 2
# cache hints, or-ed into dtype: the caller will / will not read `spatial` again soon
KEEP_SPATIAL, STREAM_SPATIAL = 0x100, 0x200
OK, ERR_ARG, ERR_DTYPE, ERR_WORKSPACE, ERR_ALIGN, ERR_UNSUPPORTED, ERR_SCRATCH = 0, -1, -2, -3, -4, -5, -6
STATIC_SCRATCH_BYTES = 16 << 20
BP_FUSED_MAX_T = 32
BP_NO_WORKSPACE_MAX_T = 1024

# name -> (restype, argtypes); must list every symbol include/snnlib_lif.h declares.
_vp, _i64, _f32, _int, _sz = ctypes.c_void_p, ctypes.c_int64, ctypes.c_float, ctypes.c_int, ctypes.c_size_t
_f64 = ctypes.c_double
SYMBOLS = {
    "snnlif_abi_version": (_int, []),
    "snnlif_target_arch": (ctypes.c_char_p, []),
    "snnlif_strerror": (ctypes.c_char_p, [_int]),
    "snnlif_time_next_kernel": (_int, [_vp, _vp]),
    "snnlif_fire_s_fp": (_int, [_vp, _vp, _int, _i64, _i64, _f32, _f32, _vp]),
    "snnlif_fire_us_fp": (_int, [_vp, _vp, _vp, _int, _i64, _i64, _f32, _f32, _vp]),
    "snnlif_fire_bp_workspace_bytes": (_sz, [_int, _i64, _i64]),
    "snnlif_fire_bp": (_int, [_vp, _vp, _vp, _int, _i64, _i64, _f32, _f32, _f32, _f32, _vp, _sz, _vp]),
    "snnlif_fire_bp_strided": (_int, [_vp, _vp, _vp, _int, _i64, _i64, _i64, _f32, _f32, _f32, _f32, _vp,
                                      _sz, _vp]),
    "snnlif_bn_stats_workspace_bytes": (_sz, [_int, _i64, _i64, _i64, _i64]),
    "snnlif_bn_stats": (_int, [_vp, _vp, _vp, _int, _i64, _i64, _i64, _i64, _int, _vp, _sz, _vp]),
    "snnlif_bn_stats_running": (_int, [_vp] * 7 + [_f64, _f64, _f64, _int, _i64, _i64, _i64, _i64, _vp, _sz, _vp]),
    "snnlif_bn_moments_finish": (_int, [_vp] * 8 + [_f64, _f64, _f64, _f64, _int, _i64, _vp]),
    "snnlif_channel_sum": (_int, [_vp, _vp, _int, _i64, _i64, _i64, _i64, _vp, _sz, _vp]),
    "snnlif_bn_fire_s_fp": (_int, [_vp] * 7 + [_int, _i64, _i64, _i64, _i64, _f32, _f32, _f32, _vp]),
    "snnlif_bn_fire_s_recompute": (_int, [_vp] * 6 + [_int, _i64, _i64, _i64, _i64, _f32, _f32, _vp]),
    "snnlif_bn_fire_bp_workspace_bytes": (_sz, [_int, _i64, _i64, _i64, _i64]),
    "snnlif_bn_fire_bp": (_int, [_vp] * 9 + [_int, _i64, _i64, _i64, _i64, _f32, _f32, _f32, _f32, _vp, _sz, _vp]),
    "snnlif_bn_fire_bp_static": (_int, [_vp] * 9 + [_int, _i64, _i64, _i64, _i64, _f32, _f32, _f32, _f32, _vp]),
    "snnlif_bn_fire_bp_dist1": (_int, [_vp] * 10 + [_int, _i64, _i64, _i64, _i64, _f32, _f32, _f32, _f32, _vp, _sz, _vp]),
    "snnlif_bn_fire_bp_dist2": (_int, [_vp] * 9 + [_int, _i64, _i64, _i64, _i64, _f32, _f32, _f32, _f32, _vp]),
    "snnlif_bn_fp": (_int, [_vp] * 7 + [_int, _i64, _i64, _i64, _i64, _f32, _vp]),
    "snnlif_bn_bp_workspace_bytes": (_sz, [_int, _i64, _i64, _i64, _i64]),
    "snnlif_bn_bp": (_int, [_vp] * 8 + [_int, _i64, _i64, _i64, _i64, _vp, _sz, _vp]),
    "snnlif_bn_bp_dist1": (_int, [_vp] * 9 + [_int, _i64, _i64, _i64, _i64, _vp, _sz, _vp]),
    "snnlif_bn_bp_dist2": (_int, [_vp] * 8 + [_int, _i64, _i64, _i64, _i64, _vp]),
}
ABI_VERSION = 3

_lib = None


class SnnlifError(RuntimeError):
    def __init__(self, code, where):
        self.code = code
        super().__init__(f"{where}: {strerror(code)} (code {code})")


def load():
    """Load the library once and type its entry points.  Raises if it has not been built.
    ``SNNLIF_LIBRARY`` in the environment names another build of the same library to load instead of
    the in-tree one (e.g. one compiled with different tuning macros, for A/B measurements)."""
    global _lib
    if _lib is not None:
        return _lib
    path = os.environ.get("SNNLIF_LIBRARY") or LIB_PATH
    if not os.path.exists(path):
        raise ImportError(
            f"{path} is missing: build it with `python -m snn_gpu_training_bptt_amd.build` "
            "(there is no CPU or PyTorch fallback for the LIF fire kernels)")
    lib = ctypes.CDLL(path)
    for name, (restype, argtypes) in SYMBOLS.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def strerror(code):
    return load().snnlif_strerror(int(code)).decode()


def _check(rc, where):
    if rc != OK:
        raise SnnlifError(rc, where)


# ---- thin tensor-unwrapping helpers (used by tests and bench; torch is plumbing only) ----------

def _torch_dtype_code(t):
    import torch
    codes = {torch.float32: DTYPE_F32, torch.float64: DTYPE_F64, torch.bfloat16: DTYPE_BF16}
    if t.dtype not in codes:
        raise TypeError(f"unsupported dtype {t.dtype}")
    return codes[t.dtype]


def _dims(t):
    T = t.shape[0]
    return T, (t.numel() // T if T else 0)


def _stream_handle(t):
    import torch
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _require_dense_gpu(*tensors):
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise ValueError("device tensor required")
        if not t.is_contiguous():
            raise ValueError("dense (contiguous) tensor required")


def _require_like(spatial, **tensors):
    """Every named tensor must have ``spatial``'s shape, dtype and device: the C ABI sees only
    pointers and derives all sizes from ``spatial``, so a smaller or differently typed buffer would
    become an out-of-bounds device access."""
    for name, t in tensors.items():
        if t is None:
            continue
        if t.shape != spatial.shape:
            raise ValueError(f"{name} has shape {tuple(t.shape)}, spatial has {tuple(spatial.shape)}")
        if t.dtype != spatial.dtype:
            raise ValueError(f"{name} has dtype {t.dtype}, spatial has {spatial.dtype}")
        if t.device != spatial.device:
            raise ValueError(f"{name} is on {t.device}, spatial is on {spatial.device}")


def _require_per_channel(spatial, channels, **tensors):
    """Per-channel vectors: ``channels`` values of ``spatial``'s dtype on its device."""
    for name, t in tensors.items():
        if t.numel() != channels:
            raise ValueError(f"{name} has {t.numel()} values, spatial has {channels} channels")
        if t.dtype != spatial.dtype:
            raise ValueError(f"{name} has dtype {t.dtype}, spatial has {spatial.dtype}")
        if t.device != spatial.device:
            raise ValueError(f"{name} is on {t.device}, spatial is on {spatial.device}")


def _require_workspace(spatial, workspace, need, what):
    """A uint8 device buffer of at least ``need`` bytes (``None`` allowed when nothing is needed)."""
    import torch
    if workspace is None:
        if need:
            raise ValueError(f"{what} needs a workspace of {need} bytes")
        return
    if workspace.dtype != torch.uint8:
        raise ValueError(f"workspace must be a uint8 tensor, got {workspace.dtype}")
    if workspace.device != spatial.device:
        raise ValueError(f"workspace is on {workspace.device}, spatial is on {spatial.device}")
    if workspace.numel() < need:
        raise ValueError(f"workspace holds {workspace.numel()} bytes, {what} needs {need}")


def _workspace_args(workspace):
    """(pointer, bytes) of a uint8 workspace tensor; (NULL, 0) for ``None``."""
    if workspace is None:
        return None, 0
    return workspace.data_ptr(), workspace.numel() * workspace.element_size()


def time_next_kernel(start_event, stop_event):
    """Attach two ``torch.cuda.Event(enable_timing=True)`` objects to the next kernel this thread
    launches through the library (see ``snnlif_time_next_kernel``).  The events must already exist
    on the device side, i.e. have been recorded at least once; ``None`` stands for no event."""
    handle = lambda e: ctypes.c_void_p(None if e is None else e.cuda_event)
    _check(load().snnlif_time_next_kernel(handle(start_event), handle(stop_event)),
           "snnlif_time_next_kernel")


def _hinted(dtype_code, keep_spatial):
    """``keep_spatial``: True -> SNNLIF_KEEP_SPATIAL, False -> SNNLIF_STREAM_SPATIAL, None -> no hint."""
    if keep_spatial is None:
        return dtype_code
    return dtype_code | (KEEP_SPATIAL if keep_spatial else STREAM_SPATIAL)


def fire_s_fp_into(spatial, spike, alpha, thresh, keep_spatial=None):
    """``snnlif_fire_s_fp`` on torch tensors already resident on the GPU; writes ``spike``.
    ``keep_spatial`` (True / False / None) selects the cache hint, see ``_hinted``."""
    _require_like(spatial, spike=spike)
    T, N = _dims(spatial)
    _require_dense_gpu(spatial, spike)
    rc = load().snnlif_fire_s_fp(spatial.data_ptr(), spike.data_ptr(),
                                 _hinted(_torch_dtype_code(spatial), keep_spatial), T, N, alpha,
                                 thresh, _stream_handle(spatial))
    _check(rc, "snnlif_fire_s_fp")
    return spike


def fire_us_fp_into(spatial, mem, spike, alpha, thresh, keep_spatial=None):
    """``snnlif_fire_us_fp``; ``mem`` or ``spike`` may be None to skip that output."""
    _require_like(spatial, mem=mem, spike=spike)
    T, N = _dims(spatial)
    _require_dense_gpu(spatial, mem, spike)
    rc = load().snnlif_fire_us_fp(spatial.data_ptr(),
                                  mem.data_ptr() if mem is not None else None,
                                  spike.data_ptr() if spike is not None else None,
                                  _hinted(_torch_dtype_code(spatial), keep_spatial), T, N, alpha,
                                  thresh, _stream_handle(spatial))
    _check(rc, "snnlif_fire_us_fp")
    return mem, spike


def fire_bp_workspace_bytes(dtype_code, T, N):
    return int(load().snnlif_fire_bp_workspace_bytes(dtype_code, T, N))


def _grad_row_stride(grad_spike, N):
    """Elements between consecutive time rows of ``grad_spike`` as ``snnlif_fire_bp_strided`` takes
    them: N for a dense tensor, 0 for one row expanded over time, more than N for rows of a wider
    tensor.  Each row itself must be dense."""
    if grad_spike.is_contiguous():
        return N
    if grad_spike.dim() >= 2 and grad_spike[0].is_contiguous():
        stride = grad_spike.stride(0)
        if stride == 0 or stride >= N:
            return stride
    raise ValueError("grad_spike: dense time rows required (the time axis may have any stride >= N, or 0)")


def fire_bp_into(spatial, grad_spike, grad_spatial, alpha, thresh, beta, interval, workspace=None,
                 keep_spatial=None):
    """``snnlif_fire_bp_strided`` (``snnlif_fire_bp`` for a dense gradient); ``workspace`` is a uint8
    device tensor when the shape needs one.  ``grad_spike`` may be a stride-0 expansion over time
    (``row.expand(T, ...)``): it is read in place."""
    _require_like(spatial, grad_spike=grad_spike, grad_spatial=grad_spatial)
    T, N = _dims(spatial)
    _require_workspace(spatial, workspace, fire_bp_workspace_bytes(_torch_dtype_code(spatial), T, N),
                       "snnlif_fire_bp")
    ws_ptr = workspace.data_ptr() if workspace is not None else None
    ws_bytes = workspace.numel() * workspace.element_size() if workspace is not None else 0
    grad_row_stride = _grad_row_stride(grad_spike, N)
    if not grad_spike.is_cuda:
        raise ValueError("device tensor required")
    _require_dense_gpu(spatial, grad_spatial, workspace)
    if grad_row_stride == N:
        rc = load().snnlif_fire_bp(spatial.data_ptr(), grad_spike.data_ptr(), grad_spatial.data_ptr(),
                                   _hinted(_torch_dtype_code(spatial), keep_spatial), T, N, alpha,
                                   thresh, beta, interval, ws_ptr, ws_bytes, _stream_handle(spatial))
        _check(rc, "snnlif_fire_bp")
    else:
        rc = load().snnlif_fire_bp_strided(spatial.data_ptr(), grad_spike.data_ptr(),
                                           grad_spatial.data_ptr(),
                                           _hinted(_torch_dtype_code(spatial), keep_spatial), T, N,
                                           grad_row_stride, alpha, thresh, beta, interval, ws_ptr,
                                           ws_bytes, _stream_handle(spatial))
        _check(rc, "snnlif_fire_bp_strided")
    return grad_spatial


def _bn_dims(t):
    T, B, C = t.shape[0], t.shape[1], t.shape[2]
    HW = t.numel() // (T * B * C) if T * B * C else 0
    return T, B, C, HW


def bn_stats_workspace_bytes(dtype_code, T, B, C, HW):
    return int(load().snnlif_bn_stats_workspace_bytes(dtype_code, T, B, C, HW))


def bn_stats_into(spatial, mean, var, workspace, raw_moments=False):
    """``snnlif_bn_stats``: per-channel mean and biased variance of ``spatial`` ([T, B, C, ...]) over all
    axes but the channel's, or E[x] and E[x^2] with ``raw_moments``; writes ``mean`` and ``var`` ([C])."""
    T, B, C, HW = _bn_dims(spatial)
    _require_per_channel(spatial, C, mean=mean, var=var)
    _require_workspace(spatial, workspace,
                       bn_stats_workspace_bytes(_torch_dtype_code(spatial), T, B, C, HW),
                       "snnlif_bn_stats")
    _require_dense_gpu(spatial, mean, var, workspace)
    rc = load().snnlif_bn_stats(spatial.data_ptr(), mean.data_ptr(), var.data_ptr(),
                                _torch_dtype_code(spatial), T, B, C, HW, int(bool(raw_moments)),
                                workspace.data_ptr(), workspace.numel(), _stream_handle(spatial))
    _check(rc, "snnlif_bn_stats")
    return mean, var


def bn_stats_running_into(spatial, mean, var, running_mean, running_var, new_running_mean, new_running_var,
                          workspace, keep, gain_mean, gain_var):
    """``snnlif_bn_stats_running``: ``bn_stats_into`` plus the layer's running statistics,
    ``new = running * keep + statistic * gain`` rounded like the framework's element-wise expression."""
    T, B, C, HW = _bn_dims(spatial)
    _require_per_channel(spatial, C, mean=mean, var=var, running_mean=running_mean, running_var=running_var,
                         new_running_mean=new_running_mean, new_running_var=new_running_var)
    _require_workspace(spatial, workspace,
                       bn_stats_workspace_bytes(_torch_dtype_code(spatial), T, B, C, HW),
                       "snnlif_bn_stats_running")
    _require_dense_gpu(spatial, mean, var, running_mean, running_var, new_running_mean, new_running_var, workspace)
    rc = load().snnlif_bn_stats_running(spatial.data_ptr(), mean.data_ptr(), var.data_ptr(),
                                        running_mean.data_ptr(), running_var.data_ptr(),
                                        new_running_mean.data_ptr(), new_running_var.data_ptr(),
                                        float(keep), float(gain_mean), float(gain_var),
                                        _torch_dtype_code(spatial), T, B, C, HW, workspace.data_ptr(),
                                        workspace.numel(), _stream_handle(spatial))
    _check(rc, "snnlif_bn_stats_running")
    return mean, var, new_running_mean, new_running_var


def bn_moments_finish_into(first, second, mean, var, world_size, running=None):
    """``snnlif_bn_moments_finish``: mean and variance of a sharded batch from its all-reduced moments;
    ``running`` = (running_mean, running_var, new_running_mean, new_running_var, keep, gain_mean, gain_var)
    also advances the running pair."""
    C = first.numel()
    _require_per_channel(first, C, second=second, mean=mean, var=var)
    tensors = [first, second, mean, var]
    ptrs = [0, 0, 0, 0]
    factors = (1.0, 0.0, 0.0)
    if running is not None:
        _require_per_channel(first, C, running_mean=running[0], running_var=running[1],
                             new_running_mean=running[2], new_running_var=running[3])
        tensors += list(running[:4])
        ptrs = [t.data_ptr() for t in running[:4]]
        factors = tuple(float(f) for f in running[4:7])
    _require_dense_gpu(*tensors)
    rc = load().snnlif_bn_moments_finish(first.data_ptr(), second.data_ptr(), mean.data_ptr(), var.data_ptr(),
                                         ptrs[0] or None, ptrs[1] or None, ptrs[2] or None, ptrs[3] or None,
                                         float(world_size), factors[0], factors[1], factors[2],
                                         _torch_dtype_code(first), C, _stream_handle(first))
    _check(rc, "snnlif_bn_moments_finish")
    return mean, var


def channel_sum_into(grad, total, workspace):
    """``snnlif_channel_sum``: per-channel sum of ``grad`` ([T, B, C, ...]) over all axes but the
    channel's; writes ``total`` ([C]).  ``workspace`` as for ``bn_stats_into``."""
    T, B, C, HW = _bn_dims(grad)
    _require_per_channel(grad, C, total=total)
    _require_workspace(grad, workspace, bn_stats_workspace_bytes(_torch_dtype_code(grad), T, B, C, HW),
                       "snnlif_channel_sum")
    _require_dense_gpu(grad, total, workspace)
    rc = load().snnlif_channel_sum(grad.data_ptr(), total.data_ptr(), _torch_dtype_code(grad), T, B, C,
                                   HW, workspace.data_ptr(), workspace.numel(), _stream_handle(grad))
    _check(rc, "snnlif_channel_sum")
    return total


def bn_fire_s_fp_into(spatial, weight, bias, var, mean, ivar, spike, eps, alpha, thresh, keep_spatial=None):
    """``snnlif_bn_fire_s_fp`` on fp32 / fp64 device tensors; writes ``ivar`` ([C]) and ``spike``.
    ``keep_spatial``: the cache hint as in the fire helpers (True / False / None = by size)."""
    T, B, C, HW = _bn_dims(spatial)
    _require_like(spatial, spike=spike)
    _require_per_channel(spatial, C, weight=weight, bias=bias, var=var, mean=mean, ivar=ivar)
    _require_dense_gpu(spatial, weight, bias, var, mean, ivar, spike)
    rc = load().snnlif_bn_fire_s_fp(spatial.data_ptr(), weight.data_ptr(), bias.data_ptr(),
                                    var.data_ptr(), mean.data_ptr(), ivar.data_ptr(),
                                    spike.data_ptr(), _hinted(_torch_dtype_code(spatial), keep_spatial),
                                    T, B, C, HW, eps, alpha, thresh, _stream_handle(spatial))
    _check(rc, "snnlif_bn_fire_s_fp")
    return ivar, spike


def bn_fire_s_recompute_into(spatial, weight, bias, ivar, mean, spike, alpha, thresh, keep_spatial=None):
    """``snnlif_bn_fire_s_recompute``: spikes from saved ``ivar`` / ``mean`` (backward-side scale)."""
    T, B, C, HW = _bn_dims(spatial)
    _require_like(spatial, spike=spike)
    _require_per_channel(spatial, C, weight=weight, bias=bias, ivar=ivar, mean=mean)
    _require_dense_gpu(spatial, weight, bias, ivar, mean, spike)
    rc = load().snnlif_bn_fire_s_recompute(spatial.data_ptr(), weight.data_ptr(), bias.data_ptr(),
                                           ivar.data_ptr(), mean.data_ptr(), spike.data_ptr(),
                                           _hinted(_torch_dtype_code(spatial), keep_spatial), T, B, C,
                                           HW, alpha, thresh, _stream_handle(spatial))
    _check(rc, "snnlif_bn_fire_s_recompute")
    return spike


def bn_fire_bp_workspace_bytes(dtype_code, T, B, C, HW):
    return int(load().snnlif_bn_fire_bp_workspace_bytes(dtype_code, T, B, C, HW))


def bn_fire_bp_into(spatial, weight, bias, ivar, mean, grad_spike, grad_spatial, grad_weight,
                    grad_bias, alpha, thresh, beta, interval, workspace):
    """``snnlif_bn_fire_bp`` on fp32 device tensors; ``workspace`` is a uint8 device tensor."""
    T, B, C, HW = _bn_dims(spatial)
    _require_like(spatial, grad_spike=grad_spike, grad_spatial=grad_spatial)
    _require_per_channel(spatial, C, weight=weight, bias=bias, ivar=ivar, mean=mean,
                         grad_weight=grad_weight, grad_bias=grad_bias)
    _require_workspace(spatial, workspace,
                       bn_fire_bp_workspace_bytes(_torch_dtype_code(spatial), T, B, C, HW),
                       "snnlif_bn_fire_bp")
    _require_dense_gpu(spatial, weight, bias, ivar, mean, grad_spike, grad_spatial, grad_weight,
                       grad_bias, workspace)
    rc = load().snnlif_bn_fire_bp(spatial.data_ptr(), weight.data_ptr(), bias.data_ptr(),
                                  ivar.data_ptr(), mean.data_ptr(), grad_spike.data_ptr(),
                                  grad_spatial.data_ptr(), grad_weight.data_ptr(),
                                  grad_bias.data_ptr(), _torch_dtype_code(spatial), T, B, C, HW,
                                  alpha, thresh, beta, interval, workspace.data_ptr(),
                                  workspace.numel() * workspace.element_size(),
                                  _stream_handle(spatial))
    _check(rc, "snnlif_bn_fire_bp")
    return grad_spatial, grad_weight, grad_bias


def bn_fire_bp_static_into(spatial, weight, bias, ivar, mean, grad_spike, grad_spatial, grad_weight,
                           grad_bias, alpha, thresh, beta, interval):
    """``snnlif_bn_fire_bp_static``: the same backward with its partial sums in the library's fixed
    device array instead of a caller workspace (shapes beyond it raise ``SnnlifError`` with code
    ``ERR_SCRATCH``)."""
    T, B, C, HW = _bn_dims(spatial)
    _require_like(spatial, grad_spike=grad_spike, grad_spatial=grad_spatial)
    _require_per_channel(spatial, C, weight=weight, bias=bias, ivar=ivar, mean=mean,
                         grad_weight=grad_weight, grad_bias=grad_bias)
    _require_dense_gpu(spatial, weight, bias, ivar, mean, grad_spike, grad_spatial, grad_weight,
                       grad_bias)
    rc = load().snnlif_bn_fire_bp_static(spatial.data_ptr(), weight.data_ptr(), bias.data_ptr(),
                                         ivar.data_ptr(), mean.data_ptr(), grad_spike.data_ptr(),
                                         grad_spatial.data_ptr(), grad_weight.data_ptr(),
                                         grad_bias.data_ptr(), _torch_dtype_code(spatial), T, B, C,
                                         HW, alpha, thresh, beta, interval, _stream_handle(spatial))
    _check(rc, "snnlif_bn_fire_bp_static")
    return grad_spatial, grad_weight, grad_bias


def bn_fire_bp_dist1_into(spatial, weight, bias, ivar, mean, grad_spike, mean_gxhat, mean_gxhatx,
                          grad_weight, grad_bias, alpha, thresh, beta, interval, workspace):
    """``snnlif_bn_fire_bp_dist1`` on fp32 device tensors: the half of the backward before the
    all-reduce of a sharded batch."""
    T, B, C, HW = _bn_dims(spatial)
    _require_like(spatial, grad_spike=grad_spike)
    _require_per_channel(spatial, C, weight=weight, bias=bias, ivar=ivar, mean=mean,
                         mean_gxhat=mean_gxhat, mean_gxhatx=mean_gxhatx, grad_weight=grad_weight,
                         grad_bias=grad_bias)
    _require_workspace(spatial, workspace,
                       bn_fire_bp_workspace_bytes(_torch_dtype_code(spatial), T, B, C, HW),
                       "snnlif_bn_fire_bp_dist1")
    _require_dense_gpu(spatial, weight, bias, ivar, mean, grad_spike, mean_gxhat, mean_gxhatx,
                       grad_weight, grad_bias, workspace)
    rc = load().snnlif_bn_fire_bp_dist1(spatial.data_ptr(), weight.data_ptr(), bias.data_ptr(),
                                        ivar.data_ptr(), mean.data_ptr(), grad_spike.data_ptr(),
                                        mean_gxhat.data_ptr(), mean_gxhatx.data_ptr(),
                                        grad_weight.data_ptr(), grad_bias.data_ptr(),
                                        _torch_dtype_code(spatial), T, B, C, HW, alpha, thresh, beta,
                                        interval, workspace.data_ptr(),
                                        workspace.numel() * workspace.element_size(),
                                        _stream_handle(spatial))
    _check(rc, "snnlif_bn_fire_bp_dist1")
    return mean_gxhat, mean_gxhatx, grad_weight, grad_bias


def bn_fire_bp_dist2_into(spatial, weight, bias, ivar, mean, grad_spike, grad_xhat, grad_xhatx,
                          grad_spatial, alpha, thresh, beta, interval):
    """``snnlif_bn_fire_bp_dist2`` on fp32 device tensors: the half after the all-reduce."""
    T, B, C, HW = _bn_dims(spatial)
    _require_like(spatial, grad_spike=grad_spike, grad_spatial=grad_spatial)
    _require_per_channel(spatial, C, weight=weight, bias=bias, ivar=ivar, mean=mean,
                         grad_xhat=grad_xhat, grad_xhatx=grad_xhatx)
    _require_dense_gpu(spatial, weight, bias, ivar, mean, grad_spike, grad_xhat, grad_xhatx,
                       grad_spatial)
    rc = load().snnlif_bn_fire_bp_dist2(spatial.data_ptr(), weight.data_ptr(), bias.data_ptr(),
                                        ivar.data_ptr(), mean.data_ptr(), grad_spike.data_ptr(),
                                        grad_xhat.data_ptr(), grad_xhatx.data_ptr(),
                                        grad_spatial.data_ptr(), _torch_dtype_code(spatial), T, B, C,
                                        HW, alpha, thresh, beta, interval, _stream_handle(spatial))
    _check(rc, "snnlif_bn_fire_bp_dist2")
    return grad_spatial


def bn_fp_into(x_bn, weight, bias, var, mean, ivar, y_bn, eps):
    """``snnlif_bn_fp`` on fp32 / fp64 device tensors; writes ``ivar`` ([C]) and ``y_bn``."""
    T, B, C, HW = _bn_dims(x_bn)
    _require_like(x_bn, y_bn=y_bn)
    _require_per_channel(x_bn, C, weight=weight, bias=bias, var=var, mean=mean, ivar=ivar)
    _require_dense_gpu(x_bn, weight, bias, var, mean, ivar, y_bn)
    rc = load().snnlif_bn_fp(x_bn.data_ptr(), weight.data_ptr(), bias.data_ptr(), var.data_ptr(),
                             mean.data_ptr(), ivar.data_ptr(), y_bn.data_ptr(), _torch_dtype_code(x_bn),
                             T, B, C, HW, eps, _stream_handle(x_bn))
    _check(rc, "snnlif_bn_fp")
    return ivar, y_bn


def bn_bp_workspace_bytes(dtype_code, T, B, C, HW):
    return int(load().snnlif_bn_bp_workspace_bytes(dtype_code, T, B, C, HW))


def bn_bp_into(x_bn, weight, ivar, mean, grad_y, grad_x, grad_weight, grad_bias, workspace):
    """``snnlif_bn_bp``: the plain batch-norm backward; ``workspace`` is a uint8 device tensor."""
    T, B, C, HW = _bn_dims(x_bn)
    _require_like(x_bn, grad_y=grad_y, grad_x=grad_x)
    _require_per_channel(x_bn, C, weight=weight, ivar=ivar, mean=mean, grad_weight=grad_weight,
                         grad_bias=grad_bias)
    _require_workspace(x_bn, workspace, bn_bp_workspace_bytes(_torch_dtype_code(x_bn), T, B, C, HW),
                       "snnlif_bn_bp")
    _require_dense_gpu(x_bn, weight, ivar, mean, grad_y, grad_x, grad_weight, grad_bias, workspace)
    rc = load().snnlif_bn_bp(x_bn.data_ptr(), weight.data_ptr(), ivar.data_ptr(), mean.data_ptr(),
                             grad_y.data_ptr(), grad_x.data_ptr(), grad_weight.data_ptr(),
                             grad_bias.data_ptr(), _torch_dtype_code(x_bn), T, B, C, HW,
                             *_workspace_args(workspace), _stream_handle(x_bn))
    _check(rc, "snnlif_bn_bp")
    return grad_x, grad_weight, grad_bias


def bn_bp_dist1_into(x_bn, weight, ivar, mean, grad_y, mean_gxhat, mean_gxhatx, grad_weight, grad_bias,
                     workspace):
    """``snnlif_bn_bp_dist1``: the half of the plain batch-norm backward before the all-reduce."""
    T, B, C, HW = _bn_dims(x_bn)
    _require_like(x_bn, grad_y=grad_y)
    _require_per_channel(x_bn, C, weight=weight, ivar=ivar, mean=mean, mean_gxhat=mean_gxhat,
                         mean_gxhatx=mean_gxhatx, grad_weight=grad_weight, grad_bias=grad_bias)
    _require_workspace(x_bn, workspace, bn_bp_workspace_bytes(_torch_dtype_code(x_bn), T, B, C, HW),
                       "snnlif_bn_bp_dist1")
    _require_dense_gpu(x_bn, weight, ivar, mean, grad_y, mean_gxhat, mean_gxhatx, grad_weight, grad_bias,
                       workspace)
    rc = load().snnlif_bn_bp_dist1(x_bn.data_ptr(), weight.data_ptr(), ivar.data_ptr(), mean.data_ptr(),
                                   grad_y.data_ptr(), mean_gxhat.data_ptr(), mean_gxhatx.data_ptr(),
                                   grad_weight.data_ptr(), grad_bias.data_ptr(), _torch_dtype_code(x_bn),
                                   T, B, C, HW, *_workspace_args(workspace), _stream_handle(x_bn))
    _check(rc, "snnlif_bn_bp_dist1")
    return mean_gxhat, mean_gxhatx, grad_weight, grad_bias


def bn_bp_dist2_into(x_bn, weight, ivar, mean, grad_y, grad_xhat, grad_xhatx, grad_x):
    """``snnlif_bn_bp_dist2``: the half after the all-reduce."""
    T, B, C, HW = _bn_dims(x_bn)
    _require_like(x_bn, grad_y=grad_y, grad_x=grad_x)
    _require_per_channel(x_bn, C, weight=weight, ivar=ivar, mean=mean, grad_xhat=grad_xhat,
                         grad_xhatx=grad_xhatx)
    _require_dense_gpu(x_bn, weight, ivar, mean, grad_y, grad_xhat, grad_xhatx, grad_x)
    rc = load().snnlif_bn_bp_dist2(x_bn.data_ptr(), weight.data_ptr(), ivar.data_ptr(), mean.data_ptr(),
                                   grad_y.data_ptr(), grad_xhat.data_ptr(), grad_xhatx.data_ptr(),
                                   grad_x.data_ptr(), _torch_dtype_code(x_bn), T, B, C, HW,
                                   _stream_handle(x_bn))
    _check(rc, "snnlif_bn_bp_dist2")
    return grad_x
