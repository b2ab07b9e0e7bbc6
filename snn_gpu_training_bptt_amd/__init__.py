"""LIF "fire" forward / backward operators of snnlib as hand-written HIP kernels for MI355X.

Layout
    csrc/lif_*.hip, lif_kernels.h   kernels + C ABI            -> lib/libsnnlif_gfx950.so  (include/snnlib_lif.h)
    csrc/snnlib_ext.cpp    PyTorch-ROCm binding       -> lib/snnlib.so            (module ``snnlib``)
    lif_cabi.py            ctypes view of the C ABI
    snnlib_func.py         ``FireFunc`` / ``fire_func`` / hyper-parameters
    snnlib_op.py           ``Fire`` layer module
    build.py               in-tree build of both shared objects

Importing the package does not touch the GPU and does not load the native code; importing
``snnlib_func`` / ``snnlib_op`` loads ``snnlib.so`` and fails loudly if it has not been built.
"""

__all__ = ["build", "lif_cabi", "snnlib_func", "snnlib_op"]
