"""Locate the native ``snnlib`` extension module.

The reference installs its extension as a top-level module and ``snnlib_func.py`` does
``import snnlib`` (snnlib/example/snnlib_func.py:8).  Here the module is built in-tree as
``snn_gpu_training_bptt_amd/lib/snnlib.so``; it is loaded under the same top-level name and registered
in ``sys.modules`` so that reference-style code doing ``import snnlib`` afterwards gets this build.
There is no fallback: without the built extension the import fails.
"""
import importlib.machinery
import importlib.util
import os
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
EXT_PATH = os.path.join(PKG_DIR, "lib", "snnlib.so")


def load_snnlib():
    mod = sys.modules.get("snnlib")
    if mod is not None:
        if getattr(mod, "__backend__", None) != "hip-gfx950":
            raise ImportError(
                f"a different module named 'snnlib' is already imported from "
                f"{getattr(mod, '__file__', '?')}; it is not the gfx950 build")
        return mod
    if not os.path.exists(EXT_PATH):
        raise ImportError(
            f"{EXT_PATH} is missing: build it with `python -m snn_gpu_training_bptt_amd.build` "
            "(the LIF fire operators have no pure-PyTorch fallback)")
    import torch  # noqa: F401  -- loads libtorch / the HIP runtime the extension links against

    loader = importlib.machinery.ExtensionFileLoader("snnlib", EXT_PATH)
    spec = importlib.util.spec_from_file_location("snnlib", EXT_PATH, loader=loader)
    mod = importlib.util.module_from_spec(spec)
    loader.exec_module(mod)
    sys.modules["snnlib"] = mod
    return mod
