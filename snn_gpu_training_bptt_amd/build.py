"""In-tree build of the native pieces (no setuptools, no JIT cache).

Two artefacts land in ``lib/`` next to this file (a directory that holds nothing else, so it can
be put on ``sys.path`` to make ``import snnlib`` work for reference-style code):

* ``libsnnlif_gfx950.so`` -- HIP kernels + C ABI (``csrc/lif_kernels.h`` instantiated by
  ``csrc/lif_f32.hip``, ``lif_f64.hip``, ``lif_bf16.hip``, and ``csrc/lif_bn_kernels.h`` by
  ``lif_bn_f32.hip``, ``lif_bn_f64.hip``; entry points in ``csrc/lif_abi.hip``,
  declared in ``include/snnlib_lif.h``), compiled by hipcc for gfx950 only;
* ``snnlib.so``           -- the Python extension module ``snnlib`` (``csrc/snnlib_ext.cpp``), host
  C++ against PyTorch-ROCm's headers, linked to the library above through ``$ORIGIN``.

This replaces the reference's ``CUDAExtension('snnlib', ..., nvcc -arch=sm_70)`` recipe
(snnlib/setup.py:4-13).  Run ``python -m snn_gpu_training_bptt_amd.build``.
"""
import os
import shutil
import subprocess
import sys
import sysconfig
import tempfile
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_DIR = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
INCLUDE = os.path.join(REPO_DIR, "include")
LIB_DIR = os.path.join(PKG_DIR, "lib")
KERNEL_LIB = os.path.join(LIB_DIR, "libsnnlif_gfx950.so")
EXT_LIB = os.path.join(LIB_DIR, "snnlib.so")

# -ffp-contract=off: products and sums stay separately rounded (bit parity with per-op fp32).
# -packed-fp32-ops off: keep the compiler from forming packed fp32 VALU instructions.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]
KERNEL_SOURCES = ["lif_abi.hip", "lif_f32.hip", "lif_f64.hip", "lif_bf16.hip", "lif_bn_f32.hip",
                  "lif_bn_f64.hip"]


def _run(cmd, verbose):
    if verbose:
        print("+", " ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    out = "\n".join(
        line for line in (proc.stdout + proc.stderr).splitlines()
        # the host pass of hipcc does not know the AMDGPU feature name; the note is harmless
        if "packed-fp32-ops" not in line
    )
    if proc.returncode != 0:
        raise RuntimeError(f"build step failed ({proc.returncode}): {' '.join(cmd)}\n{out}")
    if verbose and out.strip():
        print(out)


def hipcc_path():
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (expected on PATH or at /opt/rocm/bin/hipcc)")


def build_kernels(verbose=False, extra_flags=(), output=KERNEL_LIB):
    """Compile the HIP kernels and their C ABI into ``libsnnlif_gfx950.so``.

    One object per translation unit (compiled in parallel), then one link step.
    """
    hipcc = hipcc_path()
    os.makedirs(os.path.dirname(output), exist_ok=True)
    with tempfile.TemporaryDirectory(prefix="snnlif_build_") as tmp:
        def compile_one(src):
            obj = os.path.join(tmp, os.path.splitext(src)[0] + ".o")
            _run([hipcc, *HIPCC_FLAGS, *extra_flags, f"-I{INCLUDE}", "-c",
                  os.path.join(CSRC, src), "-o", obj], verbose)
            return obj

        with ThreadPoolExecutor(max_workers=len(KERNEL_SOURCES)) as pool:
            objects = list(pool.map(compile_one, KERNEL_SOURCES))
        _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objects, "-o", output], verbose)
    return output


def build_extension(verbose=False):
    """Compile the ``snnlib`` Python module against the installed PyTorch-ROCm."""
    import torch  # only for paths and the C++ ABI flag

    tdir = os.path.dirname(os.path.abspath(torch.__file__))
    tinc = os.path.join(tdir, "include")
    tlib = os.path.join(tdir, "lib")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cxx = os.environ.get("CXX", "g++")
    cmd = [
        cxx, "-O2", "-std=c++17", "-fPIC", "-shared",
        "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
        "-DTORCH_EXTENSION_NAME=snnlib", "-DTORCH_API_INCLUDE_EXTENSION_H",
        f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
        f"-I{INCLUDE}", f"-I{tinc}", f"-I{os.path.join(tinc, 'torch', 'csrc', 'api', 'include')}",
        f"-I{os.path.join(rocm, 'include')}", f"-I{sysconfig.get_paths()['include']}",
        os.path.join(CSRC, "snnlib_ext.cpp"), "-o", EXT_LIB,
        f"-L{tlib}", "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-ltorch_python", "-lc10", "-lc10_hip",
        f"-L{LIB_DIR}", "-l:libsnnlif_gfx950.so",
        "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{tlib}",
    ]
    _run(cmd, verbose)
    return EXT_LIB


def build_all(verbose=False):
    return build_kernels(verbose), build_extension(verbose)


if __name__ == "__main__":
    for path in build_all(verbose="-q" not in sys.argv):
        print("built", path)
