"""Check the instruction schedule the compiler gave every kernel of the library.

    python -m snn_gpu_training_bptt_amd.schedule_check [-v]

The kernels are bound by HBM bandwidth and rely on one property of their machine code: a wavefront
issues the row requests of a window back to back and only then starts to wait.  hipcc usually keeps
that order, but for some instantiations (seen for the 40-step backward window in fp32, several
fp64 and one-neuron-per-lane bf16 windows, every window with a head before its order was pinned) it
falls back to one request at a time, each followed by ``s_waitcnt vmcnt(0)`` -- a third of the
bandwidth, with no other symptom: results stay correct and no test fails.  This tool compiles every
kernel translation unit to gfx950 assembly (device side only, nothing is linked or run, no GPU needed)
and reports, per kernel, the global loads that are immediately followed by a full wait, scratch
(spill) memory and the register count.  It exits non-zero when a kernel outside the list of known
exceptions below has more than ``SERIAL_LIMIT`` such loads or uses scratch memory; run it after
changing the kernels or the compiler.
"""
import argparse
import os
import re
import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor

from . import build

# translation units that hold kernels (lif_abi.hip holds entry points only)
UNITS = [u for u in build.KERNEL_SOURCES if u != "lif_abi.hip"]
SERIAL_LIMIT = 4

# Instantiations known to be scheduled one request at a time, with the reason they are left so.
KNOWN = [
    (r"lif_forward_kernelId.*Lb0EEEv", "fp64 forward behind per-row tests (lengths without a straight-line "
                                      "instantiation, and the kept form): 8-byte loads are serialised behind the tests"),
    (r"lif_backward_segmented_kernelI(d|NS_6bf16_tE)", "segmented backward in fp64 / bf16: the partial last segment"),
    (r"lif_bn_backward_input_kernelIdLi(28|32)E", "fp64 batch-norm + fire input sweep of 28 / 32 steps"),
]


def compile_unit(unit, out_dir):
    out = os.path.join(out_dir, os.path.splitext(unit)[0] + ".s")
    cmd = [build.hipcc_path(), *build.HIPCC_FLAGS, f"-I{build.INCLUDE}", "-S", "--cuda-device-only",
           os.path.join(build.CSRC, unit), "-o", out]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"{' '.join(cmd)}\n{proc.stderr}")
    return out


def scan(path):
    """[(kernel, loads, stores, loads followed by a full wait, scratch bytes, vgprs)] of one .s file."""
    rows, name, seq = [], None, []
    meta = {}
    for line in open(path):
        m = re.match(r"^(_Z\w+):", line)
        if m:
            name, seq = m.group(1), []
            continue
        m = re.match(r"\s*\.set (_Z\w+)\.(num_vgpr|private_seg_size), (\d+)", line)
        if m:
            meta.setdefault(m.group(1), {})[m.group(2)] = int(m.group(3))
            continue
        if name is None:
            continue
        if "global_load" in line:
            seq.append("L")
        elif "global_store" in line:
            seq.append("S")
        elif "s_waitcnt" in line and "vmcnt" in line:
            seq.append("w" + re.search(r"vmcnt\((\d+)\)", line).group(1))
        elif "s_endpgm" in line:
            serial = sum(1 for a, b in zip(seq, seq[1:]) if a == "L" and b == "w0")
            rows.append([name, seq.count("L"), seq.count("S"), serial])
            name = None
    return [r + [meta.get(r[0], {}).get("private_seg_size", 0), meta.get(r[0], {}).get("num_vgpr", 0)]
            for r in rows]


def main():
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("-v", "--verbose", action="store_true", help="list every kernel, not only the flagged ones")
    args = ap.parse_args()
    with tempfile.TemporaryDirectory(prefix="snnlif_sched_") as tmp:
        with ThreadPoolExecutor(max_workers=len(UNITS)) as pool:
            files = list(pool.map(lambda u: compile_unit(u, tmp), UNITS))
        rows = [r for f in files for r in scan(f)]
    bad = 0
    for name, loads, stores, serial, scratch, vgprs in rows:
        flagged = serial > SERIAL_LIMIT or scratch > 0
        reason = next((why for pat, why in KNOWN if re.search(pat, name)), None)
        if flagged or args.verbose:
            tag = "ok      " if not flagged else ("known   " if reason and scratch == 0 else "SERIAL  ")
            print(f"{tag}{name[:120]:120s} loads {loads:4d} stores {stores:4d} load->full wait {serial:4d} "
                  f"scratch {scratch:4d} vgprs {vgprs:4d}" + (f"   [{reason}]" if flagged and reason else ""))
        if flagged and not (reason and scratch == 0):
            bad += 1
    print(f"{len(rows)} kernels in {len(UNITS)} translation units, {bad} with an unexpected schedule or scratch memory")
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(main())
