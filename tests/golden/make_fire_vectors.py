#!/usr/bin/env python3
"""Writes ``tests/golden/fire_vectors.json``: small input/output vectors for the LIF fire forward
and backward, produced by the pure-Python fp32 tape in ``fp32_tape.py`` (NOT by the reference, whose
own tests hold no stored vectors: snnlib/example/test_fire.py and test_utils.py draw unseeded random
inputs on a GPU and print differences).

Cases: the reference test's fc shape [T=6, B=2, C=8] (snnlib/example/test_utils.py:18) with the
reference's default hyper-parameters (snnlib/example/snnlib_func.py:10-15), the same shape with the
benchmark's threshold 0.5, and a [5, 1, 12] case with a decay that is not a power of two.
Values are stored as fp32 bit patterns (hex) so that nothing is lost in text form.

Run from the repository root:  python tests/golden/make_fire_vectors.py
"""
import json
import os
import random
import struct
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
import fp32_tape  # noqa: E402


def bits(v):
    return struct.unpack("<I", struct.pack("<f", v))[0]


def make_case(name, shape, hyper, seed, mean, std):
    rng = random.Random(seed)
    T = shape[0]
    n = 1
    for d in shape[1:]:
        n *= d
    x = [[fp32_tape.f32(rng.gauss(mean, std)) for _ in range(n)] for _ in range(T)]
    g = [[fp32_tape.f32(rng.gauss(0.0, 1.0)) for _ in range(n)] for _ in range(T)]
    u = [[0.0] * n for _ in range(T)]
    s = [[0.0] * n for _ in range(T)]
    gx = [[0.0] * n for _ in range(T)]
    for i in range(n):
        ui, si, gi = fp32_tape.gold_fire_neuron([x[t][i] for t in range(T)], [g[t][i] for t in range(T)], **hyper)
        for t in range(T):
            u[t][i], s[t][i], gx[t][i] = ui[t], si[t], gi[t]

    def pack(rows):
        return ["".join(f"{bits(v):08x}" for v in row) for row in rows]

    return {"name": name, "shape": list(shape), "hyper": hyper, "seed": seed,
            "x": pack(x), "grad_spike": pack(g), "mem": pack(u), "spike": pack(s), "grad_x": pack(gx)}


def main():
    cases = [
        make_case("fc_shape_reference_defaults", (6, 2, 8),
                  dict(alpha=0.25, thresh=0.25, beta=1.0, interval=0.5), seed=1, mean=0.0, std=1.0),
        make_case("fc_shape_benchmark_threshold", (6, 2, 8),
                  dict(alpha=0.25, thresh=0.5, beta=1.0, interval=0.5), seed=2, mean=0.5, std=1.0),
        make_case("odd_decay", (5, 1, 12),
                  dict(alpha=0.3, thresh=0.4, beta=0.7, interval=0.6), seed=3, mean=0.3, std=0.8),
    ]
    out = os.path.join(HERE, "fire_vectors.json")
    with open(out, "w") as f:
        json.dump({"generator": "tests/golden/make_fire_vectors.py (fp32_tape.py)", "cases": cases}, f, indent=1)
    print("wrote", out)


if __name__ == "__main__":
    main()
