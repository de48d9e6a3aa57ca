"""Writes tests/golden/golden.npz: outputs of the REFERENCE's own serial k-means on seeded inputs.

Runs only in the authoring container: it needs oracle/_ref/libref_serial.so, which oracle/Makefile
compiles from /root/reference/experimental/k-means/k-means/headers/serial.hpp where it lies. The
reference ships no golden vectors of its own, so these are the vectors that pin the CPU oracle
(tests/test_oracle.py compares oracle/liboracle.so with them bit for bit on every box).

Inputs are not stored: the seeded generator (cuda-kmeans_amd/host/datagen.c) reproduces them; the
fixture keeps an FNV-1a hash of every input so that generator drift is caught as such.

    python tests/golden/make_golden.py
"""
import importlib
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
km = importlib.import_module("cuda-kmeans_amd")
from oracle import binding as orc  # noqa: E402

AOS, SOA = 0, 1

# name, config id, n (None = full), iterations (None = config's), layout, layout_means
CASES = [
    ("cfg1_full", 1, None, None, AOS, AOS),
    ("cfg1_soa_soa", 1, 8192, 4, SOA, SOA),
    ("cfg1_aos_soa", 1, 8192, 4, AOS, SOA),
    ("cfg1_soa_aos", 1, 8192, 4, SOA, AOS),
    ("cfg2_small", 2, 32768, 4, AOS, AOS),
    ("cfg3_small", 3, 65536, 3, AOS, AOS),
    ("cfg4_small", 4, 8192, 2, AOS, AOS),
    ("cfg5_small", 5, 65536, 5, AOS, AOS),
]


def main():
    if orc.ref_lib() is None:
        orc.build()
    if orc.ref_lib() is None:
        raise SystemExit("oracle/_ref/libref_serial.so could not be built (reference tree missing?)")
    arrays, index = {}, {}
    for name, cid, n, iters, layout, lm in CASES:
        spec = km.baseline_config(cid)
        n = int(spec.n) if n is None else n
        iters = int(spec.iterations) if iters is None else iters
        data = km.generate_points(spec, n, layout=layout)
        means0 = km.first_k_means(spec, lm)
        means, asg = orc.ref_kmeans(data, means0, spec.dim, spec.k, n, iters, layout, lm)
        asg1 = orc.ref_assign(data, means0, spec.dim, spec.k, n, layout, lm)  # SerialAssignmentAlgorithm, one pass
        dt = np.uint8 if spec.k <= 256 else np.uint16
        arrays[name + "_assignment"] = asg.astype(dt)
        arrays[name + "_assignment_first_pass"] = asg1.astype(dt)
        arrays[name + "_counts"] = np.bincount(asg, minlength=spec.k).astype(np.uint32)
        arrays[name + "_means_head"] = means[:256].copy()
        index[name] = {
            "config": cid, "n": n, "dim": int(spec.dim), "k": int(spec.k), "iterations": iters,
            "layout": layout, "layout_means": lm,
            "data_fnv1a64": "%016x" % km.fnv1a64(data),
            "means_fnv1a64": "%016x" % km.fnv1a64(means),
        }
        print(name, index[name], flush=True)
    here = os.path.dirname(os.path.abspath(__file__))
    np.savez_compressed(os.path.join(here, "golden.npz"), **arrays)
    with open(os.path.join(here, "golden_index.json"), "w") as f:
        json.dump(index, f, indent=1, sort_keys=True)


if __name__ == "__main__":
    main()
