"""Writes tests/golden/golden_f64.npz: outputs of the REFERENCE's own serial k-means instantiated with
F = double (what its --double switch selects, k-means.cpp:341-342) on seeded inputs.

Runs only in the authoring container: it needs oracle/_ref/libref_serial.so, which oracle/Makefile
compiles from /root/reference/experimental/k-means/k-means/headers/serial.hpp where it lies. These
vectors pin the double-precision functions of the CPU oracle (tests/test_oracle.py) on every box.

Inputs are not stored: the seeded float generator reproduces them and widen_points() turns them into
doubles with full mantissas; the fixture keeps an FNV-1a hash of every input.

    python tests/golden/make_golden_f64.py
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

# name, config id, n, iterations, layout, layout_means
CASES = [
    ("cfg1_f64", 1, 8192, 4, AOS, AOS),
    ("cfg1_f64_soa_soa", 1, 8192, 4, SOA, SOA),
    ("cfg1_f64_aos_soa", 1, 4096, 3, AOS, SOA),
    ("cfg2_f64", 2, 8192, 2, AOS, AOS),
    ("cfg3_f64", 3, 16384, 2, SOA, AOS),
    ("cfg4_f64", 4, 2048, 2, AOS, AOS),
    ("cfg5_f64", 5, 32768, 4, AOS, AOS),
]


def inputs(cid, n, layout, lm):
    spec = km.baseline_config(cid)
    data = km.widen_points(km.generate_points(spec, n, layout=layout))
    means0 = km.widen_points(km.first_k_means(spec, lm))
    return spec, data, means0


def main():
    orc.build()
    if orc.ref_lib() is None or not hasattr(orc.ref_lib(), "ref_serial_kmeans_f64"):
        raise SystemExit("oracle/_ref/libref_serial.so could not be built (reference tree missing?)")
    arrays, index = {}, {}
    for name, cid, n, iters, layout, lm in CASES:
        spec, data, means0 = inputs(cid, n, layout, lm)
        means, asg = orc.ref_kmeans_f64(data, means0, spec.dim, spec.k, n, iters, layout, lm)
        asg1 = orc.ref_assign_f64(data, means0, spec.dim, spec.k, n, layout, lm)  # SerialAssignmentAlgorithm, one pass
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
    np.savez_compressed(os.path.join(here, "golden_f64.npz"), **arrays)
    with open(os.path.join(here, "golden_f64_index.json"), "w") as f:
        json.dump(index, f, indent=1, sort_keys=True)


if __name__ == "__main__":
    main()
