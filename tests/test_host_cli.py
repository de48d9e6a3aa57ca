"""The C++ host harness (cuda-kmeans_amd/host/k-means): option handling, output format, exit codes and the
serial algorithm -- everything that runs without a GPU -- plus, on the GPU box, the device algorithms
with --verify."""
import json
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "cuda-kmeans_amd", "host", "k-means")


@pytest.fixture(scope="module")
def harness(km):
    if not os.path.exists(BIN):
        subprocess.check_call(["make", "-C", os.path.dirname(BIN)])
    return BIN


def run(harness, *args):
    p = subprocess.run([harness] + list(args), capture_output=True, text=True, timeout=600)
    return p.returncode, p.stdout, p.stderr


def test_serial_two_number_line(harness):
    rc, out, err = run(harness, "--N", "4k", "--k", "16", "--dim", "8", "--iterations", "3", "--seed", "7")
    assert rc == 0
    ms, ns = (float(x) for x in out.split())          # "<ms per iteration> <ns per input float>"
    assert ms > 0 and abs(ns - ms * 1e6 / (8 * 4096)) < 1e-3 * ns
    assert "Generating input data (4096 x 8)" in err and "Selected k-means algorithm: serial" in err
    assert "Seed is set to 7" in err and err.rstrip().endswith("And we're done here.")


def test_suffixes_and_defaults(harness):
    rc, out, err = run(harness)                         # reference defaults: N=10240, dim=20, k=128, 1 iteration, serial
    assert rc == 0 and "Generating input data (10240 x 20)" in err
    rc, out, err = run(harness, "--N", "1M", "--k", "2", "--dim", "2")
    assert rc == 0 and "(1048576 x 2)" in err


def test_argument_errors_exit_1(harness):
    for bad in (["--N", "10"], ["--k", "1"], ["--dim", "1"], ["--bogus"], ["--layout", "aos32"], ["--N", "12q"],
                ["--assignmentOnly", "--iterations", "2"], ["--privatizedCopies", "5000"]):
        rc, out, err = run(harness, *bad)
        assert rc == 1 and out.startswith("Invalid arguments:") and "--cudaBlockSize" in out, bad


def test_runtime_errors_exit_2(harness):
    rc, out, err = run(harness, "--algorithm", "nope")
    assert rc == 2 and "Error: Unkown algorithm 'nope'." in out
    rc, out, err = run(harness, "--N", "128", "--k", "1k")
    assert rc == 2


def test_serial_matches_oracle_and_threads_do_not_change_bits(harness, km, orc, tmp_path):
    # benchmark configuration 1, shortened: the harness's serial algorithm against the CPU oracle, through --json
    spec = km.baseline_config(1)
    n, iters = 8192, 3
    data, means0 = km.generate_points(spec, n), km.first_k_means(spec)
    want_m, want_a, want_s = orc.kmeans(data, means0, spec.dim, spec.k, n, iters)
    prefix = str(tmp_path / "out")
    for threads in ("1", "4"):
        rc, out, err = run(harness, "--config", "1", "--N", str(n), "--iterations", str(iters), "--serialThreads", threads,
                           "--json", "--dump", prefix)
        assert rc == 0, out
        rep = json.loads(out)
        assert rep["algorithm"] == "serial" and rep["n"] == n and rep["k"] == 64 and rep["iterations"] == iters
        assert np.array_equal(np.fromfile(prefix + ".assignment.u32", dtype=np.uint32), want_a)
        assert np.array_equal(np.fromfile(prefix + ".means.f32", dtype=np.uint32), want_m.view(np.uint32))
    # other layouts: same assignment, same centroid values in the other memory order
    for layout, lm in ((km.SOA, km.AOS), (km.AOS, km.SOA), (km.SOA, km.SOA)):
        names = {km.AOS: "aos", km.SOA: "soa"}
        rc, out, err = run(harness, "--config", "1", "--N", str(n), "--iterations", str(iters), "--layout", names[layout],
                           "--layoutMeans", names[lm], "--json", "--dump", prefix)
        assert rc == 0
        assert np.array_equal(np.fromfile(prefix + ".assignment.u32", dtype=np.uint32), want_a)
        got = np.fromfile(prefix + ".means.f32", dtype=np.float32)
        got = got.reshape(spec.k, spec.dim) if lm == km.AOS else got.reshape(spec.dim, spec.k).T
        assert np.array_equal(got, want_m.reshape(spec.k, spec.dim))


def test_double_serial_matches_oracle(harness, km, orc, tmp_path):
    """--double: the harness's serial algorithm instantiated with doubles against the oracle's F = double functions
    (the benchmark generator's floats widened exactly)."""
    spec = km.baseline_config(1)
    n, iters = 4096, 3
    data = km.generate_points(spec, n).astype(np.float64)
    means0 = km.first_k_means(spec).astype(np.float64)
    want_m, want_a, _ = orc.kmeans_f64(data, means0, spec.dim, spec.k, n, iters)
    prefix = str(tmp_path / "out")
    rc, out, err = run(harness, "--config", "1", "--N", str(n), "--iterations", str(iters), "--double", "--json", "--dump", prefix)
    assert rc == 0, out
    assert np.array_equal(np.fromfile(prefix + ".assignment.u32", dtype=np.uint32), want_a)
    assert np.array_equal(np.fromfile(prefix + ".means.f64", dtype=np.uint64), want_m.view(np.uint64))


def test_no_device_is_an_error_not_a_fallback(harness, km):
    if km.device_count() > 0:
        pytest.skip("a GPU is visible here")
    rc, out, err = run(harness, "--algorithm", "hip_best")
    assert rc == 2 and "No HIP devices found!" in out
    rc, out, err = run(harness, "--algorithm", "cuda_best", "--assignmentOnly")
    assert rc == 2 and "No HIP devices found!" in out


def test_launch_parameters_that_an_algorithm_ignores_are_named(harness):
    """--regsCache / --itemsPerThread / --cudaBlockSize (k-means.cpp:318-326) shape the launches of hip_base only; given to
    a tuned algorithm they change nothing, and the harness says so on stderr (before it looks for a device)."""
    rc, out, err = run(harness, "--algorithm", "hip_best", "--regsCache", "4", "--itemsPerThread", "2", "--cudaBlockSize", "128")
    for name in ("regsCache", "itemsPerThread", "cudaBlockSize"):
        assert "Warning: --%s is ignored by hip_best" % name in err, err
    rc, out, err = run(harness, "--algorithm", "cuda_cached_regs", "--assignmentOnly", "--regsCache", "4")
    assert "Warning: --regsCache is ignored by hip_mfma" in err, err
    rc, out, err = run(harness, "--algorithm", "hip_base", "--itemsPerThread", "2", "--cudaBlockSize", "128", "--regsCache", "2")
    assert "--itemsPerThread is ignored" not in err and "--cudaBlockSize is ignored" not in err and "--regsCache is ignored by hip_base" in err, err
    rc, out, err = run(harness, "--algorithm", "hip_best")
    assert "Warning" not in err, err
    rc, out, err = run(harness, "--algorithm", "serial", "--regsCache", "4", "--N", "1k", "--k", "8", "--dim", "4")
    assert rc == 0 and "Warning" not in err, err


@pytest.mark.gpu
@pytest.mark.parametrize("config,iters,extra", [("1", "10", []), ("2", "5", ["--N", "64k"]), ("5", "6", ["--N", "256k"]), ("3", "4", ["--N", "128k", "--layout", "soa"])])
def test_serial_order_algorithm_is_bit_identical_to_the_serial_run(harness, gpu, config, iters, extra):
    """hip_best_serial_order: the selector's assignment with the update that adds in the serial order; --verify then finds
    the whole run (several iterations, free-running) equal to the serial algorithm's bit for bit."""
    rc, out, err = run(harness, "--config", config, "--algorithm", "hip_best_serial_order", "--iterations", iters, "--verify",
                       "--serialThreads", "8", "--json", *extra)
    assert rc == 0, out + err
    rep = json.loads(out)
    assert rep["bit_identical"] is True and rep["assignment_mismatches"] == 0 and rep["centroid_error"] == 0.0, rep
    assert "bit-identical to the serial run" in err


@pytest.mark.gpu
@pytest.mark.parametrize("algo", ["hip_best", "hip_mfma", "hip_mfma_bf16", "hip_base", "hip_base_shm", "cuda_best", "hip_fused",
                                  "cuda_fused_regs"])
def test_device_algorithms_verify(harness, gpu, algo):
    rc, out, err = run(harness, "--config", "1", "--algorithm", algo, "--iterations", "1", "--verify", "--serialThreads", "8", "--json")
    assert rc == 0, out + err
    rep = json.loads(out)
    assert rep["verify_errors"] == 0 and rep["assignment_mismatches"] == 0 and rep["centroid_error"] < 1e-4
    assert "Verifying results ... OK" in err


@pytest.mark.gpu
def test_device_assignment_only_and_reference_dataset(harness, gpu):
    for algo in ("hip_best", "hip_mfma", "hip_mfma_bf16", "hip_base", "hip_lds_fma", "cuda_cached_regs", "cuda_cached_fixed"):
        rc, out, err = run(harness, "--assignmentOnly", "--algorithm", algo, "--N", "64k", "--k", "256", "--dim", "16", "--verify", "--serialThreads", "8")
        assert rc == 0 and "Verifying results ... OK" in err, err
        assert len(out.split()) == 2
    # the reference's defaults on the device, both layouts
    for layout in ("aos", "soa"):
        rc, out, err = run(harness, "--algorithm", "hip_best", "--iterations", "1", "--layout", layout, "--verify")
        assert rc == 0 and "Verifying results ... OK" in err, err
    rc, out, err = run(harness, "--algorithm", "hip_lds_fma", "--assignmentOnly", "--dim", "100")
    assert rc == 2 and "not supported" in out


@pytest.mark.gpu
def test_device_algorithms_verify_in_double(harness, gpu):
    for algo in ("hip_best", "hip_base", "hip_base_shm", "hip_fused", "cuda_best"):
        rc, out, err = run(harness, "--config", "1", "--double", "--algorithm", algo, "--iterations", "1", "--verify",
                           "--serialThreads", "8", "--json")
        assert rc == 0, out + err
        rep = json.loads(out)
        assert rep["verify_errors"] == 0 and rep["assignment_mismatches"] == 0 and rep["centroid_error"] < 1e-10
    rc, out, err = run(harness, "--double", "--assignmentOnly", "--algorithm", "hip_best", "--N", "64k", "--k", "256", "--dim", "16",
                       "--verify", "--serialThreads", "8")
    assert rc == 0 and "Verifying results ... OK" in err, err
    # the matrix-core sweeps rank float copies and leave the rest to the double arithmetic
    for algo in ("hip_mfma", "hip_mfma_bf16"):
        rc, out, err = run(harness, "--config", "2", "--N", "64k", "--double", "--algorithm", algo, "--iterations", "1", "--verify",
                           "--serialThreads", "8", "--json")
        assert rc == 0 and json.loads(out)["assignment_mismatches"] == 0, out + err


@pytest.mark.gpu
def test_recorded_iterations_verify(harness, gpu):
    """--graph: the first iteration call by call, then a recorded pair of iterations replayed; one iteration cannot
    diverge from the serial run, several are checked through the harness's own loose centroid rule."""
    rc, out, err = run(harness, "--config", "1", "--algorithm", "hip_best", "--iterations", "5", "--graph")
    assert rc == 0 and len(out.split()) == 2, out + err
    rc, out, err = run(harness, "--algorithm", "hip_best", "--iterations", "4", "--graph", "--verify", "--N", "64k", "--k", "256", "--dim", "16")
    assert rc == 0 and "Verifying results ..." in err, out + err
