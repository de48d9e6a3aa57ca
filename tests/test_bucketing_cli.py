"""The update micro-benchmark harness (cuda-kmeans_amd/host/bucketing), counterpart of the reference's bucketing-cuda:
option handling, output format, exit codes and the serial algorithm on the CPU; the device algorithms with --verify and
the C ABI entry point behind them (kmx_bucket_sum_f32) on the GPU box."""
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "cuda-kmeans_amd", "host", "bucketing")


@pytest.fixture(scope="module")
def harness(km):
    if not os.path.exists(BIN):
        subprocess.check_call(["make", "-C", os.path.dirname(BIN)])
    return BIN


def run(harness, *args):
    p = subprocess.run([harness] + list(args), capture_output=True, text=True, timeout=600)
    return p.returncode, p.stdout, p.stderr


def test_serial_line_and_saved_sums(harness, tmp_path):
    out_file = str(tmp_path / "sums.txt")
    rc, out, err = run(harness, "--N", "4k", "--k", "16", "--dim", "8", "--iterations", "2", "--seed", "7", "--out", out_file)
    assert rc == 0, out + err
    ms, ns = (float(x) for x in out.split())          # "<ms per batch> <ns per input float>"
    assert ms > 0 and ns > 0
    assert "Selected algorithm: serial" in err and "And we're done here." in err
    sums = np.loadtxt(out_file)
    assert sums.shape == (2 * 16, 8)                  # iterations x k rows of dim sums
    # data uniform in [0,1): every batch's grand total is about N * dim / 2
    for it in range(2):
        total = sums[it * 16:(it + 1) * 16].sum()
        assert abs(total - 4096 * 8 / 2) < 0.05 * 4096 * 8 / 2


def test_layouts_give_the_same_sums(harness, tmp_path):
    results = []
    for layout in ("aos", "soa", "aos32", "soa32"):
        out_file = str(tmp_path / (layout + ".txt"))
        rc, out, err = run(harness, "--N", "1k", "--k", "7", "--dim", "5", "--layout", layout, "--out", out_file)
        assert rc == 0, out + err
        results.append(np.loadtxt(out_file))
    # padded layouts draw their padding from the same random stream, so only equal-sized layouts see equal inputs
    assert results[0].shape == results[1].shape == results[2].shape == results[3].shape == (7, 5)


def test_errors(harness):
    rc, out, err = run(harness, "--dim", "1")
    assert rc == 1 and out.startswith("Invalid arguments:") and "default 20" in out
    rc, out, err = run(harness, "--algorithm", "nope")
    assert rc == 2 and "Error: Unkown algorithm 'nope'." in out
    rc, out, err = run(harness, "--double", "--N", "1k", "--k", "8", "--dim", "3")   # the serial algorithm on doubles
    assert rc == 0 and len(out.split()) == 2
    rc, out, err = run(harness, "--help")
    assert "hip_fake_shm" in out and "hip_atomic_shm2" in out


@pytest.mark.gpu
@pytest.mark.parametrize("algo", ["hip_atomic_shm", "hip_atomic_fine", "hip_atomic_point", "hip_atomic_warp", "cuda_atomic_shm",
                                  "cuda_atomic_shm2"])
@pytest.mark.parametrize("layout", ["aos", "soa", "aos32", "soa32"])
def test_device_algorithms_verify(harness, gpu, algo, layout):
    rc, out, err = run(harness, "--algorithm", algo, "--layout", layout, "--N", "64k", "--k", "512", "--dim", "20",
                       "--iterations", "2", "--verify")
    assert rc == 0 and "Verifying results ... OK" in err, out + err
    assert len(out.split()) == 2


@pytest.mark.gpu
def test_base_and_emulated_atomics(harness, gpu, tmp_path):
    """hip_base has no atomics and adds in point order: its sums have the bits of the serial algorithm's. --emul swaps
    the hardware atomic for a compare-and-swap loop in the point, warp and fine algorithms."""
    common = ["--N", "8k", "--k", "64", "--dim", "12", "--iterations", "2", "--seed", "3"]
    a, b = str(tmp_path / "serial.txt"), str(tmp_path / "base.txt")
    rc, out, err = run(harness, "--algorithm", "serial", "--out", a, *common)
    assert rc == 0
    rc, out, err = run(harness, "--algorithm", "cuda_base", "--verify", "--out", b, *common)
    assert rc == 0 and "Verifying results ... OK" in err, out + err
    assert open(a).read() == open(b).read()
    for algo in ("hip_atomic_point", "hip_atomic_warp", "hip_atomic_fine", "hip_atomic_shm"):
        rc, out, err = run(harness, "--algorithm", algo, "--emul", "--verify", "--privatizedCopies", "2", *common)
        assert rc == 0 and "Verifying results ... OK" in err, algo + out + err


@pytest.mark.gpu
@pytest.mark.parametrize("layout", ["aos", "soa", "aos32"])
def test_fake_algorithms_add_up_to_their_closed_form(harness, gpu, layout):
    """The atomic-throughput probes (kernels.cu:452-531): real atomic additions of the constant 0.1 to bucket
    (i / dim) % k, checked by --verify against 0.1 * #{points congruent to the bucket modulo k} at the micro-benchmark's
    tolerance (5e-5 relative)."""
    for algo, extra in (("hip_fake", []), ("cuda_fake", ["--emul"]), ("hip_fake", ["--privatizedCopies", "3"]),
                        ("cuda_fake_shm", []), ("hip_fake_shm", ["--cudaSharedMemorySize", "4096"]),
                        ("hip_fake_shm", ["--k", "3000", "--dim", "24"])):
        args = ["--algorithm", algo, "--layout", layout, "--N", "64k", "--k", "500", "--dim", "20", "--iterations", "2", "--verify"] + extra
        rc, out, err = run(harness, *args)
        assert rc == 0 and "Verifying results ... OK" in err, " ".join(args) + "\n" + out + err


@pytest.mark.gpu
def test_atomic_shm2_honours_its_lds_copies(harness, gpu):
    """atomic_shm2 (kernels.cu:381-447): as many private copies of the whole k x dim block as the LDS budget holds; not
    even one copy: the reference's error."""
    for extra in ([], ["--cudaSharedMemorySize", "49152"], ["--cudaSharedMemorySize", "40960", "--privatizedCopies", "2"],
                  ["--k", "16", "--dim", "16", "--layout", "soa"], ["--k", "1024", "--dim", "32", "--cudaBlockSize", "1024"]):
        args = ["--algorithm", "cuda_atomic_shm2", "--N", "64k", "--k", "512", "--dim", "20", "--iterations", "2", "--verify"] + extra
        rc, out, err = run(harness, *args)
        assert rc == 0 and "Verifying results ... OK" in err, " ".join(args) + "\n" + out + err
    rc, out, err = run(harness, "--algorithm", "hip_atomic_shm2", "--k", "512", "--dim", "20", "--cudaSharedMemorySize", "16384")
    assert rc == 2 and "Insufficient shared memory size for given parameters." in out


@pytest.mark.gpu
def test_double_precision(harness, gpu):
    for algo in ("hip_atomic_shm", "hip_atomic_fine", "hip_atomic_point"):
        for extra in (["--k", "512", "--dim", "20"], ["--k", "16", "--dim", "16", "--layout", "soa"], ["--k", "2048", "--dim", "32"]):
            rc, out, err = run(harness, "--double", "--algorithm", algo, "--N", "64k", "--iterations", "2", "--verify", *extra)
            assert rc == 0 and "Verifying results ... OK" in err, algo + " ".join(extra) + out + err
    for algo in ("hip_base", "cuda_atomic_shm2", "hip_fake"):             # the baselines and probes of the micro-benchmark are float-only
        rc, out, err = run(harness, "--double", "--algorithm", algo)
        assert rc == 2 and "doubles" in out, algo + out


@pytest.mark.gpu
def test_device_shapes_and_replicas(harness, gpu):
    for extra in (["--k", "16", "--dim", "16", "--N", "256k"], ["--k", "1024", "--dim", "32", "--N", "256k"],
                  ["--k", "4096", "--dim", "4", "--N", "128k"], ["--k", "64", "--dim", "256", "--N", "16k"],
                  ["--k", "512", "--dim", "20", "--privatizedCopies", "4", "--algorithm", "hip_atomic_fine"]):
        args = ["--algorithm", "hip_atomic_shm", "--verify"] + extra
        rc, out, err = run(harness, *args)
        assert rc == 0 and "Verifying results ... OK" in err, " ".join(args) + "\n" + out + err


@pytest.mark.gpu
def test_bucket_sum_entry_point_matches_numpy(km, gpu):
    """kmx_bucket_sum_f32 through ctypes: sums only (no counts, no divide), float64 reference."""
    rng = np.random.default_rng(5)
    for dim, k, n in ((32, 1024, 100000), (16, 16, 50000), (3, 5, 1000)):
        data = rng.random(n * dim, dtype=np.float32)
        idx = rng.integers(0, k, size=n).astype(np.uint32)
        want = np.zeros((k, dim))
        np.add.at(want, idx, data.reshape(n, dim).astype(np.float64))
        d = km.DeviceBuffer(data.nbytes); d.write(data)
        i = km.DeviceBuffer(idx.nbytes); i.write(idx)
        for variant in (km.UPDATE_ATOMIC_SHM, km.UPDATE_ATOMIC_FINE, km.UPDATE_ATOMIC_POINT, km.UPDATE_ATOMIC_WARP, km.UPDATE_ATOMIC_SHM2,
                        km.UPDATE_ATOMIC_FINE | km.UPDATE_EMULATED_ATOMICS, km.UPDATE_ATOMIC_WARP | km.UPDATE_EMULATED_ATOMICS):
            r = km.DeviceBuffer(4 * k * dim); r.zero()
            km.bucket_sum(variant, d, km.AOS, dim, i, r, km.AOS, dim, dim, k, n)
            km.sync()
            got = r.read(np.float32, k * dim).reshape(k, dim)
            r.free()
            assert np.allclose(got, want, rtol=5e-5, atol=1e-4), (dim, k, n, variant)
        # the probes: result[b][d] = 0.1 * #{i < n : i % k == b}, whatever the inputs
        closed = 0.1 * (n // k + (np.arange(k) < n % k))[:, None] * np.ones((1, dim))
        for variant in (km.UPDATE_FAKE, km.UPDATE_FAKE | km.UPDATE_EMULATED_ATOMICS, km.UPDATE_FAKE_SHM):
            r = km.DeviceBuffer(4 * k * dim); r.zero()
            km.bucket_sum(variant, d, km.AOS, dim, i, r, km.AOS, dim, dim, k, n)
            km.sync()
            got = r.read(np.float32, k * dim).reshape(k, dim)
            r.free()
            # (thousands of fp32 additions of the same constant to one word round the same way every time: looser there)
            assert np.allclose(got, closed, rtol=5e-5 if n // k <= 200 else 1e-3, atol=0), (dim, k, n, variant)
        d.free(); i.free()
    # the probes are not an update: the k-means entry point refuses them
    d = km.DeviceBuffer(64); s_ = km.DeviceBuffer(64)
    with pytest.raises(km.KmxError, match="kmx_bucket_sum_f32 only"):
        km.update(km.UPDATE_FAKE, d, km.AOS, 2, d, d, km.AOS, 2, s_, 2, 2, 4)
    d.free(); s_.free()
