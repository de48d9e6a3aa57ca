"""Parity of the double-precision HIP path (kmx_assign_f64 / kmx_update_f64 / kmx_fused_f64, the counterpart of
the reference's --double instantiation) with the CPU oracle's F = double functions, through the C ABI (-m gpu).

Bar: assignment and counts bit-exact (KMX_ASSIGN_BASE evaluates the serial arithmetic itself for every pair; the ranking
sweeps behind the other variants certify their result or hand the point to that arithmetic);
centroids within 1e-12 relative to the rms coordinate (the sums are accumulated by atomics in another order).
"""
import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
AOS, SOA = 0, 1
CENTROID_RTOL = 1e-12


def F64_VARIANTS(km):
    """BASE: serial arithmetic for every pair; LDS_FMA: fp64 FMA ranking; MFMA, MFMA_BF16X3, BEST: the float sweeps rank
    rounded copies. All hand what they cannot certify to the serial arithmetic on the doubles."""
    return (km.ASSIGN_BASE, km.ASSIGN_LDS_FMA, km.ASSIGN_MFMA, km.ASSIGN_MFMA_BF16X3, km.ASSIGN_BEST)


def rel_err(got, want):
    scale = float(np.sqrt(np.mean(want ** 2)))
    return float(np.abs(got - want).max() / max(scale, 1e-300))


def gpu_assign(km, variant, data, means, dim, k, n, layout=AOS, layout_means=AOS):
    alg = km.HipAssignmentAlgorithm(variant, None, layout, layout_means, dtype=np.float64)
    alg.initialize(dim, k, n, data, means)
    alg.run()
    out = alg.getAssignment()
    alg.cleanup()
    return out


def gpu_update(km, variant, data, assignment, dim, k, n, layout=AOS, layout_means=AOS):
    d = km.DeviceBuffer(8 * max(data.size, 1)); d.write(data)
    a = km.DeviceBuffer(4 * max(n, 1)); a.write(assignment)
    msize = km.layout_size(layout_means, k, dim)
    m = km.DeviceBuffer(8 * msize); m.zero()
    s = km.DeviceBuffer(4 * k); s.zero()
    km.update(variant, d, layout, km.layout_stride(layout, n, dim), a, m, layout_means,
              km.layout_stride(layout_means, k, dim), s, dim, k, n, dtype=np.float64)
    km.sync()
    means, sizes = m.read(np.float64, msize), s.read(np.uint32, k)
    for b in (d, a, m, s):
        b.free()
    return means, sizes


@pytest.fixture(scope="module")
def golden():
    with open(os.path.join(HERE, "golden", "golden_f64_index.json")) as f:
        index = json.load(f)
    return index, np.load(os.path.join(HERE, "golden", "golden_f64.npz"))


@pytest.mark.parametrize("name", ["cfg1_f64", "cfg1_f64_soa_soa", "cfg1_f64_aos_soa", "cfg2_f64", "cfg3_f64", "cfg4_f64",
                                  "cfg5_f64"])
def test_first_pass_equals_reference_golden(km, gpu, golden, name):
    """One assignment pass from the initial centroids against the REFERENCE's own double-precision output."""
    index, arrays = golden
    c = index[name]
    spec = km.baseline_config(c["config"])
    data = km.widen_points(km.generate_points(spec, c["n"], layout=c["layout"]))
    means0 = km.widen_points(km.first_k_means(spec, c["layout_means"]))
    want = arrays[name + "_assignment_first_pass"].astype(np.uint32)
    for v in F64_VARIANTS(km):
        got = gpu_assign(km, v, data, means0, c["dim"], c["k"], c["n"], c["layout"], c["layout_means"])
        assert np.array_equal(got, want), "variant %d: %d mismatches" % (v, int((got != want).sum()))


SHAPES = [(20, 128, 10240), (3, 5, 257), (7, 33, 1000), (2, 2, 128), (16, 16, 5000), (32, 1000, 4099), (64, 96, 2048),
          (100, 40, 1500), (256, 300, 700), (1, 7, 300), (5, 4100, 777), (9, 8, 64), (33, 9, 513), (4, 1, 100), (3, 5, 1), (40, 1, 1), (300, 260, 300), (400, 256, 200),
          (4, 4096, 3000), (3, 300, 70001), (2, 700, 5000), (12, 1024, 9000), (8, 256, 20000)]


@pytest.mark.parametrize("dim,k,n", SHAPES)
@pytest.mark.parametrize("layout,layout_means", [(AOS, AOS), (SOA, SOA), (AOS, SOA), (SOA, AOS)])
def test_assignment_is_bit_exact(km, orc, gpu, dim, k, n, layout, layout_means):
    rng = np.random.default_rng(dim * 7919 + k)
    data = rng.normal(size=n * dim) * 3.0
    means = rng.normal(size=k * dim) * 3.0
    want = orc.assign_f64(data, means, dim, k, n, layout, layout_means, threads=0)
    for v in F64_VARIANTS(km):
        if dim > 256 and v in (km.ASSIGN_MFMA, km.ASSIGN_MFMA_BF16X3):
            with pytest.raises(km.KmxError):   # the matrix-core sweeps take rows of up to 256 dimensions, for either element type
                gpu_assign(km, v, data, means, dim, k, n, layout, layout_means)
            continue
        got = gpu_assign(km, v, data, means, dim, k, n, layout, layout_means)
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, "variant %d: %d mismatches, first at %s" % (v, bad.size, bad[:5])


@pytest.mark.parametrize("dim,k,n", [(32, 1024, 100000), (64, 512, 50000), (16, 256, 100000), (8, 100, 100000), (3, 300, 100000), (100, 300, 20000)])
@pytest.mark.parametrize("offset", [0.0, 1000.0, 1.0e6])
def test_data_far_from_the_origin(km, orc, gpu, dim, k, n, offset):
    """The float sweeps rank float copies of x - m and c - m (m: the mean of the first points, subtracted in double), and the
    exact pass takes their thresholds back to the frame of the data: the oracle's assignment wherever the data lie, and
    no more points left to the exact pass far from the origin than around it."""
    rng = np.random.default_rng(dim * 5 + k)
    centres = rng.uniform(-10, 10, (k, dim))
    base = centres[rng.integers(0, k, n)] + rng.normal(size=(n, dim)) + offset
    means = base[:k].copy()
    want = orc.assign_f64(base.ravel(), means.ravel(), dim, k, n, AOS, AOS, threads=0)
    for v in (km.ASSIGN_BEST, km.ASSIGN_MFMA, km.ASSIGN_MFMA_BF16X3):
        for layout in (AOS, SOA):
            d = base if layout == AOS else np.ascontiguousarray(base.T)
            got = gpu_assign(km, v, d.ravel(), means.ravel(), dim, k, n, layout, AOS)
            bad = np.nonzero(got != want)[0]
            assert bad.size == 0, "variant %d, layout %d: %d mismatches, first at %s" % (v, layout, bad.size, bad[:5])
            assert km.last_rechecked() < n // 10, "variant %d: %d of %d points left to the exact pass" % (v, km.last_rechecked(), n)


@pytest.mark.parametrize("dim,k,n", [(32, 2048, 66000), (48, 1100, 65536), (64, 1000, 65600)])
@pytest.mark.parametrize("layout,layout_means", [(AOS, AOS), (SOA, SOA)])
def test_centroids_swept_in_slices(km, orc, gpu, dim, k, n, layout, layout_means):
    """Doubles, ranked by the float sweeps: from 65536 points on, rows of 17 to 64 dimensions whose centroids do not fit the
    LDS are swept once per slice of centroids (the float copy of the points is read once per slice)."""
    rng = np.random.default_rng(dim * 13 + k)
    centres = rng.uniform(-10, 10, (40, dim))
    base = centres[rng.integers(0, 40, n)] + rng.normal(size=(n, dim))
    means = base[rng.permutation(n)[:k]].copy()
    d = base if layout == AOS else np.ascontiguousarray(base.T)
    m = means if layout_means == AOS else np.ascontiguousarray(means.T)
    want = orc.assign_f64(d.ravel(), m.ravel(), dim, k, n, layout, layout_means, threads=0)
    for v in (km.ASSIGN_MFMA_BF16X3, km.ASSIGN_BEST):
        got = gpu_assign(km, v, d.ravel(), m.ravel(), dim, k, n, layout, layout_means)
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, "variant %d: %d mismatches, first at %s" % (v, bad.size, bad[:5])


@pytest.mark.parametrize("dim,k,n", [(8, 64, 4096), (32, 256, 3000), (40, 70, 1000), (4, 300, 5000), (2, 600, 4000), (8, 512, 3000)])
def test_hard_inputs(km, orc, gpu, dim, k, n):
    """Exact ties, duplicated centroids, coincident points, NaN / inf / huge / tiny values, float-invisible gaps."""
    rng = np.random.default_rng(99 + dim)
    base = rng.normal(size=(n, dim))
    means = rng.normal(size=(k, dim))
    cases = {}
    m = means.copy(); m[k // 2] = m[3]; m[k - 1] = m[3]; m[7] = m[5]
    d = base.copy(); d[: k] = m
    d[k: 2 * k] = (m + m[::-1]) / 2.0
    cases["duplicates_and_midpoints"] = (d, m)
    m = means.copy(); m[9] = m[2] * (1.0 + 2.0 ** -45)       # differs from centroid 2 far below float resolution
    d = base.copy(); d[:50] = m[2] * 1.5
    cases["gap_below_float_resolution"] = (d, m)
    cases["all_points_identical"] = (np.repeat(base[:1], n, 0), means)
    cases["all_centroids_identical"] = (base, np.repeat(means[:1], k, 0))
    d = base.copy(); d[5, 0] = np.nan; d[9, dim - 1] = np.inf; d[11, 0] = -np.inf
    cases["nan_inf_points"] = (d, means)
    m = means.copy(); m[4, 1] = np.nan
    cases["nan_centroid"] = (base, m)
    m = means.copy(); m[0, 0] = np.nan
    cases["nan_centroid_zero"] = (base, m)
    cases["huge"] = (base * 1e160, means * 1e160)          # squares overflow to inf
    cases["tiny"] = (base * 1e-170, means * 1e-170)        # squares underflow
    cases["grid_ties"] = (np.round(base * 2) / 2, np.round(means * 2) / 2)
    for name, (d, m) in cases.items():
        d = np.ascontiguousarray(d).ravel()
        m = np.ascontiguousarray(m).ravel()
        want = orc.assign_f64(d, m, dim, k, n, threads=0)
        for v in F64_VARIANTS(km):
            got = gpu_assign(km, v, d, m, dim, k, n)
            bad = np.nonzero(got != want)[0]
            assert bad.size == 0, "%s, variant %d: %d mismatches, first at %s (gpu %s, oracle %s)" % (
                name, v, bad.size, bad[:5], got[bad[:5]], want[bad[:5]])


UPDATE_SHAPES = [(8, 64, 65536), (20, 128, 10240), (3, 5, 257), (32, 1024, 50000), (4, 4096, 100000), (16, 16, 300000),
                 (256, 1024, 4096), (33, 7, 1000), (300, 260, 3000), (5000, 3, 64), (128, 700, 30000), (130, 33, 5000), (1100, 40, 2500),
                 (17, 300, 40000), (64, 1000, 70001), (100, 90, 33000), (127, 513, 9000), (40, 2000, 20000)]


@pytest.mark.parametrize("dim,k,n", UPDATE_SHAPES)
@pytest.mark.parametrize("layout,layout_means", [(AOS, AOS), (SOA, SOA), (AOS, SOA), (SOA, AOS)])
def test_update_matches_oracle(km, orc, gpu, dim, k, n, layout, layout_means):
    rng = np.random.default_rng(dim + k + n)
    data = rng.normal(size=n * dim) * 2.0 + 1.0
    asg = rng.integers(0, k, size=n, dtype=np.uint32)
    asg[asg == k // 2] = 0                                 # an empty cluster (k > 1)
    want_m, want_s = orc.update_f64(data, asg, dim, k, n, layout, layout_means, threads=0)
    for v in (km.UPDATE_ATOMIC_POINT, km.UPDATE_ATOMIC_FINE, km.UPDATE_ATOMIC_SHM):
        got_m, got_s = gpu_update(km, v, data, asg, dim, k, n, layout, layout_means)
        assert np.array_equal(got_s, want_s), v
        assert rel_err(got_m, want_m) < CENTROID_RTOL, (v, rel_err(got_m, want_m))
        if k > 1:
            c = k // 2
            empty = got_m.reshape(k, dim)[c] if layout_means == AOS else got_m.reshape(dim, k)[:, c]
            assert np.array_equal(empty, np.zeros(dim)), "an empty cluster stays at the origin"


@pytest.mark.parametrize("cid,n,iters", [(1, 65536, 6), (2, 32768, 3), (5, 200000, 4), (4, 4096, 2)])
def test_every_iteration_matches_oracle(km, orc, gpu, cid, n, iters):
    """Teacher-forced: every iteration's assignment against the oracle's on the centroids the GPU used (exact), every
    update against the oracle's on that assignment (tolerance); then the free-running result."""
    spec = km.baseline_config(cid)
    data = km.widen_points(km.generate_points(spec, n))
    means0 = km.widen_points(km.first_k_means(spec))
    alg = km.HipKMeansAlgorithm(dtype=np.float64)
    alg.initialize(spec.dim, spec.k, n, iters, data, means0)
    prev = means0
    for it in range(iters):
        nxt = alg.iteration()
        km.sync()
        got_a = alg.cu_assignment[nxt].read(np.uint32, n)
        want_a = orc.assign_f64(data, prev, spec.dim, spec.k, n, threads=0)
        assert np.array_equal(got_a, want_a), "iteration %d: %d mismatches" % (it, int((got_a != want_a).sum()))
        alg.update_step(nxt)
        km.sync()
        got_m, got_s = alg.getMeans(), alg.getClusterSizes()
        want_m, want_s = orc.update_f64(data, want_a, spec.dim, spec.k, n, threads=0)
        assert np.array_equal(got_s, want_s)
        assert rel_err(got_m, want_m) < CENTROID_RTOL
        prev = got_m
    alg.cleanup()


@pytest.mark.parametrize("dim,k,n", [(8, 64, 65536), (3, 5, 257), (32, 1024, 50000), (4, 4096, 100000), (16, 16, 300000), (256, 1024, 4096),
                                     (2, 70000, 4096), (8, 64, 0)])
@pytest.mark.parametrize("layout,layout_means", [(AOS, AOS), (SOA, SOA), (AOS, SOA), (SOA, AOS)])
def test_serial_order_update_has_the_bits_of_the_serial_loop(km, orc, gpu, dim, k, n, layout, layout_means):
    """KMX_UPDATE_SERIAL_ORDER on doubles against the oracle's update, bit for bit."""
    rng = np.random.default_rng(dim * 7 + k + n)
    data = rng.normal(size=n * dim) * 2.0 + 1.0
    asg = rng.integers(0, k, size=n, dtype=np.uint32)
    if k > 2 and n:
        asg[asg == 1] = 0
        asg[rng.random(n) < 0.3] = k - 1
    want_m, want_s = orc.update_f64(data, asg, dim, k, n, layout, layout_means, threads=0)
    got_m, got_s = gpu_update(km, km.UPDATE_SERIAL_ORDER, data, asg, dim, k, n, layout, layout_means)
    assert np.array_equal(got_s, want_s)
    assert np.array_equal(got_m.view(np.uint64), want_m.view(np.uint64))


def test_whole_runs_equal_the_reference_golden(km, gpu, golden):
    """Free-running double-precision runs with the serial-order update against what the REFERENCE's
    SerialKMeansAlgorithm<double> left (tests/golden/make_golden_f64.py): assignment, counts, centroids bit for bit."""
    index, arrays = golden
    for name, c in sorted(index.items()):
        spec = km.baseline_config(c["config"])
        data = km.widen_points(km.generate_points(spec, c["n"], layout=c["layout"]))
        means0 = km.widen_points(km.first_k_means(spec, c["layout_means"]))
        alg = km.HipKMeansAlgorithm(km.ASSIGN_BEST, km.UPDATE_SERIAL_ORDER, layout=c["layout"], layout_means=c["layout_means"], dtype=np.float64)
        alg.initialize(c["dim"], c["k"], c["n"], c["iterations"], data, means0)
        alg.run()
        means, asg, sizes = alg.getMeans(), alg.getAssignment(), alg.getClusterSizes()
        alg.cleanup()
        assert np.array_equal(asg, arrays[name + "_assignment"].astype(np.uint32)), name
        assert np.array_equal(sizes, arrays[name + "_counts"]), name
        head = arrays[name + "_means_head"]
        assert np.array_equal(means[:head.size].view(np.uint64), head.view(np.uint64)), name
        assert "%016x" % km.fnv1a64(means) == c["means_fnv1a64"], name


def test_prepared_points_do_not_outlive_their_buffer(km, orc, gpu):
    """The float copy made by kmx_prepare_points_f64 is dropped when the announced buffer is rewritten through the library
    (kmx_h2d, kmx_d2d, kmx_fill_zero_u32) or released (kmx_free): a later call on the same address, which hipMalloc readily
    hands out again, must see the new contents."""
    dim, k, n = 16, 128, 20000
    rng = np.random.default_rng(5)
    first = rng.normal(size=n * dim) * 3
    other = rng.normal(size=n * dim) * 3 + 1
    means = first.reshape(n, dim)[:k].copy().ravel()
    lib = km.hip_lib()
    m = km.DeviceBuffer(8 * k * dim); m.write(means)
    a = km.DeviceBuffer(4 * n)
    spare = km.DeviceBuffer(8 * n * dim); spare.write(other)

    def run(buf):
        km.assign(km.ASSIGN_BEST, buf, km.AOS, dim, m, km.AOS, dim, a, dim, k, n, dtype=np.float64)
        km.sync()
        return a.read(np.uint32, n)

    want_first = orc.assign_f64(first, means, dim, k, n, threads=0)
    want_other = orc.assign_f64(other, means, dim, k, n, threads=0)
    want_zero = orc.assign_f64(np.zeros(n * dim), means, dim, k, n, threads=0)
    d = km.DeviceBuffer(8 * n * dim); d.write(first)
    km.check(lib.kmx_prepare_points_f64(d.ptr, km.AOS, dim, dim, n))
    assert np.array_equal(run(d), want_first)
    d.write(other)                                       # rewritten in place through kmx_h2d, no kmx_forget_points_f64
    assert np.array_equal(run(d), want_other)
    km.check(lib.kmx_prepare_points_f64(d.ptr, km.AOS, dim, dim, n))
    km.check(lib.kmx_d2d(d.ptr, spare.ptr, 8 * n * dim)) # the same contents again: harmless, but the copy is dropped
    d.zero()                                             # kmx_fill_zero_u32
    assert np.array_equal(run(d), want_zero)
    d.write(first)
    km.check(lib.kmx_prepare_points_f64(d.ptr, km.AOS, dim, dim, n))
    d.free()                                             # kmx_free: the announcement goes with the buffer
    d = km.DeviceBuffer(8 * n * dim)                     # very likely the same address
    d.write(other)
    assert np.array_equal(run(d), want_other)
    for b in (d, m, a, spare):
        b.free()


def test_fused_call_and_argument_errors(km, orc, gpu):
    spec = km.baseline_config(1)
    n = 20000
    data = km.widen_points(km.generate_points(spec, n))
    means0 = km.widen_points(km.first_k_means(spec))
    alg = km.HipFusedKMeansAlgorithm(dtype=np.float64)
    alg.initialize(spec.dim, spec.k, n, 1, data, means0)
    alg.run()
    want_a = orc.assign_f64(data, means0, spec.dim, spec.k, n, threads=0)
    want_m, want_s = orc.update_f64(data, want_a, spec.dim, spec.k, n, threads=0)
    assert np.array_equal(alg.getClusterSizes(), want_s)
    assert rel_err(alg.getMeans(), want_m) < CENTROID_RTOL
    alg.cleanup()
    with pytest.raises(km.KmxError) as e:
        gpu_assign(km, 17, data[:100 * spec.dim], means0, spec.dim, spec.k, 100)
    assert e.value.code == km.KMX_ERR_INVALID_ARGUMENT
    # the single-pass fused kernel is float-only and says so instead of running something else
    with pytest.raises(km.KmxError) as e:
        a = km.HipFusedKMeansAlgorithm(km.FUSED_ONE_PASS, dtype=np.float64)
        a.initialize(spec.dim, spec.k, 100, 1, data[:100 * spec.dim], means0)
        try:
            a.run()
        finally:
            a.cleanup()
    assert e.value.code == km.KMX_ERR_UNSUPPORTED
    # empty input: nothing to do
    assert gpu_assign(km, km.ASSIGN_BEST, np.zeros(0), means0, spec.dim, spec.k, 0).size == 0


def test_prepared_points_are_converted_once_and_forgotten_on_request(km, orc, gpu):
    """kmx_prepare_points_f64: assignment calls on the announced points reuse their float copy; the result is the one without the
    announcement; other points in between, and new values after kmx_forget_points_f64, are converted afresh."""
    dim, k, n = 32, 256, 20000
    rng = np.random.default_rng(11)
    first = rng.normal(size=n * dim) * 3
    other = rng.normal(size=n * dim) * 3 + 1
    means = first.reshape(n, dim)[:k].copy().ravel()
    lib = km.hip_lib()
    d1 = km.DeviceBuffer(8 * n * dim); d1.write(first)
    d2 = km.DeviceBuffer(8 * n * dim); d2.write(other)
    m = km.DeviceBuffer(8 * k * dim); m.write(means)
    a = km.DeviceBuffer(4 * n)

    def run(buf):
        km.assign(km.ASSIGN_BEST, buf, km.AOS, dim, m, km.AOS, dim, a, dim, k, n, dtype=np.float64)
        km.sync()
        return a.read(np.uint32, n)

    want_first = orc.assign_f64(first, means, dim, k, n, threads=0)
    want_other = orc.assign_f64(other, means, dim, k, n, threads=0)
    assert np.array_equal(run(d1), want_first)
    km.check(lib.kmx_prepare_points_f64(d1.ptr, km.AOS, dim, dim, n))
    assert np.array_equal(run(d1), want_first)
    assert np.array_equal(run(d1), want_first)
    assert np.array_equal(run(d2), want_other)          # other points: the library forgets by itself
    assert np.array_equal(run(d1), want_first)
    km.check(lib.kmx_prepare_points_f64(d1.ptr, km.AOS, dim, dim, n))
    km.check(lib.kmx_forget_points_f64())
    d1.write(other)                                      # allowed again: nothing is kept
    assert np.array_equal(run(d1), want_other)
    with pytest.raises(km.KmxError):
        km.check(lib.kmx_prepare_points_f64(d1.ptr, km.AOS, dim - 1, dim, n))   # stride < dim
    for b in (d1, d2, m, a):
        b.free()
