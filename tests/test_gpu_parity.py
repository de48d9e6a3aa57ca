"""Parity of the HIP path with the CPU oracle, through the C ABI, on a real MI355X (-m gpu).

Bar (from the benchmark definition): assignment and per-cluster counts bit-exact, except points
whose best and second-best reference distances differ by less than 1e-5 relative, which must be
reported; centroids within 1e-4 relative in fp32.

What "relative" means for a centroid coordinate: |gpu - oracle| / rms(oracle coordinates). Sums of
n fp32 terms in a different order differ by O(sqrt(n) eps |sum|); coordinates near zero would make
a per-coordinate relative error meaningless.

Lloyd trajectories are chaotic at the last bit: the update's fp32 sums are accumulated in a different
order from the serial loop (atomics, as in the reference's own GPU path), so after the first update the
two runs hold centroids that differ in their last bits and a near-tie point may then legitimately go
the other way, which moves two centroids by O(1/cluster size). Per-step ("teacher-forced") parity
therefore feeds the oracle the centroids / assignment the GPU actually used: that comparison is exact
and is the one that must show zero mismatches. The free-running comparison is reported and gated on
the near-tie rule for the first assignment and on cluster-count conservation afterwards.
"""
import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
AOS, SOA = 0, 1
CENTROID_RTOL = 1e-4   # relative to the rms centroid coordinate
NEAR_TIE = 1e-5        # relative gap between best and second-best reference distance


def rel_err(got, want):
    scale = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
    return float(np.abs(got.astype(np.float64) - want).max() / max(scale, 1e-30))


def gpu_assign(km, variant, data, means, dim, k, n, layout=AOS, layout_means=AOS, exec_params=None):
    alg = km.HipAssignmentAlgorithm(variant, exec_params, layout, layout_means)
    alg.initialize(dim, k, n, data, means)
    alg.run()
    out = alg.getAssignment()
    rechecked = km.last_rechecked()
    alg.cleanup()
    return out, rechecked


def gpu_update(km, variant, data, assignment, dim, k, n, layout=AOS, layout_means=AOS, exec_params=None, dirty=False):
    ex = exec_params if exec_params is not None else km.ExecParams()
    copies = max(1, ex.privatized_copies)
    d = km.DeviceBuffer(4 * max(data.size, 1)); d.write(data)
    a = km.DeviceBuffer(4 * max(n, 1)); a.write(assignment)
    msize = km.layout_size(layout_means, k, dim)
    m = km.DeviceBuffer(4 * msize * copies)
    s = km.DeviceBuffer(4 * k)
    if dirty:   # outputs full of leftovers (NaN bit patterns and large counts) instead of zeros
        m.write(np.full(msize * copies, 0x7FC12345, np.uint32)); s.write(np.full(k, 0xDEADBEEF, np.uint32))
    else:
        m.zero(); s.zero()
    km.update(variant, d, layout, km.layout_stride(layout, n, dim), a, m, layout_means,
              km.layout_stride(layout_means, k, dim), s, dim, k, n, ex)
    km.sync()
    means, sizes = m.read(np.float32, msize), s.read(np.uint32, k)
    for b in (d, a, m, s):
        b.free()
    return means, sizes


def variants(km, dim=1):
    v = [km.ASSIGN_BASE, km.ASSIGN_MFMA, km.ASSIGN_MFMA_BF16X3, km.ASSIGN_BEST]
    return v + [km.ASSIGN_LDS_FMA] if dim <= 64 else v


# ---------------------------------------------------------------- golden vectors of the reference

@pytest.fixture(scope="module")
def golden():
    with open(os.path.join(HERE, "golden", "golden_index.json")) as f:
        index = json.load(f)
    return index, np.load(os.path.join(HERE, "golden", "golden.npz"))


@pytest.mark.parametrize("name", ["cfg1_full", "cfg1_soa_soa", "cfg1_aos_soa", "cfg1_soa_aos", "cfg2_small",
                                  "cfg3_small", "cfg4_small", "cfg5_small"])
def test_first_pass_equals_reference_golden(km, gpu, golden, name):
    """One assignment pass from the initial centroids against the REFERENCE's own output (bit-exact)."""
    index, arrays = golden
    c = index[name]
    spec = km.baseline_config(c["config"])
    data = km.generate_points(spec, c["n"], layout=c["layout"])
    means0 = km.first_k_means(spec, c["layout_means"])
    want = arrays[name + "_assignment_first_pass"].astype(np.uint32)
    for v in variants(km, c["dim"]):
        got, _ = gpu_assign(km, v, data, means0, c["dim"], c["k"], c["n"], c["layout"], c["layout_means"])
        assert np.array_equal(got, want), "variant %d: %d mismatches" % (v, int((got != want).sum()))


# ---------------------------------------------------------------- single-step parity on awkward shapes

SHAPES = [
    (20, 128, 10240),   # the reference CLI's defaults (k-means.cpp:298-300)
    (3, 5, 257),        # odd everything
    (7, 33, 1000),
    (2, 2, 128),        # the CLI's minima
    (16, 16, 5000),
    (32, 1000, 4099),   # k not a multiple of the tile, n prime
    (64, 96, 2048),
    (100, 40, 1500),    # wide rows: 128-dimension MFMA instantiation, padded
    (256, 300, 700),    # widest supported row
    (130, 2000, 400),   # wide rows, centroids streamed through LDS in chunks
    (1, 7, 300),
    (5, 4100, 777),     # centroids do not fit one LDS chunk of the narrow layout
    (48, 300, 3000),    # exact pass with one centroid row per lane, rows of 33..64 floats
    (37, 2100, 2500),   # the same with a padded row and three chunks of centroids
    (64, 1024, 6000),
    (4, 9000, 3000),    # packed rows (at most 4 dimensions), more centroids than LDS holds: streamed
    (3, 200, 4000),     # packed rows, padded to 4 dimensions, screened exact pass
    (2, 600, 5000),
    (4, 1, 100),        # one centroid, one point
    (3, 5, 1),
    (40, 1, 1),
]


@pytest.mark.parametrize("dim,k,n", SHAPES)
@pytest.mark.parametrize("layout,layout_means", [(AOS, AOS), (SOA, SOA), (AOS, SOA), (SOA, AOS)])
def test_assignment_is_bit_exact(km, orc, gpu, dim, k, n, layout, layout_means):
    rng = np.random.default_rng(dim * 7919 + k)
    data = rng.normal(size=n * dim).astype(np.float32) * np.float32(3)
    means = data.reshape(-1)[:k * dim].copy() if n >= k and layout == AOS and layout_means == AOS \
        else rng.normal(size=k * dim).astype(np.float32) * np.float32(3)
    want = orc.assign(data, means, dim, k, n, layout, layout_means, threads=0, fast=True)
    for v in variants(km, dim):
        got, _ = gpu_assign(km, v, data, means, dim, k, n, layout, layout_means)
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, "variant %d: %d mismatches, first at %s" % (v, bad.size, bad[:5])


@pytest.mark.parametrize("dim,k,n", [(8, 64, 4096), (32, 256, 3000), (4, 512, 2000), (48, 160, 2000), (21, 1500, 4000), (96, 200, 1500)])
def test_hard_inputs(km, orc, gpu, dim, k, n):
    """Exact ties, duplicated centroids, coincident points, NaN / inf / huge / tiny values."""
    rng = np.random.default_rng(99 + dim)
    base = rng.normal(size=(n, dim)).astype(np.float32)
    means = rng.normal(size=(k, dim)).astype(np.float32)
    cases = {}
    m = means.copy(); m[k // 2] = m[3]; m[k - 1] = m[3]; m[7] = m[5]
    d = base.copy(); d[: k] = m                              # points exactly on (duplicated) centroids
    d[k: 2 * k] = (m + m[::-1]) / np.float32(2)              # midpoints: exact or near ties
    cases["duplicates_and_midpoints"] = (d, m)
    cases["all_points_identical"] = (np.repeat(base[:1], n, 0), means)
    cases["all_centroids_identical"] = (base, np.repeat(means[:1], k, 0))
    d = base.copy(); d[5, 0] = np.nan; d[9, dim - 1] = np.inf; d[11, 0] = -np.inf
    cases["nan_inf_points"] = (d, means)
    m = means.copy(); m[4, 1] = np.nan
    cases["nan_centroid"] = (base, m)
    m = means.copy(); m[0, 0] = np.nan
    cases["nan_centroid_zero"] = (base, m)
    m = means.copy(); m[6, 0] = np.inf
    cases["inf_centroid"] = (base, m)
    cases["huge"] = (base * np.float32(1e18), means * np.float32(1e18))       # squares overflow to inf
    cases["large"] = (base * np.float32(1e6) + np.float32(1e7), means * np.float32(1e6) + np.float32(1e7))
    cases["tiny"] = (base * np.float32(1e-25), means * np.float32(1e-25))     # squares underflow
    cases["grid_ties"] = (np.round(base * 2) / 2, np.round(means * 2) / 2)    # many exactly equal distances
    for name, (d, m) in cases.items():
        d = np.ascontiguousarray(d, dtype=np.float32).ravel()
        m = np.ascontiguousarray(m, dtype=np.float32).ravel()
        want = orc.assign(d, m, dim, k, n, threads=0, fast=True)
        for v in variants(km, dim):
            got, rechecked = gpu_assign(km, v, d, m, dim, k, n)
            bad = np.nonzero(got != want)[0]
            assert bad.size == 0, "%s, variant %d: %d mismatches, first at %s (gpu %s, oracle %s)" % (
                name, v, bad.size, bad[:5], got[bad[:5]], want[bad[:5]])


@pytest.mark.parametrize("dim,k,n,lds_budget", [
    (32, 2048, 66000, 0),       # two slices of 32 tiles
    (48, 1024, 65536, 0),       # two slices of the pipelined kernel for rows of 33..48 dimensions
    (64, 1100, 65537, 0),       # three slices would be needed: rows of 49..64 dimensions then stream (wide-row step)
    (60, 1000, 66000, 0),       # two slices of the wide-row kernel (AoS points; SoA points stream)
    (40, 1100, 65537, 0),       # k not a multiple of the tile: the last slice is shorter and padded
    (33, 300, 65600, 40000),    # a small LDS budget: many short slices
    (17, 250, 70000, 24000),
    (20, 3000, 70001, 0),
    (32, 800, 66000, 27700),    # LDS for four tiles: 25 tiles in six slices of four and a last slice of ONE tile under the pipelined step
    (48, 800, 66000, 35900),    # the same for rows of 33..48 dimensions
    (24, 130, 66000, 13400),    # LDS for one tile: five slices of one tile each
])
def test_centroids_swept_in_slices(km, orc, gpu, dim, k, n, lds_budget):
    """From 65536 points on, rows of 17 to 64 dimensions whose centroids do not fit the LDS are swept once per slice of
    centroids (49 to 64 dimensions: two slices at most, AoS points only); the leader and the two smallest values of a point
    travel between the launches. Plain data in all layouts;
    then duplicates of a centroid in the first and the last slice (a tie across slices), a NaN and an infinite centroid in
    the last slice, ties on a grid."""
    rng = np.random.default_rng(dim * 31 + k)
    centres = rng.uniform(-10, 10, (40, dim)).astype(np.float32)
    base = centres[rng.integers(0, 40, n)] + rng.normal(size=(n, dim)).astype(np.float32)
    means = base[rng.permutation(n)[:k]].copy()
    ex = lambda: km.ExecParams(shared_mem_bytes=lds_budget) if lds_budget else None
    v = km.ASSIGN_MFMA_BF16X3
    want = orc.assign(base.ravel(), means.ravel(), dim, k, n, threads=0, fast=True)
    for layout, layout_means in [(AOS, AOS), (SOA, SOA), (AOS, SOA)]:
        d = base if layout == AOS else np.ascontiguousarray(base.T)
        m = means if layout_means == AOS else np.ascontiguousarray(means.T)
        got, rechecked = gpu_assign(km, v, d.ravel(), m.ravel(), dim, k, n, layout, layout_means, ex())
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, "layouts %s/%s: %d mismatches, first at %s" % (layout, layout_means, bad.size, bad[:5])
        assert rechecked < n // 4    # the certificate decides most points: the slices were merged, not each one flagged
    cases = {}
    m = means.copy(); m[k - 1] = m[3]; m[k // 2] = m[3]
    d = base.copy(); d[:k] = m
    cases["duplicates_across_slices"] = (d, m)
    m = means.copy(); m[k - 2, 1] = np.nan
    cases["nan_centroid_in_the_last_slice"] = (base, m)
    m = means.copy(); m[k - 3, 0] = np.inf
    cases["inf_centroid_in_the_last_slice"] = (base, m)
    d = base.copy(); d[5, 0] = np.nan; d[9, dim - 1] = np.inf
    cases["nan_inf_points"] = (d, means)
    cases["grid_ties"] = (np.round(base), np.round(means))
    for name, (d, m) in cases.items():
        d = np.ascontiguousarray(d, dtype=np.float32).ravel()
        m = np.ascontiguousarray(m, dtype=np.float32).ravel()
        want = orc.assign(d, m, dim, k, n, threads=0, fast=True)
        got, _ = gpu_assign(km, v, d, m, dim, k, n, AOS, AOS, ex())
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, "%s: %d mismatches, first at %s (gpu %s, oracle %s)" % (name, bad.size, bad[:5], got[bad[:5]], want[bad[:5]])


@pytest.mark.parametrize("dim,k,n", [(32, 1024, 200000), (64, 512, 100000), (16, 256, 200000), (8, 100, 100000),
                                     (48, 2048, 70000), (128, 300, 50000), (200, 1024, 20000)])
@pytest.mark.parametrize("offset", [0.0, 100.0, 3000.0])
def test_data_far_from_the_origin(km, orc, gpu, dim, k, n, offset):
    """The split-bf16 sweep works in a frame moved to the middle of the centroids: the assignment is the oracle's wherever the
    data lie, and the share of the points that the sweep leaves to the exact pass does not grow with their distance from
    the origin (clusters of spread 1 inside [-10, 10]^d, moved by `offset` in every coordinate; in the frame of the data
    the certificate would give up on every point at the last offset)."""
    rng = np.random.default_rng(dim + k)
    centres = rng.uniform(-10, 10, (k, dim)).astype(np.float32)
    base = (centres[rng.integers(0, k, n)] + rng.normal(size=(n, dim)).astype(np.float32) + np.float32(offset)).astype(np.float32)
    means = base[:k].copy()
    want = orc.assign(base.ravel(), means.ravel(), dim, k, n, threads=0, fast=True)
    for layout in (AOS, SOA):
        d = base if layout == AOS else np.ascontiguousarray(base.T)
        got, rechecked = gpu_assign(km, km.ASSIGN_MFMA_BF16X3, d.ravel(), means.ravel(), dim, k, n, layout, AOS)
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, "layout %d: %d mismatches, first at %s" % (layout, bad.size, bad[:5])
        assert rechecked < n // 10, "%d of %d points left to the exact pass" % (rechecked, n)


@pytest.mark.parametrize("dim,k,n", [(2, 50, 200000), (3, 100, 200000), (2, 500, 100000), (8, 64, 200000), (4, 16, 200000),
                                     (12, 40, 200000), (40, 300, 50000), (100, 64, 30000)])
@pytest.mark.parametrize("offset", [0.0, 1000.0])
def test_data_far_from_the_origin_in_the_fp32_sweeps(km, orc, gpu, dim, k, n, offset):
    """The same for the fp32 MFMA sweep and the sweep on the vector ALU (and whatever the selector picks): they move their
    frame too and hand the exact pass thresholds of the frame of the data."""
    rng = np.random.default_rng(dim * 3 + k)
    centres = rng.uniform(-10, 10, (k, dim)).astype(np.float32)
    base = (centres[rng.integers(0, k, n)] + rng.normal(size=(n, dim)).astype(np.float32) + np.float32(offset)).astype(np.float32)
    means = base[:k].copy()
    want = orc.assign(base.ravel(), means.ravel(), dim, k, n, threads=0, fast=True)
    for v in [km.ASSIGN_MFMA, km.ASSIGN_BEST] + ([km.ASSIGN_LDS_FMA] if dim <= 64 else []):
        for layout in (AOS, SOA):
            d = base if layout == AOS else np.ascontiguousarray(base.T)
            got, rechecked = gpu_assign(km, v, d.ravel(), means.ravel(), dim, k, n, layout, AOS)
            bad = np.nonzero(got != want)[0]
            assert bad.size == 0, "variant %d, layout %d: %d mismatches, first at %s" % (v, layout, bad.size, bad[:5])
            assert rechecked < n // 10, "variant %d: %d of %d points left to the exact pass" % (v, rechecked, n)


@pytest.mark.parametrize("dim,k,n", [(32, 256, 3000), (21, 1500, 4000), (96, 200, 1500), (4, 512, 5000)])
def test_soa_points_in_the_exact_pass(km, orc, gpu, dim, k, n):
    """SoA points: the exact pass copies the rows of the queued points into a compact block. Inputs that queue every point
    (identical centroids, ties on a grid), with the default bound and with a bound of 1024 rows, which leaves most of
    the queue to the kernels that read the SoA data directly."""
    rng = np.random.default_rng(7 + dim)
    base = rng.normal(size=(n, dim)).astype(np.float32)
    means = rng.normal(size=(k, dim)).astype(np.float32)
    cases = {
        "all_centroids_identical": (base, np.repeat(means[:1], k, 0)),
        "grid_ties": (np.round(base * 2) / 2, np.round(means * 2) / 2),
        "plain": (base, means),
    }
    try:
        for limit in (1 << 30, 4096):
            km.set_queued_rows_limit(limit)
            for name, (d, m) in cases.items():
                want = orc.assign(np.ascontiguousarray(d).ravel(), np.ascontiguousarray(m).ravel(), dim, k, n, threads=0, fast=True)
                for layout_means in (km.AOS, km.SOA):
                    dd = np.ascontiguousarray(d.T).ravel()
                    mm = np.ascontiguousarray(m if layout_means == km.AOS else m.T).ravel()
                    for v in variants(km, dim):
                        got, _ = gpu_assign(km, v, dd, mm, dim, k, n, km.SOA, layout_means)
                        bad = np.nonzero(got != want)[0]
                        assert bad.size == 0, "%s, limit %d, variant %d: %d mismatches, first at %s" % (name, limit, v, bad.size, bad[:5])
    finally:
        km.set_queued_rows_limit(1 << 30)


def test_sqrt_is_correctly_rounded_on_device(km, orc, gpu):
    """The exact pass compares sqrt values: a 1-ulp device sqrt would flip ties. d = 1, k = n centroids such
    that point i's nearest candidates have adjacent squared distances; also a direct sweep through BASE."""
    rng = np.random.default_rng(5)
    n, k = 4096, 64
    data = rng.uniform(0.5, 100, size=n).astype(np.float32)
    means = np.sort(rng.uniform(0, 200, size=k).astype(np.float32))
    want = orc.assign(data, means, 1, k, n)
    for v in variants(km, 1):
        got, _ = gpu_assign(km, v, data, means, 1, k, n)
        assert np.array_equal(got, want)


def test_empty_input_and_argument_errors(km, gpu):
    ex = km.ExecParams()
    d = km.DeviceBuffer(8192); m = km.DeviceBuffer(8192); a = km.DeviceBuffer(64)
    km.assign(km.ASSIGN_BEST, d, AOS, 4, m, AOS, 4, a, 4, 2, 0, ex)        # n = 0 is a no-op
    assert ex.block_count == 0
    with pytest.raises(km.KmxError) as e:
        km.assign(99, d, AOS, 4, m, AOS, 4, a, 4, 2, 4, ex)
    assert e.value.code == km.KMX_ERR_INVALID_ARGUMENT
    with pytest.raises(km.KmxError) as e:
        km.assign(km.ASSIGN_BEST, d, AOS, 2, m, AOS, 4, a, 4, 2, 4, ex)    # stride < dim
    assert e.value.code == km.KMX_ERR_INVALID_ARGUMENT
    with pytest.raises(km.KmxError) as e:
        km.assign(km.ASSIGN_MFMA, d, AOS, 300, m, AOS, 300, a, 300, 2, 1, ex)  # dim beyond the MFMA variant
    assert e.value.code == km.KMX_ERR_UNSUPPORTED
    km.sync()
    for b in (d, m, a):
        b.free()


# ---------------------------------------------------------------- update

UPDATE_SHAPES = [(8, 64, 65536), (20, 128, 10240), (3, 5, 257), (32, 1024, 50000), (4, 4096, 100000),
                 (16, 16, 300000), (256, 1024, 4096), (33, 7, 1000), (2, 70000, 4096)]


@pytest.mark.parametrize("dim,k,n", UPDATE_SHAPES)
@pytest.mark.parametrize("layout,layout_means", [(AOS, AOS), (SOA, SOA), (AOS, SOA), (SOA, AOS)])
def test_update_matches_oracle(km, orc, gpu, dim, k, n, layout, layout_means):
    rng = np.random.default_rng(k + dim)
    data = rng.normal(size=n * dim).astype(np.float32) * np.float32(5) + np.float32(2)
    # skewed assignment with empty clusters: cluster 1 (if any) never occurs, low indices are hot
    asg = np.minimum((rng.exponential(scale=k / 4, size=n)).astype(np.uint32), k - 1).astype(np.uint32)
    if k > 2:
        asg[asg == 1] = 0
    want_means, want_sizes = orc.update(data, asg, dim, k, n, layout, layout_means, threads=0)
    cases = [(km.UPDATE_ATOMIC_POINT, km.ExecParams()), (km.UPDATE_ATOMIC_FINE, km.ExecParams()),
             (km.UPDATE_ATOMIC_SHM, km.ExecParams()),
             (km.UPDATE_ATOMIC_FINE, km.ExecParams(privatized_copies=3, items_per_thread=4)),
             (km.UPDATE_ATOMIC_SHM, km.ExecParams(shared_mem_bytes=48 * 1024)),
             (km.UPDATE_ATOMIC_WARP, km.ExecParams())]
    if n <= 70000:   # the micro-benchmark's baselines: compare-and-swap loops and the O(n k dim) kernel without atomics
        cases += [(km.UPDATE_ATOMIC_WARP | km.UPDATE_EMULATED_ATOMICS, km.ExecParams(privatized_copies=2)),
                  (km.UPDATE_ATOMIC_POINT | km.UPDATE_EMULATED_ATOMICS, km.ExecParams()),
                  (km.UPDATE_ATOMIC_FINE | km.UPDATE_EMULATED_ATOMICS, km.ExecParams()),
                  (km.UPDATE_BASE, km.ExecParams())]
    for variant, ex in cases:
        means, sizes = gpu_update(km, variant, data, asg, dim, k, n, layout, layout_means, ex)
        assert np.array_equal(sizes, want_sizes), "variant %d: counts differ" % variant
        assert rel_err(means, want_means) < CENTROID_RTOL, "variant %d" % variant
        if variant == km.UPDATE_BASE:   # no atomics, sums in point order: the serial loop's bits
            assert np.array_equal(means.view(np.uint32), want_means.view(np.uint32))
        if k > 2:
            lm = means.reshape(k, dim) if layout_means == AOS else means.reshape(dim, k).T
            assert np.all(lm[1] == 0), "empty cluster must stay at the origin"


@pytest.mark.gpu
@pytest.mark.parametrize("dim,k,n", [(32, 1024, 300000), (4, 4096, 200000), (256, 1024, 70000), (24, 700, 100000), (7, 300, 50000),
                                     (64, 2048, 1 << 20), (32, 1024, 700)])
def test_update_with_clusters_that_span_the_ranges_of_many_lane_groups(km, gpu, dim, k, n):
    """The sorted update cuts a chunk's sorted points into equal ranges per lane group; a cluster larger than a range is
    summed in pieces. Assignments that make such clusters (everything in one cluster, nine points in ten, sorted points,
    two clusters) against float64 sums of the same assignment; counts exact, empty clusters at the origin."""
    rng = np.random.default_rng(dim + k)
    rows = (rng.normal(size=(n, dim)) * 3 + 1).astype(np.float32)
    patterns = {
        "all in the last": np.full(n, k - 1, np.uint32),
        "all in the first": np.zeros(n, np.uint32),
        "nine in ten in one": np.where(rng.random(n) < 0.9, k // 3, rng.integers(0, k, n)).astype(np.uint32),
        "sorted": np.sort(rng.integers(0, k, n)).astype(np.uint32),
        "two clusters": np.where(rng.random(n) < 0.5, 5, k - 2).astype(np.uint32),
        "runs": (np.arange(n) // 1500 % k).astype(np.uint32),
    }
    for name, asg in patterns.items():
        means, sizes = gpu_update(km, km.UPDATE_ATOMIC_SHM, rows.ravel(), asg, dim, k, n, AOS, AOS, km.ExecParams(), dirty=True)
        counts = np.bincount(asg, minlength=k)
        assert np.array_equal(sizes, counts), name
        sums = np.zeros((k, dim)); np.add.at(sums, asg, rows.astype(np.float64))
        want = np.where(counts[:, None] > 0, sums / np.maximum(counts, 1)[:, None], 0.0)
        got = means.reshape(k, dim)
        assert np.all(got[counts == 0] == 0), name
        scale = float(np.sqrt(np.mean(want[counts > 0] ** 2)))
        assert float(np.abs(got - want).max()) / scale < 1e-5, name


@pytest.mark.parametrize("dim,k,n", UPDATE_SHAPES + [(8, 64, 0), (32, 1024, 0), (8, 1024, 9000000)])   # the last: more than 256 chunks of sorted points
@pytest.mark.parametrize("layout,layout_means", [(AOS, AOS), (SOA, SOA), (AOS, SOA), (SOA, AOS)])
def test_tuned_update_needs_no_zeroed_outputs(km, orc, gpu, dim, k, n, layout, layout_means):
    """KMX_UPDATE_ATOMIC_SHM overwrites or clears its outputs itself: leftovers in them change nothing."""
    rng = np.random.default_rng(3 * k + dim)
    data = rng.normal(size=n * dim).astype(np.float32) * np.float32(5) + np.float32(2)
    asg = np.minimum((rng.exponential(scale=k / 4, size=n)).astype(np.uint32), k - 1).astype(np.uint32)
    if k > 2:
        asg[asg == 1] = 0
    want_means, want_sizes = orc.update(data, asg, dim, k, n, layout, layout_means, threads=0)
    for ex in (km.ExecParams(), km.ExecParams(shared_mem_bytes=48 * 1024)):
        means, sizes = gpu_update(km, km.UPDATE_ATOMIC_SHM, data, asg, dim, k, n, layout, layout_means, ex, dirty=True)
        assert np.array_equal(sizes, want_sizes)
        assert rel_err(means, want_means) < CENTROID_RTOL
        if k > 2:
            lm = means.reshape(k, dim) if layout_means == AOS else means.reshape(dim, k).T
            assert np.all(lm[1] == 0), "empty cluster must end at the origin"


# ---------------------------------------------------------------- the Lloyd loop

def forced_run(km, orc, cid, n, iters, av, uv, layout=AOS, layout_means=AOS):
    """Runs the GPU loop and checks every step against the oracle fed with the GPU's own inputs."""
    spec = km.baseline_config(cid)
    dim, k = spec.dim, spec.k
    data = km.generate_points(spec, n, layout=layout)
    means0 = km.first_k_means(spec, layout_means)
    alg = km.HipKMeansAlgorithm(av, uv, layout=layout, layout_means=layout_means)
    alg.initialize(dim, k, n, iters, data, means0)
    report = []
    for it in range(iters):
        prev = alg.getMeans()
        nxt = alg.iteration()
        rechecked = km.last_rechecked()
        ga = alg.cu_assignment[nxt].read(np.uint32, n)
        oa = orc.assign(data, prev, dim, k, n, layout, layout_means, threads=0, fast=True)
        alg.update_step(nxt)
        gm, gs = alg.getMeans(), alg.getClusterSizes()
        om, osz = orc.update(data, ga, dim, k, n, layout, layout_means, threads=0)
        report.append(dict(iteration=it, rechecked=rechecked, mismatches=int((ga != oa).sum()),
                           counts_equal=bool(np.array_equal(gs, osz)), centroid_err=rel_err(gm, om)))
    alg.cleanup()
    return report


LOOP_CASES = [(1, 65536, 10), (2, 65536, 4), (3, 131072, 3), (5, 1 << 20, 4), (4, 8192, 2)]


@pytest.mark.parametrize("cid,n,iters", LOOP_CASES)
def test_every_iteration_matches_oracle(km, orc, gpu, cid, n, iters):
    spec = km.baseline_config(cid)
    combos = [(km.ASSIGN_BEST, km.UPDATE_ATOMIC_SHM)]
    combos += [(km.ASSIGN_MFMA, km.UPDATE_ATOMIC_FINE), (km.ASSIGN_MFMA_BF16X3, km.UPDATE_ATOMIC_SHM)]
    if spec.dim <= 64:
        combos += [(km.ASSIGN_LDS_FMA, km.UPDATE_ATOMIC_SHM)]
    if n * spec.k * spec.dim <= 1 << 31:
        combos += [(km.ASSIGN_BASE, km.UPDATE_ATOMIC_POINT)]
    for av, uv in combos:
        for r in forced_run(km, orc, cid, n, iters, av, uv):
            assert r["mismatches"] == 0 and r["counts_equal"], (av, uv, r)
            assert r["centroid_err"] < CENTROID_RTOL, (av, uv, r)


@pytest.mark.gpu
@pytest.mark.parametrize("cid,n,iters,layout,layout_means", [(1, 65536, 4, AOS, AOS), (2, 32768, 2, AOS, AOS),
                                                             (5, 1 << 18, 3, AOS, AOS), (1, 20000, 2, SOA, AOS)])
def test_fused_iterations_match_oracle(km, orc, gpu, cid, n, iters, layout, layout_means):
    """FUSED kernel call (kernels.cuh:107-116): every iteration checked against the oracle fed with the same centroids;
    the assignment it reports afterwards is the serial argmin against the FINAL centroids (cuda.hpp:199-221)."""
    spec = km.baseline_config(cid)
    dim, k = spec.dim, spec.k
    data = km.generate_points(spec, n, layout=layout)
    means0 = km.first_k_means(spec, layout_means)
    alg = km.HipFusedKMeansAlgorithm(layout=layout, layout_means=layout_means)   # one pass for configuration 5, two otherwise
    alg.initialize(dim, k, n, iters, data, means0)
    for _ in range(iters):
        prev = alg.getMeans()
        alg.iteration()
        gm, gs = alg.getMeans(), alg.getClusterSizes()
        oa = orc.assign(data, prev, dim, k, n, layout, layout_means, threads=0, fast=True)
        om, osz = orc.update(data, oa, dim, k, n, layout, layout_means, threads=0)
        assert np.array_equal(gs, osz)
        assert rel_err(gm, om) < CENTROID_RTOL
    final = alg.getMeans()
    want = orc.assign(data, final, dim, k, n, layout, layout_means, threads=0, fast=True)
    assert np.array_equal(alg.getAssignment(), want)
    alg.cleanup()


def near_tie_report(orc, data, means, dim, k, n, points):
    """For each listed point: relative gap between the smallest and the second smallest serial distance to `means`
    (the rule of the benchmark definition: a point whose gap is below 1e-5 may legitimately differ between two runs)."""
    sub = np.ascontiguousarray(data.reshape(n, dim)[points]).ravel()
    best = orc.assign(sub, means, dim, k, points.size, threads=0, fast=True)
    x = sub.reshape(points.size, dim)
    c = means.reshape(k, dim)
    dist = np.empty((points.size, k), np.float32)
    for j in range(k):                                    # the serial arithmetic: fp32, ascending dimension, unfused
        acc = np.zeros(points.size, np.float32)
        for q in range(dim):
            diff = (x[:, q] - c[j, q]).astype(np.float32)
            acc = (acc + (diff * diff).astype(np.float32)).astype(np.float32)
        dist[:, j] = np.sqrt(acc, dtype=np.float32)
    assert np.array_equal(dist.argmin(1), best)
    two = np.partition(dist, 1, axis=1)[:, :2].astype(np.float64)
    return (two[:, 1] - two[:, 0]) / np.maximum(two[:, 1], 1e-30)


def test_free_running_loop_reports_only_near_ties(km, orc, gpu):
    """Whole run against the oracle's whole run (config 1 in full, as the reference's --verify does,
    k-means.cpp:171-182). The first assignment must be identical. After that the runs may part at near-ties (the
    update's fp32 sums are taken in another order): the first iteration at which the assignments differ is looked at,
    where both runs still hold centroids that agree to rounding, and every point that differs there must be a near-tie
    of the oracle's own centroids: best and second-best serial distance closer than 1e-5 relative. The count is reported."""
    spec = km.baseline_config(1)
    n, dim, k, iters = int(spec.n), spec.dim, spec.k, spec.iterations
    data, means0 = km.generate_points(spec), km.first_k_means(spec)
    alg = km.HipKMeansAlgorithm(km.ASSIGN_BEST, km.UPDATE_ATOMIC_SHM)
    alg.initialize(dim, k, n, iters, data, means0)
    o_means = means0.copy()
    first_split = None
    for it in range(iters):
        nxt = alg.iteration()
        ga = alg.cu_assignment[nxt].read(np.uint32, n)
        alg.update_step(nxt)
        o_prev = o_means
        oa = orc.assign(data, o_prev, dim, k, n, threads=0, fast=True)
        o_means, _ = orc.update(data, oa, dim, k, n, threads=0)
        differ = np.nonzero(ga != oa)[0]
        if it == 0:
            assert differ.size == 0, "the first assignment reads identical centroids and must be identical"
        if differ.size and first_split is None:
            first_split = it
            gaps = near_tie_report(orc, data, o_prev, dim, k, n, differ)
            print("free-running config 1: runs part at iteration %d, %d points differ, largest relative gap %.3e"
                  % (it, differ.size, float(gaps.max())))
            assert np.all(gaps < NEAR_TIE), "%d differing points are no near-ties" % int((gaps >= NEAR_TIE).sum())
    gm, ga, gs = alg.getMeans(), alg.getAssignment(), alg.getClusterSizes()
    alg.cleanup()
    assert int(gs.sum()) == n and np.array_equal(gs, np.bincount(ga, minlength=k).astype(np.uint32))
    differ = np.nonzero(ga != oa)[0]
    print("free-running config 1: %d of %d points differ after %d iterations; centroid error %.3e"
          % (differ.size, n, iters, rel_err(gm, o_means)))
    assert differ.size <= n // 1000     # a split moves two centroids by O(1 / cluster size); bound the damage
    if first_split is None:
        _, osz = orc.update(data, oa, dim, k, n, threads=0)
        assert np.array_equal(gs, osz) and rel_err(gm, o_means) < CENTROID_RTOL


# ---------------------------------------------------------------- whole runs with the bits of the serial run

GOLDEN_CASES = ["cfg1_full", "cfg1_soa_soa", "cfg1_aos_soa", "cfg1_soa_aos", "cfg2_small", "cfg3_small", "cfg4_small", "cfg5_small"]


@pytest.mark.parametrize("name", GOLDEN_CASES)
@pytest.mark.parametrize("update_variant", ["base", "serial_order"])
def test_whole_runs_equal_the_reference_golden(km, gpu, golden, name, update_variant):
    """A free-running Lloyd run (no teacher forcing) with the selector's assignment and an update that adds in the
    serial order, against what the REFERENCE's SerialKMeansAlgorithm left after the same number of iterations
    (tests/golden/make_golden.py): final assignment, counts and centroids bit for bit."""
    index, arrays = golden
    c = index[name]
    spec = km.baseline_config(c["config"])
    data = km.generate_points(spec, c["n"], layout=c["layout"])
    means0 = km.first_k_means(spec, c["layout_means"])
    uv = km.UPDATE_BASE if update_variant == "base" else km.UPDATE_SERIAL_ORDER
    alg = km.HipKMeansAlgorithm(km.ASSIGN_BEST, uv, layout=c["layout"], layout_means=c["layout_means"])
    alg.initialize(c["dim"], c["k"], c["n"], c["iterations"], data, means0)
    alg.run()
    means, asg, sizes = alg.getMeans(), alg.getAssignment(), alg.getClusterSizes()
    alg.cleanup()
    want = arrays[name + "_assignment"].astype(np.uint32)
    assert np.array_equal(asg, want), "%d points differ from the reference's final assignment" % int((asg != want).sum())
    assert np.array_equal(sizes, arrays[name + "_counts"])
    head = arrays[name + "_means_head"]
    assert np.array_equal(means[:head.size].view(np.uint32), head.view(np.uint32))
    assert "%016x" % km.fnv1a64(means) == c["means_fnv1a64"]


@pytest.mark.parametrize("dim,k,n", UPDATE_SHAPES + [(8, 64, 0), (5, 20000, 30000), (1, 1, 1000), (16, 16, 1 << 20)])
@pytest.mark.parametrize("layout,layout_means", [(AOS, AOS), (SOA, SOA), (AOS, SOA), (SOA, AOS)])
def test_serial_order_update_has_the_bits_of_the_serial_loop(km, orc, gpu, dim, k, n, layout, layout_means):
    """KMX_UPDATE_SERIAL_ORDER against the oracle's update, bit for bit, on random assignments with empty clusters, one
    very large cluster and outputs full of leftovers (the variant has no precondition on them)."""
    rng = np.random.default_rng(dim * 1000003 + k * 101 + n)
    data = (rng.standard_normal(max(n, 1) * dim) * 3 + 1).astype(np.float32)[:n * dim]
    asg = rng.integers(0, k, size=n, dtype=np.uint32)
    if k > 2 and n:
        asg[asg == 1] = 0                                    # cluster 1 stays empty
        asg[rng.random(n) < 0.3] = k - 1                     # one cluster with a third of the points
    if layout == SOA:
        data = np.ascontiguousarray(data.reshape(n, dim).T).ravel()
    means, sizes = gpu_update(km, km.UPDATE_SERIAL_ORDER, data, asg, dim, k, n, layout, layout_means, dirty=True)
    want_means, want_sizes = orc.update(data, asg, dim, k, n, layout, layout_means, threads=0)
    assert np.array_equal(sizes, want_sizes)
    assert np.array_equal(means.view(np.uint32), want_means.view(np.uint32)), \
        "%d of %d centroid coordinates differ in their bits" % (int((means.view(np.uint32) != want_means.view(np.uint32)).sum()), means.size)


FULL_RUNS = [(1, None), (2, None), (3, None), (4, None), (5, 1 << 20)]


@pytest.mark.parametrize("cid,n", FULL_RUNS)
def test_full_runs_are_identical_to_the_serial_run(km, orc, gpu, cid, n):
    """The benchmark configurations at their full size (configuration 5: the first 2^20 points) and full iteration
    count, free-running: selector's assignment + serial-order update on the device against the oracle's whole serial
    run (all cores; the same per-element operations as one core). Zero mismatches, counts equal, centroids bit-equal."""
    spec = km.baseline_config(cid)
    n = int(spec.n) if n is None else n
    dim, k, iters = spec.dim, spec.k, spec.iterations
    data, means0 = km.generate_points(spec, n), km.first_k_means(spec)
    alg = km.HipKMeansAlgorithm(km.ASSIGN_BEST, km.UPDATE_SERIAL_ORDER)
    alg.initialize(dim, k, n, iters, data, means0)
    alg.run()
    gm, ga, gs = alg.getMeans(), alg.getAssignment(), alg.getClusterSizes()
    alg.cleanup()
    om, oa, osz = orc.kmeans(data, means0, dim, k, n, iters, threads=0, fast=True)
    differ = int((ga != oa).sum())
    print("configuration %d, N = %d, %d iterations free-running with the serial-order update: %d assignment mismatches, "
          "centroids %s" % (cid, n, iters, differ, "bit-equal" if np.array_equal(gm.view(np.uint32), om.view(np.uint32)) else "differ"))
    assert differ == 0
    assert np.array_equal(gs, osz)
    assert np.array_equal(gm.view(np.uint32), om.view(np.uint32))


@pytest.mark.parametrize("cid,n", FULL_RUNS)
def test_free_running_default_parts_from_the_serial_run_only_at_near_ties(km, orc, gpu, cid, n):
    """The fast default (tuned update, sums in another order) free-running beside the run with the serial-order update,
    which the test above holds bit-identical to the serial run and which therefore stands for it here, iteration by
    iteration. Where the two part for the first time both still hold centroids that agree to rounding, and every point
    that differs there must be a near-tie of the serial centroids (best and second-best serial distance closer than
    1e-5 relative) or lie within the distance between the two runs' centroids. The line printed at the end is the figure of record: mismatches and centroid error after the full
    iteration count."""
    spec = km.baseline_config(cid)
    n = int(spec.n) if n is None else n
    dim, k, iters = spec.dim, spec.k, spec.iterations
    data, means0 = km.generate_points(spec, n), km.first_k_means(spec)
    fast = km.HipKMeansAlgorithm(km.ASSIGN_BEST, km.UPDATE_ATOMIC_SHM)
    ref = km.HipKMeansAlgorithm(km.ASSIGN_BEST, km.UPDATE_SERIAL_ORDER)
    fast.initialize(dim, k, n, iters, data, means0)
    ref.initialize(dim, k, n, iters, data, means0)
    first_split, split_points, near_ties, largest_gap = None, 0, 0, 0.0
    for it in range(iters):
        r_prev, f_prev = ref.getMeans(), fast.getMeans()
        fa_buf, ra_buf = fast.iteration(), ref.iteration()
        fa = fast.cu_assignment[fa_buf].read(np.uint32, n)
        ra = ref.cu_assignment[ra_buf].read(np.uint32, n)
        fast.update_step(fa_buf)
        ref.update_step(ra_buf)
        differ = np.nonzero(fa != ra)[0]
        if it == 0:
            assert differ.size == 0, "the first assignment reads identical centroids and must be identical"
        if differ.size and first_split is None:
            first_split, split_points = it, int(differ.size)
            sub = np.ascontiguousarray(data.reshape(n, dim)[differ]).ravel()
            _, best, second = orc.assign(sub, r_prev, dim, k, differ.size, threads=0, fast=False, detail=True)
            gaps = (second.astype(np.float64) - best) / np.maximum(second.astype(np.float64), 1e-30)
            largest_gap, near_ties = float(gaps.max()), int((gaps < NEAR_TIE).sum())
            # Whatever is no near-tie must be explained by how far the two runs' centroids already lie apart (the serial
            # fp32 sum of a very large cluster is itself 1e-3 off its exact value, configuration 5): moving centroid j
            # by |delta_j| changes a distance by at most |delta_j|, so the point can only go from a to b if
            # d_b - d_a <= |delta_a| + |delta_b| (distances to the serial centroids, in float64).
            x = sub.reshape(differ.size, dim).astype(np.float64)
            rc, fc = r_prev.reshape(k, dim).astype(np.float64), f_prev.reshape(k, dim).astype(np.float64)
            a, b = ra[differ], fa[differ]
            d_a, d_b = np.sqrt(((x - rc[a]) ** 2).sum(1)), np.sqrt(((x - rc[b]) ** 2).sum(1))
            moved = np.sqrt(((fc - rc) ** 2).sum(1))
            unexplained = (d_b - d_a) > moved[a] + moved[b] + NEAR_TIE * d_b
            assert not unexplained.any(), "%d differing points are neither near-ties nor within the distance between the two runs' centroids" % int(unexplained.sum())
    fm, fa, fs = fast.getMeans(), fast.getAssignment(), fast.getClusterSizes()
    rm, ra = ref.getMeans(), ref.getAssignment()
    fast.cleanup(); ref.cleanup()
    assert int(fs.sum()) == n and np.array_equal(fs, np.bincount(fa, minlength=k).astype(np.uint32))
    print("free-running default, configuration %d, N = %d: parts from the serial run at iteration %s (%d points, %d of them near-ties "
          "below 1e-5, largest relative gap %.2e, the rest within the distance between the two runs' centroids); after %d iterations "
          "%d of %d points differ, centroid error %.3e of the rms coordinate"
          % (cid, n, first_split, split_points, near_ties, largest_gap, iters, int((fa != ra).sum()), n, rel_err(fm, rm)))
    if first_split is None:
        assert rel_err(fm, rm) < CENTROID_RTOL


# ---------------------------------------------------------------- full benchmark sizes: every point against the oracle

@pytest.mark.parametrize("cid", [1, 2, 3, 4, 5])
def test_full_size_exact_parity(km, orc, gpu, cid):
    """The first two iterations of every benchmark configuration at its full size, teacher-forced: ALL points against
    the serial oracle (16 threads, the same per-element operations), counts equal, centroids within tolerance."""
    spec = km.baseline_config(cid)
    n, dim, k = int(spec.n), spec.dim, spec.k
    data, means0 = km.generate_points(spec), km.first_k_means(spec)
    alg = km.HipKMeansAlgorithm(km.ASSIGN_BEST, km.UPDATE_ATOMIC_SHM)
    alg.initialize(dim, k, n, 2, data, means0)
    for it in range(2):
        prev = alg.getMeans()
        nxt = alg.iteration()
        rechecked = km.last_rechecked()
        ga = alg.cu_assignment[nxt].read(np.uint32, n)
        oa = orc.assign(data, prev, dim, k, n, threads=0, fast=True)
        bad = np.nonzero(ga != oa)[0]
        assert bad.size == 0, "configuration %d, iteration %d: %d of %d points differ (first %s); %d went to the exact pass" % (
            cid, it, bad.size, n, bad[:5], rechecked)
        alg.update_step(nxt)
        gm, gs = alg.getMeans(), alg.getClusterSizes()
        om, osz = orc.update(data, ga, dim, k, n, threads=0)
        assert np.array_equal(gs, osz)
        # Centroids: against the means of the same members in float64, and against the serial loop within that loop's
        # own distance from them. The serial fp32 sum of millions of addends stagnates (configuration 5: eight million
        # members in one cluster, running sum beyond 2^26, so every addend is rounded to a multiple of 8): the
        # reference's CPU centroids are then off by 1e-2, which no other summation order reproduces.
        pts = data.reshape(n, dim)
        sums = np.stack([np.bincount(ga, weights=pts[:, q].astype(np.float64), minlength=k) for q in range(dim)], 1)
        truth = np.where(osz[:, None] > 0, sums / np.maximum(osz, 1)[:, None], 0.0).ravel()
        serial_off = rel_err(om, truth)
        assert rel_err(gm, truth) < CENTROID_RTOL
        assert rel_err(gm, om) < CENTROID_RTOL + serial_off
        print("configuration %d, iteration %d: %d points identical, %d through the exact pass; centroids %.1e from the float64 "
              "means (the serial fp32 loop: %.1e)" % (cid, it, n, rechecked, rel_err(gm, truth), serial_off))
    alg.cleanup()


# ---------------------------------------------------------------- full benchmark sizes: size-independent properties

@pytest.mark.parametrize("cid", [2, 3, 4, 5])
def test_full_size_properties(km, orc, gpu, cid):
    spec = km.baseline_config(cid)
    n, dim, k = int(spec.n), spec.dim, spec.k
    data, means0 = km.generate_points(spec), km.first_k_means(spec)
    alg = km.HipKMeansAlgorithm(km.ASSIGN_BEST, km.UPDATE_ATOMIC_SHM)
    alg.initialize(dim, k, n, 2, data, means0)
    alg.run(iters=1)
    means1 = alg.getMeans()
    nxt = alg.iteration()                      # second assignment, against means1
    ga = alg.cu_assignment[nxt].read(np.uint32, n)
    rechecked = km.last_rechecked()
    alg.update_step(nxt)
    km.sync()
    gm, gs = alg.getMeans(), alg.getClusterSizes()
    # idempotence: assigning again against the same centroids gives the same vector
    again, _ = gpu_assign(km, km.ASSIGN_BEST, data, means1, dim, k, n)
    assert np.array_equal(again, ga)
    alg.cleanup()
    # counts are the histogram of the assignment and sum to n
    assert ga.max() < k
    hist = np.bincount(ga, minlength=k).astype(np.uint32)
    assert np.array_equal(gs, hist) and int(gs.sum()) == n
    # centroid * count = sum of members (float64 recomputation, independent of any fp32 order)
    pts = data.reshape(n, dim)
    sums = np.stack([np.bincount(ga, weights=pts[:, d].astype(np.float64), minlength=k) for d in range(dim)], 1)
    want = np.where(hist[:, None] > 0, sums / np.maximum(hist, 1)[:, None], 0.0)
    assert rel_err(gm.reshape(k, dim), want) < CENTROID_RTOL
    # exact oracle on a seeded sample of points, all k centroids
    rng = np.random.default_rng(cid)
    sample = np.sort(rng.choice(n, size=min(n, 200000 // max(1, k // 64)), replace=False))
    want_s = orc.assign(np.ascontiguousarray(pts[sample]).ravel(), means1, dim, k, sample.size, threads=0, fast=True)
    assert np.array_equal(ga[sample], want_s)
    # every point is at least as close to its centroid as to a random other one (float64)
    other = rng.integers(0, k, size=sample.size)
    c = means1.reshape(k, dim).astype(np.float64)
    x = pts[sample].astype(np.float64)
    d_own = ((x - c[ga[sample]]) ** 2).sum(1)
    d_other = ((x - c[other]) ** 2).sum(1)
    assert np.all(d_own <= d_other * (1 + 1e-5) + 1e-12)
    assert rechecked < n // 10


# ---------------------------------------------------------------- one call per iteration

@pytest.mark.parametrize("dim,k,n", [(16, 16, 100000), (3, 5, 257), (8, 32, 5000), (20, 7, 3333), (32, 32, 4099), (4, 2, 70000),
                                     (16, 33, 20000), (40, 16, 9000), (32, 1024, 30000)])   # the last three: two passes
@pytest.mark.parametrize("layout,layout_means", [(AOS, AOS), (SOA, SOA), (AOS, SOA), (SOA, AOS)])
def test_one_call_iteration(km, orc, gpu, dim, k, n, layout, layout_means):
    """kmx_iteration_f32 (cuda.hpp:72-85 in one call): the assignment is the serial scan's, counts exact, centroids within
    tolerance, outputs full of leftovers on entry; a single pass over the points where k <= 32 and dim <= 32."""
    rng = np.random.default_rng(dim * 977 + k)
    centres = rng.uniform(-10, 10, size=(max(k // 2, 1), dim))
    pts = (centres[rng.integers(0, centres.shape[0], size=n)] + rng.normal(size=(n, dim))).astype(np.float32)
    means = pts[:k].copy()
    if k > 3:
        means[2] = means[1]                                  # a duplicate: exact ties
    data = np.ascontiguousarray(pts if layout == AOS else pts.T).ravel()
    cents = np.ascontiguousarray(means if layout_means == AOS else means.T).ravel()
    d = km.DeviceBuffer(data.nbytes); d.write(data)
    m_in = km.DeviceBuffer(cents.nbytes); m_in.write(cents)
    m_out = km.DeviceBuffer(cents.nbytes); m_out.write(np.full(cents.size, 0x7FC12345, np.uint32))
    a = km.DeviceBuffer(4 * n); a.write(np.full(n, 0xFFFFFFF0, np.uint32))
    s = km.DeviceBuffer(4 * k); s.write(np.full(k, 0xDEADBEEF, np.uint32))
    km.iteration(d, layout, km.layout_stride(layout, n, dim), m_in, m_out, layout_means, km.layout_stride(layout_means, k, dim), a, s, dim, k, n)
    km.sync()
    assert km.last_iteration_passes() == (1 if k <= 32 and dim <= 32 else 2)
    got_a, got_m, got_s = a.read(np.uint32, n), m_out.read(np.float32, cents.size), s.read(np.uint32, k)
    for b in (d, m_in, m_out, a, s):
        b.free()
    want_a = orc.assign(data, cents, dim, k, n, layout, layout_means, threads=0, fast=True)
    bad = np.nonzero(got_a != want_a)[0]
    assert bad.size == 0, "%d of %d points differ (first %s: %s, oracle %s)" % (bad.size, n, bad[:5], got_a[bad[:5]], want_a[bad[:5]])
    want_m, want_s = orc.update(data, want_a, dim, k, n, layout, layout_means, threads=0)
    assert np.array_equal(got_s, want_s)
    assert rel_err(got_m, want_m) < CENTROID_RTOL


def test_single_pass_kernel_is_bounded_by_what_a_buffer_descriptor_spans(km, gpu):
    """The single-pass kernel reads its points through one buffer descriptor (up to 0xF0000000 bytes): a larger array is
    refused by name when the kernel is asked for, and kmx_iteration_f32 takes two passes. The points are zeros: every
    point ties between all centroids, the serial scan returns centroid 0, and only the first centroid gets members."""
    dim, k = 16, 4
    n = (0xF0000000 // (4 * dim)) + 4096                   # just past the bound: 4.03 GB of points
    d = km.DeviceBuffer(4 * n * dim); d.zero()
    cents = np.zeros(k * dim, np.float32); cents[dim:] = 1.0   # centroid 0 at the origin, the others away from it
    m_in = km.DeviceBuffer(cents.nbytes); m_in.write(cents)
    m_out = km.DeviceBuffer(cents.nbytes); m_out.zero()
    s = km.DeviceBuffer(4 * k); s.zero()
    a = km.DeviceBuffer(4 * n)
    try:
        with pytest.raises(km.KmxError, match="single-pass"):
            km.fused(km.FUSED_ONE_PASS, d, AOS, dim, m_in, m_out, AOS, dim, s, dim, k, n)
        km.iteration(d, AOS, dim, m_in, m_out, AOS, dim, a, s, dim, k, n)
        km.sync()
        assert km.last_iteration_passes() == 2
        sizes = s.read(np.uint32, k)
        assert sizes.tolist() == [n, 0, 0, 0]
        assert not a.read(np.uint32, n).any()
    finally:
        for b in (d, m_in, m_out, s, a):
            b.free()


@pytest.mark.parametrize("cid,n,iters", [(5, 1 << 18, 4), (1, 65536, 3), (2, 65536, 2)])
def test_whole_runs_through_the_one_call(km, orc, gpu, cid, n, iters):
    """HipKMeansAlgorithm.run() with the default pair of kernels goes through kmx_iteration_f32: every iteration against
    the oracle fed with the centroids the device used."""
    spec = km.baseline_config(cid)
    dim, k = spec.dim, spec.k
    data, means0 = km.generate_points(spec, n), km.first_k_means(spec)
    alg = km.HipKMeansAlgorithm(km.ASSIGN_BEST, km.UPDATE_ATOMIC_SHM)
    alg.initialize(dim, k, n, iters, data, means0)
    assert alg.one_call()
    for it in range(iters):
        prev = alg.getMeans()
        alg.step()
        km.sync()
        ga, gm, gs = alg.getAssignment(), alg.getMeans(), alg.getClusterSizes()
        oa = orc.assign(data, prev, dim, k, n, threads=0, fast=True)
        assert np.array_equal(ga, oa), "iteration %d: %d mismatches" % (it, int((ga != oa).sum()))
        om, osz = orc.update(data, oa, dim, k, n, threads=0)
        assert np.array_equal(gs, osz) and rel_err(gm, om) < CENTROID_RTOL
    alg.cleanup()


# ---------------------------------------------------------------- recorded iterations (HIP graph)

def fused_step(km, variant, data, means, dim, k, n, layout=AOS, layout_means=AOS):
    d = km.DeviceBuffer(data.nbytes); d.write(data)
    mi = km.DeviceBuffer(means.nbytes); mi.write(means)
    mo = km.DeviceBuffer(means.nbytes); mo.zero()
    s = km.DeviceBuffer(4 * k); s.zero()
    km.fused(variant, d, layout, km.layout_stride(layout, n, dim), mi, mo, layout_means, km.layout_stride(layout_means, k, dim),
             s, dim, k, n)
    km.sync()
    out = mo.read(np.float32, means.size), s.read(np.uint32, k)
    for b in (d, mi, mo, s):
        b.free()
    return out


@pytest.mark.gpu
@pytest.mark.parametrize("dim,k,n", [(16, 16, 100000), (3, 5, 257), (2, 2, 128), (8, 32, 5000), (20, 7, 3333), (32, 32, 4099),
                                     (1, 3, 300), (31, 9, 1000)])
@pytest.mark.parametrize("layout,layout_means", [(AOS, AOS), (SOA, SOA), (AOS, SOA), (SOA, AOS)])
def test_single_pass_fused_kernel(km, orc, gpu, dim, k, n, layout, layout_means):
    """KMX_FUSED_ONE_PASS: counts exactly those of the serial assignment, centroids within tolerance; the variants agree."""
    rng = np.random.default_rng(dim * 131 + k)
    centres = rng.normal(size=(k, dim)).astype(np.float32) * np.float32(2)
    pts = (centres[rng.integers(0, k, size=n)] + rng.normal(size=(n, dim)).astype(np.float32)).astype(np.float32)
    pts[: k] = centres                                   # points exactly on centroids
    means = centres.copy()
    if k > 2:
        means[k - 1] = means[0]                              # a duplicated centroid: exact ties, lowest index must win
    data = np.ascontiguousarray(pts if layout == AOS else pts.T).ravel()
    mflat = np.ascontiguousarray(means if layout_means == AOS else means.T).ravel()
    oa = orc.assign(data, mflat, dim, k, n, layout, layout_means, threads=0, fast=True)
    om, osz = orc.update(data, oa, dim, k, n, layout, layout_means, threads=0)
    for variant in (km.FUSED_ONE_PASS, km.FUSED_BEST, km.FUSED_TWO_PASS):
        gm, gs = fused_step(km, variant, data, mflat, dim, k, n, layout, layout_means)
        assert np.array_equal(gs, osz), "variant %d" % variant
        assert rel_err(gm, om) < CENTROID_RTOL, "variant %d" % variant


@pytest.mark.gpu
@pytest.mark.parametrize("dim,k,n", [(16, 16, 200000), (4, 8, 100000), (32, 32, 60000), (7, 5, 50000)])
@pytest.mark.parametrize("offset", [30.0, 1000.0, -20000.0])
def test_single_pass_fused_kernel_far_from_the_origin(km, orc, gpu, dim, k, n, offset):
    """KMX_FUSED_ONE_PASS ranks in a frame moved to the middle of the centroids when they lie far from the origin, and sums
    the points as given: the serial counts, the centroids within tolerance of float64 means of the serial assignment."""
    rng = np.random.default_rng(dim * 17 + k)
    centres = rng.uniform(-10, 10, (k, dim)).astype(np.float32)
    pts = (centres[rng.integers(0, k, size=n)] + rng.normal(size=(n, dim)).astype(np.float32) + np.float32(offset)).astype(np.float32)
    means = pts[:k].copy()
    oa = orc.assign(pts.ravel(), means.ravel(), dim, k, n, threads=0, fast=True)
    osz = np.bincount(oa, minlength=k).astype(np.uint32)
    sums = np.zeros((k, dim)); np.add.at(sums, oa, pts.astype(np.float64))
    ref = np.where(osz[:, None] > 0, sums / np.maximum(osz, 1)[:, None], 0.0).ravel()
    for variant in (km.FUSED_ONE_PASS, km.FUSED_TWO_PASS):
        gm, gs = fused_step(km, variant, pts.ravel(), means.ravel(), dim, k, n)
        assert np.array_equal(gs, osz), "variant %d" % variant
        spread = float(np.sqrt(np.mean((ref.reshape(k, dim) - ref.reshape(k, dim).mean(axis=0)) ** 2)))
        # fp32 sums of coordinates about `offset`: their rounding is relative to the offset, not to the spread
        assert float(np.abs(gm - ref).max()) < CENTROID_RTOL * max(spread, abs(offset)), "variant %d" % variant


@pytest.mark.gpu
@pytest.mark.parametrize("dim,k", [(8, 16), (4, 16), (16, 20), (24, 10), (32, 32)])
def test_single_pass_fused_kernel_hard_inputs(km, orc, gpu, dim, k):
    """Near-ties of three centroids, coincident points, NaN / inf / huge / tiny values go through the exact pass and the
    fix-up kernel; a shape the single-pass kernel does not take is refused by name. Rows of 4 and 24 floats take the
    lane-per-point kernel, rows of 8, 16 and 32 the kernel that ranks on the matrix cores."""
    n = 4096
    rng = np.random.default_rng(77 + dim)
    base = rng.normal(size=(n, dim)).astype(np.float32)
    means = rng.normal(size=(k, dim)).astype(np.float32)
    cases = {}
    m = means.copy(); m[5] = m[3]; m[9] = m[3]
    cases["three_equal_centroids"] = (base, m)
    cases["all_centroids_identical"] = (base, np.repeat(means[:1], k, 0))
    cases["all_points_identical"] = (np.repeat(base[:1], n, 0), means)
    cases["grid_ties"] = (np.round(base * 2) / 2, np.round(means * 2) / 2)
    cases["huge"] = (base * np.float32(1e18), means * np.float32(1e18))
    cases["tiny"] = (base * np.float32(1e-25), means * np.float32(1e-25))
    m = means.copy(); m[4, 1] = np.nan
    cases["nan_centroid"] = (base, m)
    m = means.copy(); m[0, 0] = np.nan
    cases["nan_centroid_zero"] = (base, m)
    d = base.copy(); d[5, 0] = np.nan; d[9, dim - 1] = np.inf
    cases["nan_inf_points"] = (d, means)
    for name, (d, m) in cases.items():
        d = np.ascontiguousarray(d, dtype=np.float32).ravel()
        m = np.ascontiguousarray(m, dtype=np.float32).ravel()
        oa = orc.assign(d, m, dim, k, n, threads=0, fast=True)
        om, osz = orc.update(d, oa, dim, k, n, threads=0)
        gm, gs = fused_step(km, km.FUSED_ONE_PASS, d, m, dim, k, n)
        assert np.array_equal(gs, osz), name
        finite = np.isfinite(om)
        assert np.array_equal(np.isfinite(gm), finite), name
        # values against float64 means of the same assignment: the serial fp32 sum of thousands of equal rows (one
        # of the cases) carries more rounding error than the tolerance, the tree-shaped device sum does not
        sums = np.zeros((k, dim)); np.add.at(sums, oa, d.reshape(n, dim).astype(np.float64))
        with np.errstate(invalid="ignore", divide="ignore"):
            ref = np.where(osz[:, None] > 0, sums / np.maximum(osz, 1)[:, None], 0.0).ravel()
        if finite.any():
            scale = max(float(np.sqrt(np.mean(ref[finite] ** 2))), 1e-30)
            assert float(np.abs(gm[finite] - ref[finite]).max()) / scale < CENTROID_RTOL, name
    with pytest.raises(km.KmxError, match="single-pass"):
        fused_step(km, km.FUSED_ONE_PASS, np.zeros(64 * 40, np.float32), np.zeros(40 * 40, np.float32), 40, 40, 64)


@pytest.mark.gpu
@pytest.mark.parametrize("cid,n", [(2, 65536), (1, 65536), (5, 1 << 18)])
def test_recorded_iterations_are_correct_iterations(km, orc, gpu, cid, n):
    """Two ping-pong iterations recorded once and replayed. Two runs are not comparable bit for bit (the update's fp32
    summation order is not fixed), so every replayed run is checked the way the call-by-call loop is: its last iteration
    against the oracle fed with the centroids that iteration read (they are still in the other ping-pong buffer).
    The recording is made and replayed in several runs, with call-by-call work and synchronisations in between."""
    spec = km.baseline_config(cid)
    dim, k = spec.dim, spec.k
    data = km.generate_points(spec, n)
    means0 = km.first_k_means(spec)
    alg = km.HipKMeansAlgorithm(km.ASSIGN_BEST, km.UPDATE_ATOMIC_SHM)
    alg.initialize(dim, k, n, 8, data, means0)
    for iters in (7, 8, 3, 6):
        alg.reset(means0)
        alg.run(iters=iters, use_graph=True)
        read_means = alg.cu_means[1 - alg.last].read(np.float32, alg.means_size)
        ga, gm, gs = alg.getAssignment(), alg.getMeans(), alg.getClusterSizes()
        oa = orc.assign(data, read_means, dim, k, n, threads=0, fast=True)
        assert np.array_equal(ga, oa), "%d iterations: %d mismatches" % (iters, int((ga != oa).sum()))
        om, osz = orc.update(data, ga, dim, k, n, threads=0)
        assert np.array_equal(gs, osz)
        assert rel_err(gm, om) < CENTROID_RTOL
        alg.reset(means0)
        alg.run(iters=2)                      # call-by-call work between the recordings
    alg.cleanup()


@pytest.mark.gpu
def test_recording_refuses_what_cannot_be_recorded(km, gpu):
    buf = km.DeviceBuffer(4096)
    with pytest.raises(km.KmxError):
        with km.Graph() as g:
            buf.zero()
            km.sync()                          # waiting is refused while recording
    # the recording was closed by the context manager; the library is usable again
    with km.Graph() as g:
        buf.zero()
    g.launch()
    km.sync()
    assert not buf.read(np.uint32, 1024).any()
    g.destroy()
    # a call that would have to grow the work space is refused while recording
    dim, k, n = 16, 64, 4096
    rng = np.random.default_rng(3)
    d = km.DeviceBuffer(4 * n * dim); d.write(rng.normal(size=n * dim).astype(np.float32))
    m = km.DeviceBuffer(4 * k * dim); m.write(rng.normal(size=k * dim).astype(np.float32))
    a = km.DeviceBuffer(4 * n)
    km.check(km.hip_lib().kmx_shutdown())      # releases the work space
    with pytest.raises(km.KmxError):
        with km.Graph() as g:
            km.assign(km.ASSIGN_BEST, d, AOS, dim, m, AOS, dim, a, dim, k, n)
    km.assign(km.ASSIGN_BEST, d, AOS, dim, m, AOS, dim, a, dim, k, n)   # sizes the work space
    with km.Graph() as g:
        km.assign(km.ASSIGN_BEST, d, AOS, dim, m, AOS, dim, a, dim, k, n)
    g.launch()
    km.sync()
    g.destroy()
    for b in (buf, d, m, a):
        b.free()


@pytest.mark.gpu
@pytest.mark.parametrize("dim,k,n,layout", [(4, 1024, 1 << 16, AOS), (32, 256, 1 << 15, SOA), (64, 128, 1 << 14, AOS), (2, 16, 1 << 14, AOS),
                                                 (32, 2048, 1 << 16, AOS)])   # (the last one: centroids swept in two slices)
def test_reserved_work_space_is_enough(km, orc, gpu, dim, k, n, layout):
    """kmx_reserve_f32 on a released work space: the assignment and the update of that shape can then be recorded, which
    refuses every call that would have to allocate; the recorded pair gives the oracle's assignment and counts."""
    rng = np.random.default_rng(dim * 7 + k)
    rows = rng.normal(size=(n, dim)).astype(np.float32)
    cents = rows[rng.choice(n, k, replace=False)].copy()
    host = rows.ravel() if layout == AOS else rows.T.copy().ravel()
    stride = dim if layout == AOS else n
    d = km.DeviceBuffer(4 * n * dim); d.write(host)
    m = km.DeviceBuffer(4 * k * dim); m.write(cents.ravel())
    a = km.DeviceBuffer(4 * n); out = km.DeviceBuffer(4 * k * dim); sizes = km.DeviceBuffer(4 * k)
    km.sync()
    km.check(km.hip_lib().kmx_shutdown())
    km.reserve(km.ASSIGN_BEST, km.UPDATE_ATOMIC_SHM, layout, AOS, dim, k, n)
    with km.Graph() as g:
        km.assign(km.ASSIGN_BEST, d, layout, stride, m, AOS, dim, a, dim, k, n)
        km.update(km.UPDATE_ATOMIC_SHM, d, layout, stride, a, out, AOS, dim, sizes, dim, k, n)
    g.launch()
    km.sync()
    g.destroy()
    ga = a.read(np.uint32, n)
    oa = orc.assign(rows.ravel(), cents.ravel(), dim, k, n, threads=0, fast=True)
    assert np.array_equal(ga, oa)
    om, osz = orc.update(rows.ravel(), ga, dim, k, n, threads=0)
    assert np.array_equal(sizes.read(np.uint32, k), osz)
    assert rel_err(out.read(np.float32, k * dim), om) < CENTROID_RTOL
    for b in (d, m, a, out, sizes):
        b.free()
