"""The two-level split-bf16 sweep (rows of 17 to 32 and of 129 to 256 dimensions): one product per dimension for all points, three for those the
first level cannot settle, the exact pass for the rest. By default it runs from 2^18 points on; here it is forced
(kmx_set_two_level_sweep(2)) so that the inputs aimed at the certificates and the hard inputs of the other modules, which are
smaller, pass through both levels. Every result must be the serial scan's index, as with one level."""
import numpy as np
import pytest

import test_gpu_certificate as certificate_tests
import test_gpu_parity as parity_tests
import test_gpu_parity_f64 as parity_tests_f64

pytestmark = pytest.mark.gpu

AOS, SOA = 0, 1


@pytest.fixture
def two_levels(km):
    km.set_two_level_sweep(2)
    yield
    km.set_two_level_sweep(1)


@pytest.mark.parametrize("dim,k,n", [(32, 1024, 50000), (17, 130, 9000), (20, 100, 3000), (24, 700, 20000), (32, 33, 5000), (31, 4000, 30000),
                                     (32, 1056, 70000), (28, 64, 4097), (256, 1024, 20000), (200, 300, 9000), (129, 40, 3000), (256, 2100, 5000)])
@pytest.mark.parametrize("layout,layout_means", [(AOS, AOS), (SOA, SOA), (AOS, SOA)])
def test_assignment_is_bit_exact(km, orc, gpu, two_levels, dim, k, n, layout, layout_means):
    rng = np.random.default_rng(dim * 131 + k)
    centres = rng.uniform(-10, 10, size=(max(k // 3, 1), dim))            # three centroids per cluster: near-ties abound
    pts = (centres[rng.integers(0, centres.shape[0], size=n)] + rng.normal(size=(n, dim))).astype(np.float32)
    means = pts[:k].copy()
    data = np.ascontiguousarray(pts if layout == AOS else pts.T).ravel()
    cents = np.ascontiguousarray(means if layout_means == AOS else means.T).ravel()
    want = orc.assign(data, cents, dim, k, n, layout, layout_means, threads=0, fast=True)
    for v in (km.ASSIGN_MFMA_BF16X3, km.ASSIGN_BEST):
        got, rechecked = parity_tests.gpu_assign(km, v, data, cents, dim, k, n, layout, layout_means)
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, "variant %d: %d of %d points differ (first %s), %d went to the exact pass" % (v, bad.size, n, bad[:5], rechecked)
        assert rechecked < n // 4


def test_both_settings_return_the_same_and_the_first_level_settles_most_points(km, orc, gpu):
    """Configuration 2 (its first 2^18 points): the same assignment with one level and with two; the exact pass sees the
    same order of magnitude of points either way (what the second level cannot settle is what one level could not)."""
    spec = km.baseline_config(2)
    n, dim, k = 1 << 18, spec.dim, spec.k
    data, means0 = km.generate_points(spec, n), km.first_k_means(spec)
    want = orc.assign(data, means0, dim, k, n, threads=0, fast=True)
    counts = {}
    for mode in (0, 2, 1):
        km.set_two_level_sweep(mode)
        try:
            got, counts[mode] = parity_tests.gpu_assign(km, km.ASSIGN_BEST, data, means0, dim, k, n)
        finally:
            km.set_two_level_sweep(1)
        assert np.array_equal(got, want), "mode %d: %d mismatches" % (mode, int((got != want).sum()))
    assert counts[2] == counts[1] and abs(counts[2] - counts[0]) <= max(64, counts[0] // 2), counts


@pytest.mark.parametrize("dim,k,n", [(32, 256, 3000), (21, 1500, 4000), (32, 1024, 4096), (200, 160, 2000), (256, 300, 1500)])
def test_hard_inputs(km, orc, gpu, two_levels, dim, k, n):
    parity_tests.test_hard_inputs(km, orc, gpu, dim, k, n)


def test_worst_case_pairs_match_the_serial_scan(km, orc, gpu, two_levels):
    certificate_tests.test_worst_case_pairs_match_the_serial_scan(km, orc, gpu, 32)


@pytest.mark.parametrize("dim", [32, 256])
@pytest.mark.parametrize("offset", [0.0, 1e2, 1e4])
def test_gap_sweep(km, orc, gpu, two_levels, dim, offset):
    certificate_tests.test_gap_sweep(km, orc, gpu, dim, offset)


@pytest.mark.parametrize("dim", [32, 256])
def test_gap_sweep_with_coordinates_of_very_different_exponents(km, orc, gpu, two_levels, dim):
    certificate_tests.test_gap_sweep_with_coordinates_of_very_different_exponents(km, orc, gpu, dim)


@pytest.mark.parametrize("offset", [0.0, 100.0, 3000.0])
def test_data_far_from_the_origin(km, orc, gpu, two_levels, offset):
    parity_tests.test_data_far_from_the_origin(km, orc, gpu, 32, 1024, 200000, offset)


@pytest.mark.parametrize("layout,layout_means", [(AOS, AOS), (SOA, SOA)])
def test_doubles_ranked_in_two_levels(km, orc, gpu, two_levels, layout, layout_means):
    parity_tests_f64.test_assignment_is_bit_exact(km, orc, gpu, 32, 1000, 4099, layout, layout_means)
    parity_tests_f64.test_data_far_from_the_origin(km, orc, gpu, 32, 1024, 100000, 1000.0)


def test_every_iteration_matches_oracle(km, orc, gpu, two_levels):
    for r in parity_tests.forced_run(km, orc, 2, 65536, 4, km.ASSIGN_BEST, km.UPDATE_ATOMIC_SHM):
        assert r["mismatches"] == 0 and r["counts_equal"], r
