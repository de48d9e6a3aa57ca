"""The double-precision functions of the CPU oracle (the reference's --double instantiation, F = double):

1. golden vectors written by the reference's own SerialKMeansAlgorithm<double, ...> /
   SerialAssignmentAlgorithm<double, ...> (tests/golden/golden_f64.npz, made by tests/golden/make_golden_f64.py)
   -- bit for bit;
2. that build itself where oracle/_ref exists, on random shapes and all layout pairs -- bit for bit;
3. what the mathematics fixes: the distance is the unfused double expression in dimension order (checked against
   numpy's own double arithmetic step by step), exact arithmetic on small integers, ties, NaN rules, update closed forms.
"""
import json
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
AOS, SOA = 0, 1


@pytest.fixture(scope="module")
def golden():
    with open(os.path.join(HERE, "golden", "golden_f64_index.json")) as f:
        index = json.load(f)
    return index, np.load(os.path.join(HERE, "golden", "golden_f64.npz"))


CASES = ["cfg1_f64", "cfg1_f64_soa_soa", "cfg1_f64_aos_soa", "cfg2_f64", "cfg3_f64", "cfg4_f64", "cfg5_f64"]


def golden_inputs(km, c):
    spec = km.baseline_config(c["config"])
    data = km.widen_points(km.generate_points(spec, c["n"], layout=c["layout"]))
    assert "%016x" % km.fnv1a64(data) == c["data_fnv1a64"], "generator drift: inputs differ from the fixture's"
    return data, km.widen_points(km.first_k_means(spec, c["layout_means"]))


@pytest.mark.parametrize("name", CASES)
def test_oracle_matches_reference_golden(km, orc, golden, name):
    index, arrays = golden
    c = index[name]
    data, means0 = golden_inputs(km, c)
    means, asg, sizes = orc.kmeans_f64(data, means0, c["dim"], c["k"], c["n"], c["iterations"], c["layout"],
                                       c["layout_means"], threads=0)
    assert np.array_equal(asg, arrays[name + "_assignment"].astype(np.uint32))
    assert np.array_equal(sizes, arrays[name + "_counts"])
    assert "%016x" % km.fnv1a64(means) == c["means_fnv1a64"]
    assert np.array_equal(means[:256].view(np.uint64), arrays[name + "_means_head"].view(np.uint64))
    first = orc.assign_f64(data, means0, c["dim"], c["k"], c["n"], c["layout"], c["layout_means"], threads=0)
    assert np.array_equal(first, arrays[name + "_assignment_first_pass"].astype(np.uint32))


@pytest.mark.parametrize("dim,k,n", [(3, 5, 257), (20, 128, 1000), (7, 9, 130), (1, 2, 64), (33, 70, 500)])
@pytest.mark.parametrize("layout,layout_means", [(AOS, AOS), (SOA, AOS), (AOS, SOA), (SOA, SOA)])
def test_oracle_matches_reference_build(orc, dim, k, n, layout, layout_means):
    if orc.ref_lib() is None or not hasattr(orc.ref_lib(), "ref_serial_kmeans_f64"):
        pytest.skip("oracle/_ref is only built where the reference tree exists")
    rng = np.random.default_rng(dim * 1000 + k)
    data = rng.normal(size=n * dim)
    means0 = rng.normal(size=k * dim)
    rm, ra = orc.ref_kmeans_f64(data, means0, dim, k, n, 3, layout, layout_means)
    for threads in (1, 3):
        om, oa, _ = orc.kmeans_f64(data, means0, dim, k, n, 3, layout, layout_means, threads=threads)
        assert np.array_equal(oa, ra), threads
        assert np.array_equal(om.view(np.uint64), rm.view(np.uint64)), threads
    assert np.array_equal(orc.assign_f64(data, means0, dim, k, n, layout, layout_means),
                          orc.ref_assign_f64(data, means0, dim, k, n, layout, layout_means))


def test_distance_is_unfused_double_in_dimension_order(orc):
    """numpy's float64 scalars round after every operation: the same sequence must give the same bits. A fused
    multiply-add, a float accumulator or another summation order would differ on these inputs."""
    rng = np.random.default_rng(5)
    dim, k, n = 37, 6, 40
    data = rng.normal(size=(n, dim)) * 1e3
    means = rng.normal(size=(k, dim)) * 1e3
    _, best, second = orc.assign_f64(data.ravel(), means.ravel(), dim, k, n, detail=True)
    want = np.empty((n, k))
    for i in range(n):
        for j in range(k):
            s = np.float64(0.0)
            for d in range(dim):
                diff = np.float64(data[i, d]) - np.float64(means[j, d])
                s = s + diff * diff
            want[i, j] = np.sqrt(s)
    srt = np.sort(want, axis=1)
    assert np.array_equal(best.view(np.uint64), srt[:, 0].copy().view(np.uint64))
    assert np.array_equal(second.view(np.uint64), srt[:, 1].copy().view(np.uint64))
    # the float oracle on the same values gives other bits: the accumulator really is a double
    _, best32, _ = orc.assign(data.astype(np.float32).ravel(), means.astype(np.float32).ravel(), dim, k, n, detail=True)
    assert not np.array_equal(best32.astype(np.float64), best)


def test_resolves_what_float_cannot(orc):
    """Two centroids whose distances to the point differ in the 40th bit: equal in float, ordered in double."""
    x = np.array([0.0, 0.0])
    means = np.array([1.0, 1.0, 1.0, 1.0 - 2.0 ** -40])   # centroid 1 is closer by 2^-40 in one coordinate
    assert orc.assign_f64(x, means, 2, 2, 1)[0] == 1
    assert orc.assign(x.astype(np.float32), means.astype(np.float32), 2, 2, 1)[0] == 0   # a tie in float: lowest index


def test_ties_nan_and_empty_clusters(orc):
    dim, k, n = 3, 4, 6
    data = np.arange(n * dim, dtype=np.float64)
    means = np.zeros(k * dim)
    means[3:6] = means[6:9] = data[3:6]           # centroids 1 and 2 coincide with point 1
    asg = orc.assign_f64(data, means, dim, k, n)
    assert asg[1] == 1                            # lowest index of the tie
    d = data.copy(); d[0] = np.nan
    assert orc.assign_f64(d, means, dim, k, n)[0] == 0   # NaN distances never win: the point stays on centroid 0
    m = means.copy(); m[3] = np.nan
    assert orc.assign_f64(data, m, dim, k, n)[1] == 2    # a NaN centroid (not 0) is never chosen
    m2, sizes = orc.update_f64(data, np.array([0, 0, 2, 2, 2, 0], dtype=np.uint32), dim, k, n)
    assert list(sizes) == [3, 0, 3, 0]
    assert np.array_equal(m2[3:6], np.zeros(3)) and np.array_equal(m2[9:12], np.zeros(3))   # empty clusters stay at zero
    assert np.array_equal(m2[0:3], (data[0:3] + data[3:6] + data[15:18]) / 3.0)             # point order, then divide


def test_update_sums_in_point_order(orc):
    """1e16 + 1 + 1 - 1e16 depends on the order: ascending point order gives 0 (each +1 is absorbed), any reordering
    that adds the ones first gives 2."""
    data = np.array([1e16, 1.0, 1.0, -1e16])
    means, sizes = orc.update_f64(data, np.zeros(4, dtype=np.uint32), 1, 1, 4)
    assert sizes[0] == 4 and means[0] == 0.0
    means, _ = orc.update_f64(np.array([1.0, 1.0, 1e16, -1e16]), np.zeros(4, dtype=np.uint32), 1, 1, 4)
    assert means[0] == 0.5  # the ones first: 2 + 1e16 is exact, minus 1e16 leaves 2, divided by the 4 members
