"""Pins the CPU oracle (oracle/serial_oracle.c) -- runs everywhere, no GPU.

1. golden vectors written by the reference's own SerialKMeansAlgorithm / SerialAssignmentAlgorithm
   (tests/golden/golden.npz, made by tests/golden/make_golden.py) -- bit for bit;
2. the reference build itself (oracle/_ref), where it exists, on shapes the fixtures do not hold;
3. what the mathematics fixes: float64 brute force on tiny inputs, closed forms (k = 1, duplicated
   centroids, empty clusters, NaN rules, order of the fp32 sums) chosen so that a dropped term, a
   fused multiply-add, a `>=` instead of `>` or a wrong summation order fails at least one of them.
"""
import json
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
AOS, SOA = 0, 1


@pytest.fixture(scope="module")
def golden():
    with open(os.path.join(HERE, "golden", "golden_index.json")) as f:
        index = json.load(f)
    arrays = np.load(os.path.join(HERE, "golden", "golden.npz"))
    return index, arrays


CASES = ["cfg1_full", "cfg1_soa_soa", "cfg1_aos_soa", "cfg1_soa_aos", "cfg2_small", "cfg3_small", "cfg4_small",
         "cfg5_small"]


@pytest.mark.parametrize("name", CASES)
def test_oracle_matches_reference_golden(km, orc, golden, name):
    index, arrays = golden
    c = index[name]
    spec = km.baseline_config(c["config"])
    data = km.generate_points(spec, c["n"], layout=c["layout"])
    assert "%016x" % km.fnv1a64(data) == c["data_fnv1a64"], "generator drift: inputs differ from the fixture's"
    means0 = km.first_k_means(spec, c["layout_means"])
    # scalar single-thread restatement on the cheap cases, the accelerated variant on all of them
    modes = [dict(threads=0, fast=True)]
    if c["n"] * c["k"] * c["dim"] * c["iterations"] < 3e9:
        modes.append(dict(threads=1, fast=False))
    for mode in modes:
        means, asg, sizes = orc.kmeans(data, means0, c["dim"], c["k"], c["n"], c["iterations"], c["layout"],
                                       c["layout_means"], **mode)
        assert np.array_equal(asg, arrays[name + "_assignment"].astype(np.uint32)), mode
        assert np.array_equal(sizes, arrays[name + "_counts"]), mode
        assert "%016x" % km.fnv1a64(means) == c["means_fnv1a64"], mode
        assert np.array_equal(means[:256], arrays[name + "_means_head"]), mode
    first = orc.assign(data, means0, c["dim"], c["k"], c["n"], c["layout"], c["layout_means"], threads=0, fast=True)
    assert np.array_equal(first, arrays[name + "_assignment_first_pass"].astype(np.uint32))


SHAPES = [(3, 5, 257), (20, 128, 1000), (7, 9, 130), (1, 2, 64), (33, 70, 500), (2, 300, 400)]


@pytest.mark.parametrize("dim,k,n", SHAPES)
@pytest.mark.parametrize("layout,layout_means", [(AOS, AOS), (SOA, AOS), (AOS, SOA), (SOA, SOA)])
def test_oracle_matches_reference_build(orc, dim, k, n, layout, layout_means):
    if orc.ref_lib() is None:
        pytest.skip("oracle/_ref is only built where the reference tree exists")
    rng = np.random.default_rng(dim * 1000 + k)
    data = rng.normal(size=n * dim).astype(np.float32)
    means0 = rng.normal(size=k * dim).astype(np.float32)
    rm, ra = orc.ref_kmeans(data, means0, dim, k, n, 3, layout, layout_means)
    for mode in (dict(threads=1, fast=False), dict(threads=3, fast=False), dict(threads=2, fast=True)):
        om, oa, _ = orc.kmeans(data, means0, dim, k, n, 3, layout, layout_means, **mode)
        assert np.array_equal(oa, ra), mode
        assert np.array_equal(om.view(np.uint32), rm.view(np.uint32)), mode
    assert np.array_equal(orc.assign(data, means0, dim, k, n, layout, layout_means),
                          orc.ref_assign(data, means0, dim, k, n, layout, layout_means))


@pytest.mark.parametrize("dim,k,n", SHAPES)
def test_fast_variant_is_bit_identical(orc, dim, k, n):
    rng = np.random.default_rng(7 + dim)
    data = rng.uniform(-3, 3, size=n * dim).astype(np.float32)
    means = rng.uniform(-3, 3, size=k * dim).astype(np.float32)
    a0, b0, s0 = orc.assign(data, means, dim, k, n, detail=True)
    a1, b1, s1 = orc.assign(data, means, dim, k, n, threads=4, fast=True, detail=True)
    assert np.array_equal(a0, a1)
    assert np.array_equal(b0.view(np.uint32), b1.view(np.uint32))
    assert np.array_equal(s0.view(np.uint32), s1.view(np.uint32))


def _f32_distance_unfused(x, c):
    """sqrt(sum (x-c)^2) with every operation rounded to fp32 separately, d ascending."""
    s = np.float32(0)
    for xd, cd in zip(x, c):
        diff = np.float32(xd) - np.float32(cd)
        s = np.float32(s + np.float32(diff * diff))
    return np.sqrt(s, dtype=np.float32)


def test_distance_is_unfused_fp32_in_dimension_order(orc):
    # values chosen so that fusing the multiply-add, or summing in another order, changes the result bits
    rng = np.random.default_rng(11)
    dim, k, n = 13, 4, 200
    data = (rng.normal(size=n * dim) * 1e3).astype(np.float32)
    means = (rng.normal(size=k * dim) * 1e3).astype(np.float32)
    asg, best, second = orc.assign(data, means, dim, k, n, detail=True)
    fused_differs = 0
    for i in range(n):
        d = np.array([_f32_distance_unfused(data[i * dim:(i + 1) * dim], means[j * dim:(j + 1) * dim]) for j in range(k)])
        j = int(asg[i])
        assert best[i].view(np.uint32) == d[j].view(np.uint32)
        assert j == int(np.argmin(d))  # argmin returns the first minimum = strict comparison from centroid 0
        assert second[i] == np.min(np.delete(d, j))
        exact = np.sqrt(np.sum((data[i * dim:(i + 1) * dim].astype(np.float64) - means[j * dim:(j + 1) * dim]) ** 2))
        fused_differs += int(np.float32(exact).view(np.uint32) != best[i].view(np.uint32))
    assert fused_differs > 0, "test vectors too tame: rounding order would not be visible"


def test_float64_brute_force_disagreements_are_near_ties(orc):
    rng = np.random.default_rng(3)
    dim, k, n = 6, 50, 1000
    data = rng.uniform(0, 1, size=(n, dim)).astype(np.float32)
    means = rng.uniform(0, 1, size=(k, dim)).astype(np.float32)
    asg = orc.assign(data.ravel(), means.ravel(), dim, k, n)
    d = np.sqrt(((data[:, None, :].astype(np.float64) - means[None, :, :]) ** 2).sum(-1))
    exact = d.argmin(1)
    wrong = np.nonzero(asg != exact)[0]
    for i in wrong:
        assert abs(d[i, asg[i]] - d[i, exact[i]]) <= 1e-6 * d[i, exact[i]]
    assert wrong.size < n // 100


def test_ties_go_to_the_lowest_index(orc):
    dim, k, n = 4, 6, 32
    rng = np.random.default_rng(5)
    means = rng.normal(size=(k, dim)).astype(np.float32)
    means[4] = means[1]          # duplicated centroid
    means[5] = means[1]
    data = np.repeat(means[1][None, :], n, 0) + rng.normal(size=(n, dim)).astype(np.float32) * np.float32(1e-3)
    asg = orc.assign(np.ascontiguousarray(data).ravel(), means.ravel(), dim, k, n)
    assert np.all(asg == 1)
    # points sitting exactly on centroids: distance 0 to the first copy
    asg = orc.assign(means.ravel().copy(), means.ravel(), dim, k, k)
    assert list(asg) == [0, 1, 2, 3, 1, 1]


def test_sqrt_collisions_are_ties(orc):
    """Two different fp32 squared distances whose fp32 square roots coincide are a tie: the lower
    index wins although the higher one is strictly closer (the reference compares after the sqrt)."""
    rng = np.random.default_rng(17)
    found = False
    for _ in range(20000):
        u = np.float32(rng.uniform(1, 2))
        v = np.nextafter(u, np.float32(0))
        su = np.float32(np.float32(1) + np.float32(u * u))
        sv = np.float32(np.float32(1) + np.float32(v * v))
        if su != sv and np.sqrt(su, dtype=np.float32) == np.sqrt(sv, dtype=np.float32):
            found = True
            break
    assert found, "no colliding pair found"
    x = np.zeros(2, dtype=np.float32)
    means = np.array([1, u, 1, v], dtype=np.float32)  # centroid 1 is strictly closer in squared distance
    asg, best, second = orc.assign(x, means, 2, 2, 1, detail=True)
    assert asg[0] == 0 and best[0] == second[0]


def test_nan_rules(orc):
    dim, k, n = 3, 4, 3
    means = np.arange(k * dim, dtype=np.float32)
    data = np.array([0, 1, 2, np.nan, 4, 5, 9, 10, 11], dtype=np.float32)
    asg = orc.assign(data, means, dim, k, n)
    assert list(asg) == [0, 0, 3]            # a NaN point never leaves centroid 0
    means2 = means.copy()
    means2[3 * dim] = np.nan                  # NaN centroid (index 3) is never chosen
    assert list(orc.assign(data, means2, dim, k, n)) == [0, 0, 2]
    means3 = means.copy()
    means3[0] = np.nan                        # NaN centroid 0 keeps everything
    assert list(orc.assign(data, means3, dim, k, n)) == [0, 0, 0]


def test_update_closed_forms(orc):
    rng = np.random.default_rng(9)
    dim, n = 5, 1000
    data = (rng.normal(size=(n, dim)) * 100).astype(np.float32)
    # k = 1: the centroid is the fp32 sequential mean in point order
    means, sizes = orc.update(data.ravel(), np.zeros(n, dtype=np.uint32), dim, 1, n)
    acc = np.zeros(dim, dtype=np.float32)
    for i in range(n):
        acc = (acc + data[i]).astype(np.float32)
    assert sizes[0] == n
    assert np.array_equal(means, (acc / np.float32(n)).astype(np.float32))
    rev = np.zeros(dim, dtype=np.float32)
    for i in reversed(range(n)):
        rev = (rev + data[i]).astype(np.float32)
    assert not np.array_equal(acc, rev), "test vectors too tame: summation order would not be visible"
    assert np.allclose(means, data.astype(np.float64).mean(0), rtol=1e-5, atol=1e-4)
    # empty clusters stay at the origin; counts are the histogram
    k = 7
    asg = rng.integers(0, 5, size=n).astype(np.uint32)
    asg[asg == 2] = 3
    means, sizes = orc.update(data.ravel(), asg, dim, k, n, threads=3)
    assert np.array_equal(sizes, np.bincount(asg, minlength=k).astype(np.uint32))
    m = means.reshape(k, dim)
    assert np.all(m[2] == 0) and np.all(m[5] == 0) and np.all(m[6] == 0)
    for c in (0, 1, 3, 4):
        assert np.allclose(m[c], data[asg == c].astype(np.float64).mean(0), rtol=1e-5, atol=1e-4)
    # threaded update keeps the serial order of every sum
    m1, s1 = orc.update(data.ravel(), asg, dim, k, n, threads=1)
    assert np.array_equal(m1.view(np.uint32), means.view(np.uint32)) and np.array_equal(s1, sizes)


def test_driver_contract(orc):
    """getAssignment() is the assignment against the means BEFORE the last update (serial.hpp:89-96)."""
    rng = np.random.default_rng(21)
    dim, k, n, iters = 4, 8, 500, 3
    data = rng.normal(size=n * dim).astype(np.float32)
    m = data[:k * dim].copy()
    for _ in range(iters):
        prev = m
        asg = orc.assign(data, prev, dim, k, n)
        m, sizes = orc.update(data, asg, dim, k, n)
    fm, fa, fs = orc.kmeans(data, data[:k * dim].copy(), dim, k, n, iters)
    assert np.array_equal(fa, asg) and np.array_equal(fm, m) and np.array_equal(fs, sizes)
    assert int(fs.sum()) == n
