"""The reference-compatible data set and initialisation of the k-means harness (host/datasets.hpp: generate_clustered_data,
prepare_means with shuffle; reference experimental/k-means/k-means/headers/data.hpp:32-81). The reference's header needs
bpplib and cannot be compiled here, so the bit stream of these two functions is NOT pinned against the reference; what the
procedure fixes mathematically is: the first k points are the centres, uniform in [0,1)^d; every later point is one of those
centres plus N(0, 0.025) noise per coordinate; the initial centroids are k distinct data rows chosen by a shuffle that
depends on the seed only; both layouts hold the same values; and the engine underneath is the standard's mt19937, whose
10000th output for the default seed the C++ standard itself states (4123659995)."""
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST = os.path.join(ROOT, "cuda-kmeans_amd", "host")

DRIVER = r"""
#include "datasets.hpp"
#include <cstdio>
#include <cstdlib>
#include <string>
template<typename T> static void dump(const std::string& path, const std::vector<T>& v)
{ std::FILE* f = std::fopen(path.c_str(), "wb"); std::fwrite(v.data(), sizeof(T), v.size(), f); std::fclose(f); }
template<class LAYOUT, class LAYOUT_MEANS> static void run(const std::string& prefix, std::size_t n, std::size_t k, std::size_t dim, std::size_t seed)
{
	std::vector<float> data, means;
	generate_clustered_data<float, LAYOUT>(data, n, k, dim, seed);
	prepare_means<float, std::uint32_t, LAYOUT, LAYOUT_MEANS>(data, means, n, k, dim, true, seed);
	dump(prefix + ".data", data);
	dump(prefix + ".means", means);
}
int main(int argc, char** argv)
{
	const std::string prefix = argv[1];
	const std::size_t n = std::strtoul(argv[2], 0, 10), k = std::strtoul(argv[3], 0, 10), dim = std::strtoul(argv[4], 0, 10), seed = std::strtoul(argv[5], 0, 10);
	run<AoSLayoutPolicy<1>, AoSLayoutPolicy<1>>(prefix + ".aos", n, k, dim, seed);
	run<SoALayoutPolicy<1>, SoALayoutPolicy<1>>(prefix + ".soa", n, k, dim, seed);
	std::mt19937 engine;                      /* default seed 5489 */
	engine.discard(9999);
	std::printf("%lu\n", (unsigned long)engine());
	return 0;
}
"""


@pytest.fixture(scope="module")
def driver(tmp_path_factory):
    d = tmp_path_factory.mktemp("refdata")
    src = d / "driver.cpp"
    src.write_text(DRIVER)
    exe = d / "driver"
    subprocess.check_call(["g++", "-O2", "-std=c++14", "-I", HOST, "-I", os.path.join(ROOT, "include"), str(src),
                           os.path.join(HOST, "datagen.c"), "-x", "none", "-o", str(exe), "-lm"])
    return str(exe), d


def generate(driver, n, k, dim, seed, tag):
    exe, d = driver
    prefix = str(d / tag)
    out = subprocess.check_output([exe, prefix, str(n), str(k), str(dim), str(seed)], text=True)
    load = lambda name: np.fromfile(prefix + name, dtype=np.float32)
    return dict(aos=load(".aos.data").reshape(n, dim), soa=load(".soa.data").reshape(dim, n).T,
                means_aos=load(".aos.means").reshape(k, dim), means_soa=load(".soa.means").reshape(dim, k).T, tenthousandth=int(out))


@pytest.mark.parametrize("n,k,dim,seed", [(4096, 16, 8, 42), (10240, 128, 20, 1), (3000, 7, 3, 5)])
def test_reference_data_set_properties(driver, n, k, dim, seed):
    g = generate(driver, n, k, dim, seed, "a%d" % seed)
    assert g["tenthousandth"] == 4123659995                    # [rand.predef]: the engine is the standard's mt19937
    pts = g["aos"]
    assert np.array_equal(pts, g["soa"])                       # both layouts hold the same values
    centres = pts[:k]
    assert centres.min() >= 0.0 and centres.max() < 1.0        # the first k points: uniform in [0,1)^d
    assert abs(float(centres.mean()) - 0.5) < 4 * np.sqrt(1 / 12 / centres.size)
    # every later point lies within 6 sigma (sigma = 0.025) per coordinate of one of the first k points
    rest = pts[k:]
    dist = np.abs(rest[:, None, :] - centres[None, :, :]).max(2)          # Chebyshev distance to every centre
    nearest = dist.argmin(1)
    assert float(dist.min(1).max()) < 6 * 0.025
    noise = rest - centres[nearest]
    assert abs(float(noise.std()) - 0.025) < 0.002 and abs(float(noise.mean())) < 0.002
    # centres are picked about uniformly
    counts = np.bincount(nearest, minlength=k)
    assert counts.min() > 0 and counts.max() < 3 * (n - k) / k + 20
    # initial centroids: k distinct rows of the data, the same rows in both layouts
    means = g["means_aos"]
    assert np.array_equal(means, g["means_soa"])
    rows = [np.nonzero((pts == m).all(1))[0] for m in means]
    assert all(r.size >= 1 for r in rows)
    assert len({int(r[0]) for r in rows}) == k
    assert not np.array_equal(means, pts[:k])                  # shuffled, not the first k


def test_reference_data_set_depends_on_the_seed_only(driver):
    a = generate(driver, 2048, 8, 4, 9, "s1")
    b = generate(driver, 2048, 8, 4, 9, "s2")
    c = generate(driver, 2048, 8, 4, 10, "s3")
    assert np.array_equal(a["aos"], b["aos"]) and np.array_equal(a["means_aos"], b["means_aos"])
    assert not np.array_equal(a["aos"], c["aos"]) and not np.array_equal(a["means_aos"], c["means_aos"])
    # the shuffle uses a generator of its own started from the seed: the chosen rows do not depend on the data values
    rows_a = [int(np.nonzero((a["aos"] == m).all(1))[0][0]) for m in a["means_aos"]]
    big = generate(driver, 2048, 8, 6, 9, "s4")                # other dimension, same n and seed: same rows
    rows_big = [int(np.nonzero((big["aos"] == m).all(1))[0][0]) for m in big["means_aos"]]
    assert rows_a == rows_big
