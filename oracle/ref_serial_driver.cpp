/*
 * TEST INFRASTRUCTURE ONLY -- C entry points around the reference's own serial k-means.
 *
 * This file contains no algorithm: it includes the reference's headers where they lie
 * (/root/reference/experimental/k-means/k-means/headers/serial.hpp, pulled in with -I by
 * oracle/Makefile) and instantiates SerialKMeansAlgorithm / SerialAssignmentAlgorithm for the
 * four layout combinations the reference's CLI can select (k-means.cpp:233-287, ALIGN = 1).
 * The resulting oracle/_ref/libref_serial.so is used to write and check golden vectors and,
 * when present, as the "reference" CPU baseline.
 */
#include "serial.hpp"

#include <cstddef>
#include <cstdint>
#include <cstring>
#include <vector>

namespace {

template<class LAYOUT, class LAYOUT_MEANS>
void kmeans(const float* data, const float* means, std::size_t dim, std::size_t k, std::size_t n, std::size_t iters,
	float* meansOut, std::uint32_t* assignmentOut)
{
	std::vector<float> d(data, data + LAYOUT::size(n, dim));
	std::vector<float> m(means, means + LAYOUT_MEANS::size(k, dim));
	SerialKMeansAlgorithm<float, std::uint32_t, LAYOUT, LAYOUT_MEANS> alg;
	alg.initialize(dim, k, n, iters, d, m);
	alg.run();
	const std::vector<float>& rm = alg.getMeans();
	const std::vector<std::uint32_t>& ra = alg.getAssignment();
	std::memcpy(meansOut, rm.data(), rm.size() * sizeof(float));
	std::memcpy(assignmentOut, ra.data(), ra.size() * sizeof(std::uint32_t));
	alg.cleanup();
}

template<class LAYOUT, class LAYOUT_MEANS>
void assign(const float* data, const float* means, std::size_t dim, std::size_t k, std::size_t n, std::uint32_t* assignmentOut)
{
	std::vector<float> d(data, data + LAYOUT::size(n, dim));
	std::vector<float> m(means, means + LAYOUT_MEANS::size(k, dim));
	SerialAssignmentAlgorithm<float, std::uint32_t, LAYOUT, LAYOUT_MEANS> alg;
	alg.initialize(dim, k, n, d, m);
	alg.run();
	const std::vector<std::uint32_t>& ra = alg.getAssignment();
	std::memcpy(assignmentOut, ra.data(), ra.size() * sizeof(std::uint32_t));
	alg.cleanup();
}

} // namespace

/* layout / layout_means: 0 = AoSLayoutPolicy<1>, 1 = SoALayoutPolicy<1> */
extern "C" int ref_serial_kmeans(const float* data, int layout, const float* means, int layout_means,
	std::size_t dim, std::size_t k, std::size_t n, std::size_t iters, float* meansOut, std::uint32_t* assignmentOut)
{
	using A = AoSLayoutPolicy<1>;
	using S = SoALayoutPolicy<1>;
	if (layout == 0 && layout_means == 0) kmeans<A, A>(data, means, dim, k, n, iters, meansOut, assignmentOut);
	else if (layout == 0 && layout_means == 1) kmeans<A, S>(data, means, dim, k, n, iters, meansOut, assignmentOut);
	else if (layout == 1 && layout_means == 0) kmeans<S, A>(data, means, dim, k, n, iters, meansOut, assignmentOut);
	else if (layout == 1 && layout_means == 1) kmeans<S, S>(data, means, dim, k, n, iters, meansOut, assignmentOut);
	else return -1;
	return 0;
}

extern "C" int ref_serial_assign(const float* data, int layout, const float* means, int layout_means,
	std::size_t dim, std::size_t k, std::size_t n, std::uint32_t* assignmentOut)
{
	using A = AoSLayoutPolicy<1>;
	using S = SoALayoutPolicy<1>;
	if (layout == 0 && layout_means == 0) assign<A, A>(data, means, dim, k, n, assignmentOut);
	else if (layout == 0 && layout_means == 1) assign<A, S>(data, means, dim, k, n, assignmentOut);
	else if (layout == 1 && layout_means == 0) assign<S, A>(data, means, dim, k, n, assignmentOut);
	else if (layout == 1 && layout_means == 1) assign<S, S>(data, means, dim, k, n, assignmentOut);
	else return -1;
	return 0;
}
