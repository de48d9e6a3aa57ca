/*
 * TEST INFRASTRUCTURE ONLY -- C entry points around the reference's own serial k-means.
 *
 * This file contains no algorithm: it includes the reference's headers where they lie
 * (/root/reference/experimental/k-means/k-means/headers/serial.hpp, pulled in with -I by
 * oracle/Makefile) and instantiates SerialKMeansAlgorithm / SerialAssignmentAlgorithm for the
 * four layout combinations the reference's CLI can select (k-means.cpp:233-287, ALIGN = 1) and
 * both element types (float, and double as selected by --double, k-means.cpp:341-342).
 * The resulting oracle/_ref/libref_serial.so is used to write and check golden vectors and,
 * when present, as the "reference" CPU baseline.
 */
#include "serial.hpp"

#include <cstddef>
#include <cstdint>
#include <cstring>
#include <vector>

namespace {

template<typename F, class LAYOUT, class LAYOUT_MEANS>
void kmeans(const F* data, const F* means, std::size_t dim, std::size_t k, std::size_t n, std::size_t iters,
	F* meansOut, std::uint32_t* assignmentOut)
{
	std::vector<F> d(data, data + LAYOUT::size(n, dim));
	std::vector<F> m(means, means + LAYOUT_MEANS::size(k, dim));
	SerialKMeansAlgorithm<F, std::uint32_t, LAYOUT, LAYOUT_MEANS> alg;
	alg.initialize(dim, k, n, iters, d, m);
	alg.run();
	const std::vector<F>& rm = alg.getMeans();
	const std::vector<std::uint32_t>& ra = alg.getAssignment();
	std::memcpy(meansOut, rm.data(), rm.size() * sizeof(F));
	std::memcpy(assignmentOut, ra.data(), ra.size() * sizeof(std::uint32_t));
	alg.cleanup();
}

template<typename F, class LAYOUT, class LAYOUT_MEANS>
void assign(const F* data, const F* means, std::size_t dim, std::size_t k, std::size_t n, std::uint32_t* assignmentOut)
{
	std::vector<F> d(data, data + LAYOUT::size(n, dim));
	std::vector<F> m(means, means + LAYOUT_MEANS::size(k, dim));
	SerialAssignmentAlgorithm<F, std::uint32_t, LAYOUT, LAYOUT_MEANS> alg;
	alg.initialize(dim, k, n, d, m);
	alg.run();
	const std::vector<std::uint32_t>& ra = alg.getAssignment();
	std::memcpy(assignmentOut, ra.data(), ra.size() * sizeof(std::uint32_t));
	alg.cleanup();
}

/* layout / layout_means: 0 = AoSLayoutPolicy<1>, 1 = SoALayoutPolicy<1> */
template<typename F>
int kmeans_layouts(const F* data, int layout, const F* means, int layout_means,
	std::size_t dim, std::size_t k, std::size_t n, std::size_t iters, F* meansOut, std::uint32_t* assignmentOut)
{
	using A = AoSLayoutPolicy<1>;
	using S = SoALayoutPolicy<1>;
	if (layout == 0 && layout_means == 0) kmeans<F, A, A>(data, means, dim, k, n, iters, meansOut, assignmentOut);
	else if (layout == 0 && layout_means == 1) kmeans<F, A, S>(data, means, dim, k, n, iters, meansOut, assignmentOut);
	else if (layout == 1 && layout_means == 0) kmeans<F, S, A>(data, means, dim, k, n, iters, meansOut, assignmentOut);
	else if (layout == 1 && layout_means == 1) kmeans<F, S, S>(data, means, dim, k, n, iters, meansOut, assignmentOut);
	else return -1;
	return 0;
}

template<typename F>
int assign_layouts(const F* data, int layout, const F* means, int layout_means,
	std::size_t dim, std::size_t k, std::size_t n, std::uint32_t* assignmentOut)
{
	using A = AoSLayoutPolicy<1>;
	using S = SoALayoutPolicy<1>;
	if (layout == 0 && layout_means == 0) assign<F, A, A>(data, means, dim, k, n, assignmentOut);
	else if (layout == 0 && layout_means == 1) assign<F, A, S>(data, means, dim, k, n, assignmentOut);
	else if (layout == 1 && layout_means == 0) assign<F, S, A>(data, means, dim, k, n, assignmentOut);
	else if (layout == 1 && layout_means == 1) assign<F, S, S>(data, means, dim, k, n, assignmentOut);
	else return -1;
	return 0;
}

} // namespace

extern "C" int ref_serial_kmeans(const float* data, int layout, const float* means, int layout_means,
	std::size_t dim, std::size_t k, std::size_t n, std::size_t iters, float* meansOut, std::uint32_t* assignmentOut)
{
	return kmeans_layouts<float>(data, layout, means, layout_means, dim, k, n, iters, meansOut, assignmentOut);
}

extern "C" int ref_serial_assign(const float* data, int layout, const float* means, int layout_means,
	std::size_t dim, std::size_t k, std::size_t n, std::uint32_t* assignmentOut)
{
	return assign_layouts<float>(data, layout, means, layout_means, dim, k, n, assignmentOut);
}

extern "C" int ref_serial_kmeans_f64(const double* data, int layout, const double* means, int layout_means,
	std::size_t dim, std::size_t k, std::size_t n, std::size_t iters, double* meansOut, std::uint32_t* assignmentOut)
{
	return kmeans_layouts<double>(data, layout, means, layout_means, dim, k, n, iters, meansOut, assignmentOut);
}

extern "C" int ref_serial_assign_f64(const double* data, int layout, const double* means, int layout_means,
	std::size_t dim, std::size_t k, std::size_t n, std::uint32_t* assignmentOut)
{
	return assign_layouts<double>(data, layout, means, layout_means, dim, k, n, assignmentOut);
}
