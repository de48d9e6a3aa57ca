/*
 * Input generation and result verification of the harness.
 *
 *   generate_benchmark_data / first_k_means   the five seeded benchmark data sets (portable generator, datagen.h)
 *   generate_clustered_data / prepare_means   the reference's own procedure: the first k points uniform in
 *                                             [0,1)^d are the centres, every other point is a centre plus
 *                                             N(0, 0.025) noise; initial centroids are k points picked by a
 *                                             shuffle (experimental/k-means/k-means/headers/data.hpp:32-81)
 *   verify_assignment / verify_means          the reference's checks (data.hpp:131-202): exact assignment,
 *                                             centroids within 0.1 each and 0.01 on average
 *   classify_mismatches / centroid_error      the stricter report of this build: every differing point is
 *                                             classified by the serial distances (near-tie below 1e-5
 *                                             relative or not), centroid error relative to the rms coordinate
 */
#ifndef KMX_HOST_DATASETS_HPP
#define KMX_HOST_DATASETS_HPP

#include "datagen.h"
#include "layouts.hpp"
#include "metrics.hpp"

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <iostream>
#include <limits>
#include <numeric>
#include <random>
#include <stdexcept>
#include <vector>

template<typename F, class LAYOUT>
void generate_benchmark_data(std::vector<F>& data, const kmx_dataset_spec& spec, std::size_t n)
{
	/* the portable generator writes fp32; for doubles the same values are widened (exactly) */
	std::vector<float> raw(LAYOUT::size(n, spec.dim), 0.0f);
	if (kmx_gen_points(&spec, 0, n, LAYOUT::ID, LAYOUT::precomputeConstants(n, spec.dim), raw.data(), 0) != 0)
		throw std::runtime_error("data generator rejected its arguments");
	data.assign(raw.begin(), raw.end());
}

/* initial centroids = the first k points ("--init first") */
template<typename F, class LAYOUT, class LAYOUT_MEANS>
void first_k_means(const std::vector<F>& data, std::vector<F>& means, std::size_t n, std::size_t k, std::size_t dim)
{
	means.assign(LAYOUT_MEANS::size(k, dim), F(0));
	const auto sd = LAYOUT::precomputeConstants(n, dim);
	const auto sm = LAYOUT_MEANS::precomputeConstants(k, dim);
	for (std::size_t i = 0; i < k; ++i)
		for (std::size_t d = 0; d < dim; ++d)
			LAYOUT_MEANS::at(means.data(), i, d, sm) = LAYOUT::at(data.data(), i, d, sd);
}

template<typename F, class LAYOUT>
void generate_clustered_data(std::vector<F>& data, std::size_t n, std::size_t k, std::size_t dim, std::size_t seed)
{
	std::mt19937 generator((unsigned int)seed);
	std::uniform_real_distribution<F> uniform(F(0), F(1));
	std::uniform_int_distribution<std::size_t> pick(0, k - 1);
	std::normal_distribution<F> noise(F(0), F(0.025));
	data.assign(LAYOUT::size(n, dim), F(0));
	const auto stride = LAYOUT::precomputeConstants(n, dim);
	for (std::size_t i = 0; i < k; ++i)
		for (std::size_t d = 0; d < dim; ++d) LAYOUT::at(data.data(), i, d, stride) = uniform(generator);
	for (std::size_t i = k; i < n; ++i) {
		const std::size_t centre = pick(generator);
		for (std::size_t d = 0; d < dim; ++d)
			LAYOUT::at(data.data(), i, d, stride) = noise(generator) + LAYOUT::at(data.data(), centre, d, stride);
	}
}

template<typename F, typename IDX_T, class LAYOUT, class LAYOUT_MEANS>
void prepare_means(const std::vector<F>& data, std::vector<F>& means, std::size_t n, std::size_t k, std::size_t dim, bool shuffle, std::size_t seed)
{
	std::vector<IDX_T> order(n);
	std::iota(order.begin(), order.end(), IDX_T(0));
	if (shuffle) {
		std::mt19937 generator((unsigned int)seed);
		std::shuffle(order.begin(), order.end(), generator);
	}
	means.assign(LAYOUT_MEANS::size(k, dim), F(0));
	const auto sd = LAYOUT::precomputeConstants(n, dim);
	const auto sm = LAYOUT_MEANS::precomputeConstants(k, dim);
	for (std::size_t i = 0; i < k; ++i)
		for (std::size_t d = 0; d < dim; ++d)
			LAYOUT_MEANS::at(means.data(), i, d, sm) = LAYOUT::at(data.data(), order[i], d, sd);
}

/* number of differing entries; the first ten are printed */
template<typename IDX_T>
std::size_t verify_assignment(const std::vector<IDX_T>& res, const std::vector<IDX_T>& correct, std::size_t n)
{
	if (res.size() != correct.size() || res.size() != n) {
		std::cerr << std::endl << "Error: assignment size mismatch (" << res.size() << " vs " << correct.size() << ", expected " << n << ")!" << std::endl;
		return n;
	}
	std::size_t errors = 0;
	for (std::size_t i = 0; i < n; ++i) {
		if (res[i] == correct[i]) continue;
		if (errors == 0) std::cerr << std::endl;
		if (++errors <= 10) std::cerr << "Error at [" << i << "]: " << res[i] << " != " << correct[i] << std::endl;
	}
	if (errors) std::cerr << "Total assignment errors found: " << errors << std::endl;
	return errors;
}

/* the reference's loose centroid check: every centroid within 0.1, 0.01 on average */
template<typename F, class LAYOUT>
std::size_t verify_means(const std::vector<F>& res, const std::vector<F>& correct, std::size_t dims, std::size_t k)
{
	if (res.size() != correct.size() || res.size() != LAYOUT::size(k, dims)) {
		std::cerr << std::endl << "Error: means size mismatch (" << res.size() << " vs " << correct.size() << ")!" << std::endl;
		return correct.size();
	}
	using METRIC = EuclideanMetricPolicy<F, LAYOUT, LAYOUT>;
	const auto stride = LAYOUT::precomputeConstants(k, dims);
	std::size_t errors = 0;
	F total = F(0);
	for (std::size_t i = 0; i < k; ++i) {
		const F dist = METRIC::distance(res.data(), i, stride, correct.data(), i, stride, dims);
		total += dist;
		if (!(dist <= F(0.1))) {
			if (errors == 0) std::cerr << std::endl;
			if (++errors <= 10) std::cerr << "Error at [" << i << "]: means dist is " << dist << std::endl;
		}
	}
	if (errors) std::cerr << "Total significant errors found: " << errors << std::endl;
	total /= (F)k;
	if (!(total <= F(0.01))) {
		++errors;
		std::cerr << "Average displacement of means is " << total << " !" << std::endl;
	}
	return errors;
}

/* max |a - b| over the centroid coordinates, relative to the rms coordinate of `correct` */
template<typename F, class LAYOUT>
double centroid_error(const std::vector<F>& res, const std::vector<F>& correct, std::size_t dims, std::size_t k)
{
	const auto stride = LAYOUT::precomputeConstants(k, dims);
	double sq = 0.0, worst = 0.0;
	for (std::size_t i = 0; i < k; ++i)
		for (std::size_t d = 0; d < dims; ++d) {
			const double c = LAYOUT::at(correct.data(), i, d, stride), r = LAYOUT::at(res.data(), i, d, stride);
			sq += c * c;
			worst = std::max(worst, std::abs(r - c));
		}
	const double rms = std::sqrt(sq / (double)(k * dims));
	return worst / std::max(rms, 1e-30);
}

struct MismatchReport {
	std::size_t mismatches = 0; /* points whose assignment differs            */
	std::size_t nearTies = 0;   /* of these: best and second-best serial distance closer than 1e-5 relative */
};

/* classifies the points where res != correct using the serial distances to `means` (the centroids both were assigned against) */
template<typename F, typename IDX_T, class LAYOUT, class LAYOUT_MEANS>
MismatchReport classify_mismatches(const std::vector<IDX_T>& res, const std::vector<IDX_T>& correct, const std::vector<F>& data,
	const std::vector<F>& means, std::size_t dim, std::size_t k, std::size_t n)
{
	using METRIC = EuclideanMetricPolicy<F, LAYOUT, LAYOUT_MEANS>;
	const auto sd = LAYOUT::precomputeConstants(n, dim);
	const auto sm = LAYOUT_MEANS::precomputeConstants(k, dim);
	MismatchReport report;
	for (std::size_t i = 0; i < n; ++i) {
		if (res[i] == correct[i]) continue;
		++report.mismatches;
		F best = std::numeric_limits<F>::infinity(), second = best;
		for (std::size_t m = 0; m < k; ++m) {
			const F dist = METRIC::distance(data.data(), i, sd, means.data(), m, sm, dim);
			if (dist < best) { second = best; best = dist; }
			else if (dist < second) second = dist;
		}
		if (second - best <= F(1e-5) * second) ++report.nearTies;
	}
	return report;
}

#endif
