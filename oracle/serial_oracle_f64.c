/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the Lloyd iteration on doubles (see serial_oracle.h).
 *
 * The reference's serial k-means is a template over the element type F
 * (experimental/k-means/k-means/headers/serial.hpp:12, metric_policies.hpp:11); its --double
 * switch instantiates everything with F = double (k-means.cpp:341-342). This file restates that
 * instantiation in plain C: same operation order as the float functions in serial_oracle.c, every
 * float replaced by double. Compiled with -ffp-contract=off like the rest of the oracle.
 */
#include "serial_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* layout_policies.hpp:22-25 (SoA: dim*stride + idx), :46-49 (AoS: idx*stride + dim) */
static inline size_t at(int layout, size_t stride, size_t idx, size_t dim)
{
	return layout == 0 ? idx * stride + dim : dim * stride + idx;
}

/* metric_policies.hpp:17-30 (squared) and :33-47 (sqrt of it), F = double */
static inline double distance(const double* data, int layout, size_t stride, size_t idx,
                              const double* means, int layout_means, size_t stride_means, size_t m, uint32_t dim)
{
	double sum = 0.0;
	for (uint32_t d = 0; d < dim; ++d) {
		double dist = data[at(layout, stride, idx, d)] - means[at(layout_means, stride_means, m, d)];
		sum += dist * dist;
	}
	return sqrt(sum);
}

static inline int clamp_threads(int threads)
{
#ifdef _OPENMP
	if (threads <= 0) threads = omp_get_max_threads();
	return threads;
#else
	(void)threads;
	return 1;
#endif
}

/* serial.hpp:21-35 findNearestMean (strict `minDist > dist`, start at centroid 0), :37-42 computeAssignment */
void oracle_assign_f64(const double* data, int layout, size_t stride,
                       const double* means, int layout_means, size_t stride_means,
                       uint32_t dim, uint32_t k, uint32_t n,
                       uint32_t* assignment, double* best_dist, double* second_dist, int threads)
{
	threads = clamp_threads(threads);
	(void)threads;
#ifdef _OPENMP
#pragma omp parallel for schedule(static) num_threads(threads) if (threads > 1)
#endif
	for (int64_t i = 0; i < (int64_t)n; ++i) {
		uint32_t nearest = 0;
		double minDist = distance(data, layout, stride, (size_t)i, means, layout_means, stride_means, 0, dim);
		double second = INFINITY;
		for (uint32_t m = 1; m < k; ++m) {
			double dist = distance(data, layout, stride, (size_t)i, means, layout_means, stride_means, m, dim);
			if (minDist > dist) {
				if (second > minDist) second = minDist;
				minDist = dist;
				nearest = m;
			}
			else if (second > dist) {
				second = dist;
			}
		}
		assignment[i] = nearest;
		if (best_dist) best_dist[i] = minDist;
		if (second_dist) second_dist[i] = second;
	}
}

/* serial.hpp:44-73 updateMeans */
void oracle_update_f64(const double* data, int layout, size_t stride, const uint32_t* assignment,
                       double* means, int layout_means, size_t stride_means, uint32_t* cluster_sizes,
                       uint32_t dim, uint32_t k, uint32_t n, int threads)
{
	threads = clamp_threads(threads);
	if ((uint32_t)threads > k) threads = (int)k;
	for (uint32_t i = 0; i < k; ++i) {
		cluster_sizes[i] = 0;
		for (uint32_t d = 0; d < dim; ++d) means[at(layout_means, stride_means, i, d)] = 0.0;
	}
	/* ascending point order within every cluster (serial.hpp:57-63); thread t owns clusters c % threads == t */
#ifdef _OPENMP
#pragma omp parallel num_threads(threads) if (threads > 1)
#endif
	{
#ifdef _OPENMP
		uint32_t t = (uint32_t)omp_get_thread_num(), T = (uint32_t)omp_get_num_threads();
#else
		uint32_t t = 0, T = 1;
#endif
		for (uint32_t i = 0; i < n; ++i) {
			uint32_t target = assignment[i];
			if (T > 1 && target % T != t) continue;
			++cluster_sizes[target];
			for (uint32_t d = 0; d < dim; ++d)
				means[at(layout_means, stride_means, target, d)] += data[at(layout, stride, i, d)];
		}
	}
	for (uint32_t i = 0; i < k; ++i) {
		if (cluster_sizes[i] == 0) continue;
		double divisor = (double)cluster_sizes[i];
		for (uint32_t d = 0; d < dim; ++d) means[at(layout_means, stride_means, i, d)] /= divisor;
	}
}

/* serial.hpp:78-96 initialize + run */
void oracle_kmeans_f64(const double* data, int layout, size_t stride,
                       double* means, int layout_means, size_t stride_means, size_t means_size,
                       uint32_t dim, uint32_t k, uint32_t n, uint32_t iters,
                       uint32_t* assignment, uint32_t* cluster_sizes, int threads)
{
	double* prev = (double*)malloc(means_size * sizeof(double));
	if (!prev) abort();
	for (uint32_t iter = 0; iter < iters; ++iter) {
		memcpy(prev, means, means_size * sizeof(double)); /* mMeans.swap(mPrevMeans); the new means are rebuilt from zero */
		oracle_assign_f64(data, layout, stride, prev, layout_means, stride_means, dim, k, n, assignment, NULL, NULL, threads);
		oracle_update_f64(data, layout, stride, assignment, means, layout_means, stride_means, cluster_sizes, dim, k, n, threads);
	}
	free(prev);
}
