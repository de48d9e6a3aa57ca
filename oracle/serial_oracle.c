/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the Lloyd iteration (see serial_oracle.h).
 *
 * Restates experimental/k-means/k-means/headers/serial.hpp (reference) in plain C.
 * Must be compiled with -ffp-contract=off and without -mfma / -march=native so that every
 * multiply and add rounds separately, as in the reference's x86-64 baseline build
 * (experimental/k-means/k-means/Makefile:1-3).
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

/* metric_policies.hpp:17-30 (squared) and :33-47 (sqrt of it) */
static inline float distance(const float* data, int layout, size_t stride, size_t idx,
                             const float* means, int layout_means, size_t stride_means, size_t m, uint32_t dim)
{
	float sum = 0.0f;
	for (uint32_t d = 0; d < dim; ++d) {
		float dist = data[at(layout, stride, idx, d)] - means[at(layout_means, stride_means, m, d)];
		sum += dist * dist;
	}
	return sqrtf(sum);
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
void oracle_assign(const float* data, int layout, size_t stride,
                   const float* means, int layout_means, size_t stride_means,
                   uint32_t dim, uint32_t k, uint32_t n,
                   uint32_t* assignment, float* best_dist, float* second_dist, int threads)
{
	threads = clamp_threads(threads);
	(void)threads;
#ifdef _OPENMP
#pragma omp parallel for schedule(static) num_threads(threads) if (threads > 1)
#endif
	for (int64_t i = 0; i < (int64_t)n; ++i) {
		uint32_t nearest = 0;
		float minDist = distance(data, layout, stride, (size_t)i, means, layout_means, stride_means, 0, dim);
		float second = INFINITY;
		for (uint32_t m = 1; m < k; ++m) {
			float dist = distance(data, layout, stride, (size_t)i, means, layout_means, stride_means, m, dim);
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

/* ---- accelerated variant: 8 centroids per step, same per-lane operation sequence ---- */

typedef float v8f __attribute__((vector_size(32)));

static void assign_block(const float* x, const float* mt, uint32_t dim, uint32_t groups, uint32_t k,
                         uint32_t* out_idx, float* out_best, float* out_second)
{
	uint32_t nearest = 0;
	float minDist = 0.0f, second = INFINITY;
	for (uint32_t g = 0; g < groups; ++g) {
		const float* mg = mt + (size_t)g * dim * 8;
		v8f sum = { 0, 0, 0, 0, 0, 0, 0, 0 };
		for (uint32_t d = 0; d < dim; ++d) {
			v8f c;
			memcpy(&c, mg + (size_t)d * 8, sizeof(c));
			v8f xv = { x[d], x[d], x[d], x[d], x[d], x[d], x[d], x[d] };
			v8f diff = xv - c;
			v8f sq = diff * diff;
			sum = sum + sq;
		}
		float s[8];
		memcpy(s, &sum, sizeof(s));
		for (uint32_t l = 0; l < 8; ++l) {
			uint32_t m = g * 8 + l;
			if (m >= k) break;
			float dist = sqrtf(s[l]);
			if (m == 0) { minDist = dist; continue; }
			if (minDist > dist) {
				if (second > minDist) second = minDist;
				minDist = dist;
				nearest = m;
			}
			else if (second > dist) {
				second = dist;
			}
		}
	}
	*out_idx = nearest;
	*out_best = minDist;
	*out_second = second;
}

void oracle_assign_fast(const float* data, int layout, size_t stride,
                        const float* means, int layout_means, size_t stride_means,
                        uint32_t dim, uint32_t k, uint32_t n,
                        uint32_t* assignment, float* best_dist, float* second_dist, int threads)
{
	threads = clamp_threads(threads);
	uint32_t groups = (k + 7) / 8;
	/* repack the centroids as [group][dim][8] (values copied unchanged; padding lanes are never compared) */
	float* mt = (float*)calloc((size_t)groups * dim * 8, sizeof(float));
	if (!mt) abort();
	for (uint32_t m = 0; m < k; ++m)
		for (uint32_t d = 0; d < dim; ++d)
			mt[((size_t)(m / 8) * dim + d) * 8 + (m % 8)] = means[at(layout_means, stride_means, m, d)];

#ifdef _OPENMP
#pragma omp parallel num_threads(threads) if (threads > 1)
#endif
	{
		float* x = (float*)malloc((size_t)dim * sizeof(float));
		if (!x) abort();
#ifdef _OPENMP
#pragma omp for schedule(static)
#endif
		for (int64_t i = 0; i < (int64_t)n; ++i) {
			for (uint32_t d = 0; d < dim; ++d) x[d] = data[at(layout, stride, (size_t)i, d)];
			uint32_t idx;
			float b, s;
			assign_block(x, mt, dim, groups, k, &idx, &b, &s);
			assignment[i] = idx;
			if (best_dist) best_dist[i] = b;
			if (second_dist) second_dist[i] = s;
		}
		free(x);
	}
	free(mt);
}

/* serial.hpp:44-73 updateMeans */
void oracle_update(const float* data, int layout, size_t stride, const uint32_t* assignment,
                   float* means, int layout_means, size_t stride_means, uint32_t* cluster_sizes,
                   uint32_t dim, uint32_t k, uint32_t n, int threads)
{
	threads = clamp_threads(threads);
	if ((uint32_t)threads > k) threads = (int)k;
	/* clear (serial.hpp:49-54) */
	for (uint32_t i = 0; i < k; ++i) {
		cluster_sizes[i] = 0;
		for (uint32_t d = 0; d < dim; ++d) means[at(layout_means, stride_means, i, d)] = 0.0f;
	}
	/* accumulate in ascending point order (serial.hpp:57-63); thread t owns clusters c % threads == t */
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
	/* divide, empty clusters stay at zero (serial.hpp:66-72) */
	for (uint32_t i = 0; i < k; ++i) {
		if (cluster_sizes[i] == 0) continue;
		float divisor = (float)cluster_sizes[i];
		for (uint32_t d = 0; d < dim; ++d) means[at(layout_means, stride_means, i, d)] /= divisor;
	}
}

/* serial.hpp:78-96 initialize + run */
void oracle_kmeans(const float* data, int layout, size_t stride,
                   float* means, int layout_means, size_t stride_means, size_t means_size,
                   uint32_t dim, uint32_t k, uint32_t n, uint32_t iters,
                   uint32_t* assignment, uint32_t* cluster_sizes, int threads, int fast)
{
	float* prev = (float*)malloc(means_size * sizeof(float));
	if (!prev) abort();
	for (uint32_t iter = 0; iter < iters; ++iter) {
		memcpy(prev, means, means_size * sizeof(float)); /* mMeans.swap(mPrevMeans); the new means are rebuilt from zero */
		if (fast)
			oracle_assign_fast(data, layout, stride, prev, layout_means, stride_means, dim, k, n, assignment, NULL, NULL, threads);
		else
			oracle_assign(data, layout, stride, prev, layout_means, stride_means, dim, k, n, assignment, NULL, NULL, threads);
		oracle_update(data, layout, stride, assignment, means, layout_means, stride_means, cluster_sizes, dim, k, n, threads);
	}
	free(prev);
}
