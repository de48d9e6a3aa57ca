/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the Lloyd iteration.
 *
 * A plain-C restatement of the reference's serial k-means
 * (experimental/k-means/k-means/headers/serial.hpp, metric_policies.hpp, layout_policies.hpp).
 * Only tests, the smoke check and the CPU-baseline leg of the benchmark may load this
 * library, and only as the checker; the product never links or calls it.
 *
 * Pinning (what each function is checked against, see tests/test_oracle.py):
 *   oracle_assign / oracle_update / oracle_kmeans -- bit-for-bit against golden vectors written
 *     by the reference's own SerialKMeansAlgorithm / SerialAssignmentAlgorithm compiled from
 *     /root/reference (tests/golden/), against that build directly when oracle/_ref exists,
 *     and against float64 brute force, closed forms (k=1 mean, duplicate centroids, empty
 *     clusters, NaN handling) on tiny inputs.
 *   The *_fast variants (SIMD across centroids, threads across points) perform the same
 *     per-element operation sequence and are checked bit-for-bit against the scalar functions.
 */
#ifndef KMX_SERIAL_ORACLE_H
#define KMX_SERIAL_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* layout: 0 = AoS (elem = idx*stride + dim), 1 = SoA (elem = dim*stride + idx);
 * layout_policies.hpp:22-25,46-49. */

/*
 * Nearest centroid of every point: sqrt(sum_d (x_d - c_d)^2) in fp32, d ascending, separate
 * multiply and add, strict comparison starting from centroid 0 (serial.hpp:21-42,
 * metric_policies.hpp:23-28,40-44). best_dist / second_dist (may be NULL) receive the
 * winning distance and the smallest distance among the other centroids (for near-tie
 * classification of mismatches). threads: 1 = the reference's single thread; >1 splits points.
 */
void oracle_assign(const float* data, int layout, size_t stride,
                   const float* means, int layout_means, size_t stride_means,
                   uint32_t dim, uint32_t k, uint32_t n,
                   uint32_t* assignment, float* best_dist, float* second_dist, int threads);

/* Same results as oracle_assign, evaluated 8 centroids at a time with identical per-lane arithmetic. */
void oracle_assign_fast(const float* data, int layout, size_t stride,
                        const float* means, int layout_means, size_t stride_means,
                        uint32_t dim, uint32_t k, uint32_t n,
                        uint32_t* assignment, float* best_dist, float* second_dist, int threads);

/*
 * Centroid update: zero, count, sum members in ascending point order in fp32, divide by
 * (float)count, leave empty clusters at zero (serial.hpp:44-73). threads > 1 splits the
 * clusters over threads; every sum keeps the ascending point order.
 */
void oracle_update(const float* data, int layout, size_t stride, const uint32_t* assignment,
                   float* means, int layout_means, size_t stride_means, uint32_t* cluster_sizes,
                   uint32_t dim, uint32_t k, uint32_t n, int threads);

/*
 * iters x (swap means; assign against the previous means; update) (serial.hpp:89-96).
 * means: in = initial centroids, out = centroids after the last update; assignment = the one
 * computed in the last iteration (against the centroids before the last update).
 * fast != 0 uses oracle_assign_fast. means_size = number of floats in the means array.
 */
void oracle_kmeans(const float* data, int layout, size_t stride,
                   float* means, int layout_means, size_t stride_means, size_t means_size,
                   uint32_t dim, uint32_t k, uint32_t n, uint32_t iters,
                   uint32_t* assignment, uint32_t* cluster_sizes, int threads, int fast);

/*
 * The same three functions for F = double, the reference's --double instantiation
 * (k-means.cpp:341-342; serial.hpp and metric_policies.hpp are templates over F). Pinned like the
 * float functions: golden vectors written by the reference's SerialKMeansAlgorithm<double, ...>,
 * that build directly when oracle/_ref exists, brute force with extended precision on tiny inputs.
 */
void oracle_assign_f64(const double* data, int layout, size_t stride,
                       const double* means, int layout_means, size_t stride_means,
                       uint32_t dim, uint32_t k, uint32_t n,
                       uint32_t* assignment, double* best_dist, double* second_dist, int threads);
void oracle_update_f64(const double* data, int layout, size_t stride, const uint32_t* assignment,
                       double* means, int layout_means, size_t stride_means, uint32_t* cluster_sizes,
                       uint32_t dim, uint32_t k, uint32_t n, int threads);
void oracle_kmeans_f64(const double* data, int layout, size_t stride,
                       double* means, int layout_means, size_t stride_means, size_t means_size,
                       uint32_t dim, uint32_t k, uint32_t n, uint32_t iters,
                       uint32_t* assignment, uint32_t* cluster_sizes, int threads);

#ifdef __cplusplus
}
#endif

#endif
