/*
 * Portable seeded dataset generator for the k-means benchmark shapes (C ABI).
 *
 * Plays the role of generate_clustered_data()/prepare_means() in the reference
 * (experimental/k-means/k-means/headers/data.hpp:32-81), but for the benchmark
 * configurations this project is measured on: every point is a pure function of
 * (seed, point index, spec), built from integer hashing and IEEE-754 +,-,*,/,sqrt only,
 * so any machine produces the same bytes and any prefix of a dataset is itself the
 * dataset of a smaller N.
 */
#ifndef KMX_DATAGEN_H
#define KMX_DATAGEN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { KMX_GEN_MIXTURE_UNIFORM_CENTRES = 0,  /* centres ~ U[lo,hi]^d, points = centre + N(0,sigma) */
       KMX_GEN_UNIFORM = 1,                   /* points ~ U[lo,hi)^d, no cluster structure          */
       KMX_GEN_MIXTURE_NORMAL_CENTRES = 2 };  /* centres ~ N(0,centre_sigma)^d, points = centre + N(0,sigma) */

enum { KMX_GEN_WEIGHTS_EQUAL = 0, KMX_GEN_WEIGHTS_GEOMETRIC = 1 /* weight_j ~ 2^-j */ };

typedef struct kmx_dataset_spec {
	uint64_t seed;
	uint64_t n;          /* number of points of the full data set        */
	uint32_t dim;
	uint32_t k;          /* number of clusters asked of k-means          */
	uint32_t iterations; /* Lloyd iterations of the benchmark            */
	uint32_t kind;       /* KMX_GEN_*                                    */
	uint32_t weights;    /* KMX_GEN_WEIGHTS_*                            */
	uint32_t centres;    /* number of mixture centres (0 for uniform)    */
	double lo, hi;       /* range of centres (mixture) or points (uniform) */
	double centre_sigma; /* std. dev. of centre coordinates (kind 2)     */
	double sigma;        /* std. dev. of the noise around a centre       */
} kmx_dataset_spec;

/* Fills *spec with benchmark configuration id (1..5). Returns 0, or -1 for an unknown id. */
int kmx_gen_baseline_config(int id, kmx_dataset_spec* spec);

/*
 * Writes points [first, first+count) of the data set into out.
 * layout 0 = AoS: out[i*stride + d], layout 1 = SoA: out[d*stride + i], i = 0..count-1.
 * threads <= 0 selects all available cores. Returns 0, or -1 on a bad argument.
 */
int kmx_gen_points(const kmx_dataset_spec* spec, uint64_t first, uint64_t count,
                   int layout, size_t stride, float* out, int threads);

/* Initial centroids = the first k points of the data set ("init first"). */
int kmx_gen_first_k_means(const kmx_dataset_spec* spec, int layout, size_t stride, float* out);

/* FNV-1a 64-bit hash of a byte range (drift check for generated data sets). */
uint64_t kmx_fnv1a64(const void* bytes, size_t len);

#ifdef __cplusplus
}
#endif

#endif
