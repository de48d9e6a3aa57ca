/*
 * Portable seeded dataset generator (see datagen.h).
 *
 * Determinism rules: only 64-bit integer arithmetic and IEEE-754 double +,-,*,/,sqrt are
 * used (the natural logarithm needed by the Gaussian sampler is evaluated by a fixed series
 * below, not by libm), and the file must be compiled without floating-point contraction.
 * Every point owns a private random stream keyed by (seed, point index), so generation is
 * order-independent and can be split over threads or produced in slices.
 */
#include "datagen.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

typedef struct { uint64_t s; int has_spare; double spare; } stream_t;

static inline uint64_t splitmix64(uint64_t* s)
{
	uint64_t z = (*s += 0x9E3779B97F4A7C15ULL);
	z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
	z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
	return z ^ (z >> 31);
}

static inline void stream_init(stream_t* st, uint64_t seed, uint64_t key)
{
	uint64_t s = seed * 0xD1342543DE82EF95ULL + 0x632BE59BD9B4E019ULL * (key + 1);
	(void)splitmix64(&s);
	st->s = splitmix64(&s) ^ (seed << 32);
	st->has_spare = 0;
	st->spare = 0.0;
}

/* uniform in [0,1) with 53 random bits */
static inline double stream_uniform(stream_t* st)
{
	return (double)(splitmix64(&st->s) >> 11) * (1.0 / 9007199254740992.0);
}

/* ln(x) for normal positive doubles: x = m*2^e, m in [sqrt(1/2), sqrt(2)], ln m = 2 atanh((m-1)/(m+1)). */
static double det_log(double x)
{
	union { double d; uint64_t u; } v;
	v.d = x;
	int e = (int)((v.u >> 52) & 0x7FF) - 1023;
	v.u = (v.u & 0x000FFFFFFFFFFFFFULL) | 0x3FF0000000000000ULL;
	double m = v.d;
	if (m > 1.4142135623730951) { m *= 0.5; e += 1; }
	double z = (m - 1.0) / (m + 1.0);
	double z2 = z * z;
	double s = 1.0 / 29.0;
	for (int k = 27; k >= 1; k -= 2) s = s * z2 + 1.0 / (double)k;
	return 2.0 * z * s + (double)e * 0.6931471805599453;
}

/* standard normal by the Marsaglia polar method (pairs; the second value is kept for the next call) */
static double stream_normal(stream_t* st)
{
	if (st->has_spare) { st->has_spare = 0; return st->spare; }
	for (;;) {
		double u = 2.0 * stream_uniform(st) - 1.0;
		double v = 2.0 * stream_uniform(st) - 1.0;
		double s = u * u + v * v;
		if (s >= 1.0 || s < 1e-300) continue;
		double f = sqrt(-2.0 * det_log(s) / s);
		st->spare = v * f;
		st->has_spare = 1;
		return u * f;
	}
}

int kmx_gen_baseline_config(int id, kmx_dataset_spec* spec)
{
	if (!spec) return -1;
	memset(spec, 0, sizeof(*spec));
	spec->seed = (uint64_t)id;
	spec->weights = KMX_GEN_WEIGHTS_EQUAL;
	switch (id) {
	case 1: /* CPU-runnable plumbing */
		spec->n = 65536; spec->dim = 8; spec->k = 64; spec->iterations = 10;
		spec->kind = KMX_GEN_MIXTURE_UNIFORM_CENTRES; spec->centres = 64;
		spec->lo = -10.0; spec->hi = 10.0; spec->sigma = 1.0; break;
	case 2: /* headline */
		spec->n = 2097152; spec->dim = 32; spec->k = 1024; spec->iterations = 20;
		spec->kind = KMX_GEN_MIXTURE_UNIFORM_CENTRES; spec->centres = 1024;
		spec->lo = -10.0; spec->hi = 10.0; spec->sigma = 1.0; break;
	case 3: /* low-d / high-k, no cluster structure */
		spec->n = 4194304; spec->dim = 4; spec->k = 4096; spec->iterations = 20;
		spec->kind = KMX_GEN_UNIFORM; spec->centres = 0;
		spec->lo = 0.0; spec->hi = 1.0; break;
	case 4: /* high-d dense contraction */
		spec->n = 1048576; spec->dim = 256; spec->k = 1024; spec->iterations = 10;
		spec->kind = KMX_GEN_MIXTURE_NORMAL_CENTRES; spec->centres = 1024;
		spec->centre_sigma = 2.0; spec->sigma = 1.0; break;
	case 5: /* atomic-hot update stress, skewed weights */
		spec->n = 16777216; spec->dim = 16; spec->k = 16; spec->iterations = 20;
		spec->kind = KMX_GEN_MIXTURE_UNIFORM_CENTRES; spec->centres = 16;
		spec->weights = KMX_GEN_WEIGHTS_GEOMETRIC;
		spec->lo = -10.0; spec->hi = 10.0; spec->sigma = 0.5; break;
	default:
		return -1;
	}
	return 0;
}

static double* make_centres(const kmx_dataset_spec* spec)
{
	if (spec->kind == KMX_GEN_UNIFORM || spec->centres == 0) return NULL;
	size_t count = (size_t)spec->centres * spec->dim;
	double* c = (double*)malloc(count * sizeof(double));
	if (!c) return NULL;
	for (uint32_t j = 0; j < spec->centres; ++j) {
		stream_t st;
		stream_init(&st, spec->seed ^ 0xC3A5C85C97CB3127ULL, j); /* centre streams are disjoint from point streams */
		for (uint32_t d = 0; d < spec->dim; ++d) {
			double v;
			if (spec->kind == KMX_GEN_MIXTURE_UNIFORM_CENTRES)
				v = spec->lo + (spec->hi - spec->lo) * stream_uniform(&st);
			else
				v = spec->centre_sigma * stream_normal(&st);
			c[(size_t)j * spec->dim + d] = v;
		}
	}
	return c;
}

static uint32_t pick_centre(const kmx_dataset_spec* spec, double u)
{
	uint32_t K = spec->centres;
	if (spec->weights == KMX_GEN_WEIGHTS_GEOMETRIC) {
		/* weight_j = 2^-j / W, W = sum_{j<K} 2^-j; walk the cumulative distribution */
		double W = 0.0, w = 1.0;
		for (uint32_t j = 0; j < K; ++j) { W += w; w *= 0.5; }
		double t = u * W;
		w = 1.0;
		for (uint32_t j = 0; j + 1 < K; ++j) {
			if (t < w) return j;
			t -= w;
			w *= 0.5;
		}
		return K - 1;
	}
	uint32_t j = (uint32_t)(u * (double)K);
	return j < K ? j : K - 1;
}

static void gen_point(const kmx_dataset_spec* spec, const double* centres, uint64_t index, float* out, size_t step)
{
	stream_t st;
	stream_init(&st, spec->seed, index);
	if (spec->kind == KMX_GEN_UNIFORM) {
		for (uint32_t d = 0; d < spec->dim; ++d)
			out[d * step] = (float)(spec->lo + (spec->hi - spec->lo) * stream_uniform(&st));
		return;
	}
	uint32_t c = pick_centre(spec, stream_uniform(&st));
	const double* centre = centres + (size_t)c * spec->dim;
	for (uint32_t d = 0; d < spec->dim; ++d)
		out[d * step] = (float)(centre[d] + spec->sigma * stream_normal(&st));
}

int kmx_gen_points(const kmx_dataset_spec* spec, uint64_t first, uint64_t count,
                   int layout, size_t stride, float* out, int threads)
{
	if (!spec || !out || spec->dim == 0) return -1;
	if (layout == 0 && stride < spec->dim) return -1;
	if (layout == 1 && stride < count) return -1;
	if (layout != 0 && layout != 1) return -1;
	double* centres = make_centres(spec);
	if (!centres && spec->kind != KMX_GEN_UNIFORM) return -1;
#ifdef _OPENMP
	if (threads <= 0) threads = omp_get_max_threads();
#else
	threads = 1;
#endif
	(void)threads;
	int64_t total = (int64_t)count;
#ifdef _OPENMP
#pragma omp parallel for schedule(static) num_threads(threads)
#endif
	for (int64_t i = 0; i < total; ++i) {
		if (layout == 0)
			gen_point(spec, centres, first + (uint64_t)i, out + (size_t)i * stride, 1);
		else
			gen_point(spec, centres, first + (uint64_t)i, out + (size_t)i, stride);
	}
	free(centres);
	return 0;
}

int kmx_gen_first_k_means(const kmx_dataset_spec* spec, int layout, size_t stride, float* out)
{
	if (!spec) return -1;
	return kmx_gen_points(spec, 0, spec->k, layout, stride, out, 1);
}

uint64_t kmx_fnv1a64(const void* bytes, size_t len)
{
	const unsigned char* p = (const unsigned char*)bytes;
	uint64_t h = 0xCBF29CE484222325ULL;
	for (size_t i = 0; i < len; ++i) { h ^= p[i]; h *= 0x100000001B3ULL; }
	return h;
}
