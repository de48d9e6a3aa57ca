/*
 * The Lloyd iteration on doubles: kmx_assign_f64, kmx_update_f64, kmx_fused_f64.
 *
 * The reference instantiates every algorithm with F = double when its command line says --double
 * (experimental/k-means/k-means/k-means.cpp:341-342; kernels.cu:1200-1261 instantiates the kernels for both types).
 *
 * Assignment. gfx950 executes the fp64 vector instructions at the rate of the plain fp32 ones.
 *   KMX_ASSIGN_BASE evaluates the serial arithmetic itself -- diff, square, add, in ascending dimension, sqrt, strict
 *   comparison from centroid 0 (serial.hpp:21-35, metric_policies.hpp:17-47) -- for every (point, centroid) pair: the
 *   result is the serial one by construction. One lane per point; the centroids come eight at a time from a
 *   transposed copy ([dim][k rounded up], written by a small kernel first), where the eight values of one dimension
 *   are one 64-byte scalar load and feed the subtractions as scalar operands. Rows of up to 32 doubles stay in
 *   registers for the whole sweep; longer rows are re-read per group of 32 centroids (L1/L2 hits).
 *     bound: 3 fp64 instructions (subtract, multiply, add: the serial code has no fused multiply-add) per point,
 *     centroid and dimension, one wavefront instruction per 4 cycles and SIMD: half of the fp64 peak, which counts FMAs.
 *     Measured at N = 2M, d = 32, k = 1024: 9 ms, 28 % of the peak, 57 % of that instruction bound.
 *   KMX_ASSIGN_LDS_FMA ranks the centroids by a_j = |c_j|^2 - 2 c_j.x with one fp64 FMA per element (same data
 *   flow), keeps the smallest and the second smallest a, and certifies the point when they differ by more than
 *   tau = (16 d + 48) u (|x|^2 + max_j |c_j|^2), u = 2^-53: the rounding errors of both ranking values (at most
 *   (d + 2) u (|x|^2 + |c|^2) each, with margin), the error of the serial sums and the width of a sqrt collision stay
 *   below it (the float kernels use the same bound with u = 2^-24), so no other centroid can win or tie the serial
 *   comparison. The other points (near-ties, duplicates, and every point when values overflow, underflow or are not
 *   numbers) are queued and re-evaluated by the BASE kernel over the queue. Measured: no faster than BASE -- with a
 *   64-bit scalar operand per instruction the sweep waits for scalar loads, not for the FMA pipeline.
 *   KMX_ASSIGN_MFMA / _MFMA_BF16X3 / _BEST use the float matrix-core sweeps as the ranking stage: points and centroids
 *   are rounded to float copies, the float sweep ranks and certifies them, and the BASE kernel re-evaluates the
 *   uncertified points on the doubles. The float certificate already covers the errors of float arithmetic on float
 *   inputs, a float serial sum and a float sqrt collision, all of which dominate their double counterparts; rounding
 *   the inputs moves a by at most 2^-23 (|c|^2 + 2 |c||x|) <= 2^-22 (|x|^2 + |c|^2) per ranking value, so the
 *   certificate is widened by 6 * 2^-23 (two values, with margin). Values beyond the float range become infinities or
 *   zeros, which the sweeps never certify (they require 1e-30 < |x|^2 + max |c|^2 and finite values).
 *   At N = 2M, d = 32, k = 1024 this is the float sweep's 0.4 ms plus two conversions instead of 8-9 ms.
 *
 * Update. One lane per element of the input (coalesced in either layout), as in the reference's updateAtomicFineKernel
 * (kernels.cu:770-809), with fp64 atomics, which gfx950 has natively in LDS and in L2: a work-group first adds into a
 * private copy of the sums in LDS when k * d doubles fit 32 KB and flushes it with one global atomic per element;
 * larger sums are split into ranges of clusters that fit, one work-group per (slice of the points, range); beyond 256
 * ranges, and for the POINT / FINE variants, the lanes add to global memory directly. Counts are
 * integer atomics issued by the lane of dimension 0.
 * The order of the additions is not the serial one (it is not in the reference's kernels either).
 */
#include "kmx_internal.h"
#include <type_traits>

#include <algorithm>

#pragma clang fp contract(off) /* every multiply and add rounds separately, as in the serial code */

namespace kmx {

constexpr int GROUP = 8;       /* centroids per step: 8 doubles = one s_load_dwordx16 */
constexpr int WIDE_GROUP = 32; /* the same for rows that are re-read per step */

static inline uint32_t round_up_u32(uint32_t v, uint32_t m) { return (v + m - 1) / m * m; }

/* work space of the double-precision calls: transposed centroids; owned by this file, released by kmx_shutdown
 * through release_f64_workspace() */
static double* g_means_t = nullptr;                /* [dim][kp] */
static size_t g_means_t_cap = 0;
static double* g_norms = nullptr;                  /* [kp]: |c|^2, +inf for the padding */
static size_t g_norms_cap = 0;
static double* g_queue = nullptr;                  /* n 32-bit point numbers (allocated in units of doubles) */
static size_t g_queue_cap = 0;
static double* g_misc = nullptr;                   /* 64-bit words: [0] queue length, [1] bits of max |c|^2 */
static size_t g_misc_cap = 0;
static double* g_data32 = nullptr;                 /* float copy of the points (same layout and stride) */
static size_t g_data32_cap = 0;
/* the points whose float copy g_data32 currently holds because the caller announced them with kmx_prepare_points_f64 and has
 * promised to leave them alone: kmx_assign_f64 then skips the conversion (null: nobody's) */
struct PreparedPoints {
	const double* data = nullptr;
	int layout = 0;
	size_t stride = 0;
	uint32_t dim = 0, n = 0;
	bool holds(const double* d, int l, size_t s, uint32_t dm, uint32_t nn) const { return data && data == d && layout == l && stride == s && dim == dm && n == nn; }
};
static PreparedPoints g_prepared;
static double* g_means32 = nullptr;                /* float copy of the centroids */
static size_t g_means32_cap = 0;
/* The float copies are taken of x - m and c - m, subtracted in double: m (dim doubles, then |m|^2) is the mean of the
 * first 16 points whose copy g_data32 holds. The float sweeps then rank data that lie around the origin whatever the
 * doubles do, and their certificate scales with the spread of the data (certificate.h); the exact pass takes their
 * thresholds back to the frame of the data in double. */
static double* g_frame = nullptr;
static size_t g_frame_cap = 0;

__global__ void reset_f64_kernel(unsigned long long* __restrict__ misc)
{
	if (threadIdx.x < 2) misc[threadIdx.x] = 0;
}

/* the count kmx_assign_last_rechecked() reports, for the variants that do not go through the float sweeps */
__global__ void publish_queue_length_kernel(const unsigned long long* __restrict__ misc, uint32_t* __restrict__ counters, bool queued)
{
	if (threadIdx.x == 0) counters[0] = queued ? (uint32_t)misc[0] : 0u;
}

/* m: a thread per dimension, the finite coordinates of the first 16 points; one work-group of 256 threads */
template <int LD>
__global__ void __launch_bounds__(256)
point_frame_f64_kernel(const double* __restrict__ data, size_t stride, uint32_t dim, uint32_t n, double* __restrict__ frame)
{
	__shared__ double parts[256 / WAVE];
	const uint32_t sample = min(n, 16u);
	double m2 = 0.0;
	for (uint32_t q = threadIdx.x; q < dim; q += blockDim.x) {
		double sum = 0.0;
		for (uint32_t r = 0; r < sample; ++r) {
			const double v = data[elem<LD>(stride, r, q)];
			sum += __builtin_fabs(v) < __builtin_inf() ? v : 0.0;
		}
		sum /= (double)sample;
		sum = __builtin_fabs(sum) < __builtin_inf() ? sum : 0.0;
		sum = (double)(float)sum; /* (a float's worth of m is enough, and x - m stays exact for more inputs) */
		sum = __builtin_fabs(sum) < __builtin_inf() ? sum : 0.0;
		frame[q] = sum;
		m2 = __builtin_fma(sum, sum, m2);
	}
	for (int off = WAVE / 2; off > 0; off >>= 1) m2 += __shfl_xor(m2, off);
	if ((threadIdx.x & (WAVE - 1)) == 0) parts[threadIdx.x / WAVE] = m2;
	__syncthreads();
	if (threadIdx.x == 0) frame[dim] = (parts[0] + parts[1]) + (parts[2] + parts[3]);
}

/* float copy of (in - m), subtracted in double (element e of a buffer with the layout and stride of the original) */
template <int LD>
__global__ void __launch_bounds__(256)
round_moved_to_float_kernel(const double* __restrict__ in, float* __restrict__ out, size_t count, size_t stride, uint32_t dim,
                            const double* __restrict__ frame)
{
	const bool narrow = count <= 0xFFFFFFFFull && stride <= 0xFFFFFFFFull; /* (32-bit division is several times cheaper) */
	for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < count; e += (size_t)gridDim.x * blockDim.x) {
		size_t q;
		if (narrow) q = LD == KMX_AOS ? (uint32_t)e % (uint32_t)stride : (uint32_t)e / (uint32_t)stride;
		else q = LD == KMX_AOS ? e % stride : e / stride;
		out[e] = (float)(q < dim ? in[e] - frame[q] : in[e]); /* (AoS rows may be padded) */
	}
}

/* one lane per (padded) centroid: transposed copy, |c|^2, and the largest |c|^2 as the maximum of the bit patterns
 * (non-negative doubles order like their bits; a NaN or an infinity ends up as the maximum and disables every
 * certificate, as it must) */
template <int LM>
__global__ void __launch_bounds__(256)
prepare_means_f64_kernel(const double* __restrict__ means, size_t stride_means, double* __restrict__ means_t,
                         double* __restrict__ norms, unsigned long long* __restrict__ misc, uint32_t dim, uint32_t k, uint32_t kp)
{
	const uint32_t j = blockIdx.x * blockDim.x + threadIdx.x;
	if (j >= kp) return;
	double c2 = 0.0;
	for (uint32_t q = 0; q < dim; ++q) {
		const double v = j < k ? means[elem<LM>(stride_means, j, q)] : 0.0;
		means_t[(size_t)q * kp + j] = v;
		c2 = __builtin_fma(v, v, c2);
	}
	norms[j] = j < k ? c2 : __builtin_inf();
	if (j < k) atomicMax(&misc[1], (unsigned long long)__double_as_longlong(c2 != c2 ? __builtin_nan("") : c2));
}

/* The same for AoS centroids: a work-group takes 32 centroids and turns their rows through LDS in tiles of 32 dimensions, so
 * that both the reads (along a row) and the writes (along the centroids) are contiguous; one lane per centroid walks the
 * tile for |c|^2, dimension by dimension in order. (One lane per centroid reading its own row, as above, took 56 us for 1024
 * rows of 256 doubles; this takes 21 us, and 6 instead of 12 us for rows of 32.) */
__global__ void __launch_bounds__(256)
prepare_rows_f64_kernel(const double* __restrict__ means, size_t stride_means, double* __restrict__ means_t,
                        double* __restrict__ norms, unsigned long long* __restrict__ misc, uint32_t dim, uint32_t k, uint32_t kp)
{
	__shared__ double tile[32][33];
	const uint32_t j0 = blockIdx.x * 32, tx = threadIdx.x % 32, ty = threadIdx.x / 32;
	double c2 = 0.0; /* lanes 0..31: centroid j0 + lane */
	for (uint32_t q0 = 0; q0 < dim; q0 += 32) {
#pragma unroll
		for (uint32_t r = 0; r < 4; ++r) {
			const uint32_t j = j0 + ty + 8 * r, q = q0 + tx;
			tile[ty + 8 * r][tx] = (j < k && q < dim) ? means[(size_t)j * stride_means + q] : 0.0;
		}
		__syncthreads();
#pragma unroll
		for (uint32_t r = 0; r < 4; ++r) {
			const uint32_t q = q0 + ty + 8 * r, j = j0 + tx;
			if (q < dim && j < kp) means_t[(size_t)q * kp + j] = tile[tx][ty + 8 * r];
		}
		if (threadIdx.x < 32) {
			for (uint32_t qq = 0; qq < min(32u, dim - q0); ++qq) {
				const double v = tile[threadIdx.x][qq];
				c2 = __builtin_fma(v, v, c2);
			}
		}
		__syncthreads();
	}
	const uint32_t j = j0 + threadIdx.x;
	if (threadIdx.x < 32 && j < kp) {
		norms[j] = j < k ? c2 : __builtin_inf();
		if (j < k) atomicMax(&misc[1], (unsigned long long)__double_as_longlong(c2 != c2 ? __builtin_nan("") : c2));
	}
}

/*
 * DPAD > 0: the row (dim <= DPAD) is held in registers; DPAD == 0: any dim, the row is re-read for every group of G
 * centroids (per-lane reads of an AoS row are not coalesced, so the wide rows take 32 centroids per read).
 * The comparison of the serial code is on sqrt(sum), and a correctly rounded double sqrt costs some 30 instructions.
 * sqrt is monotone, so a sum that is not below the best sum so far cannot give a smaller distance; and a sum below
 * the best one by more than a factor 1 - 2^-49 gives a distance at least two units in the last place smaller, which
 * no rounding can close: both cases are decided on the sums. Only a sum inside that band (a near-duplicate of the
 * best centroid so far, in practice never) takes both square roots, and wins only if its distance is smaller (two
 * sums may share their sqrt: then the lower index stays, as in the serial scan). Below 2^-900 the product that
 * forms the band's edge would lose bits, so every smaller sum counts as inside the band there.
 * NaN sums fail every comparison and never win, and a NaN at centroid 0 is never replaced: serial.hpp:21-35.
 */
template <int LD, int DPAD, int G>
__global__ void __launch_bounds__(256)
assign_f64_kernel(const double* __restrict__ data, size_t stride, const double* __restrict__ means_t,
                  uint32_t* __restrict__ assignment, uint32_t dim, uint32_t k, uint32_t kp, uint32_t n)
{
	const uint32_t total = n;
	for (uint32_t first = blockIdx.x * blockDim.x; first < total; first += gridDim.x * blockDim.x) {
	const uint32_t i = first + threadIdx.x;
	const uint32_t at = min(i, total - 1); /* lanes past the end repeat the last point and store nothing */
	const uint32_t pt = at;
	double x[DPAD > 0 ? DPAD : 1];
	if (DPAD > 0) {
#pragma unroll
		for (int q = 0; q < DPAD; ++q) x[q] = (uint32_t)q < dim ? data[elem<LD>(stride, pt, q)] : 0.0;
	}
	uint32_t nearest = 0;
	double best_sum = 0.0, sure_below = 0.0;
	auto band_edge = [](double s) { return s > 0x1p-900 ? s * (1.0 - 0x1p-49) : 0.0; };
	for (uint32_t g = 0; g < kp; g += G) {
		double sum[G];
#pragma unroll
		for (int j = 0; j < G; ++j) sum[j] = 0.0;
		if (DPAD > 0) {
#pragma unroll
			for (int q = 0; q < DPAD; ++q) {
				if ((uint32_t)q < dim) { /* uniform */
					const double* row = means_t + (size_t)q * kp + g; /* uniform address: scalar loads */
#pragma unroll
					for (int j = 0; j < G; ++j) {
						double diff = x[q] - row[j];
						double sq = diff * diff;
						sum[j] = sum[j] + sq;
					}
				}
			}
		}
		else {
#pragma unroll 2
			for (uint32_t q = 0; q < dim; ++q) {
				const double xq = data[elem<LD>(stride, pt, q)];
				const double* row = means_t + (size_t)q * kp + g;
#pragma unroll
				for (int j = 0; j < G; ++j) {
					double diff = xq - row[j];
					double sq = diff * diff;
					sum[j] = sum[j] + sq;
				}
			}
		}
#pragma unroll
		for (int j = 0; j < G; ++j) {
			const uint32_t m = g + j;
			if (m == 0) { best_sum = sum[0]; sure_below = band_edge(best_sum); }
			else if (m < k) { /* uniform */
				bool take = sum[j] < sure_below;
				if (__builtin_expect(!take && sum[j] < best_sum, 0)) take = __builtin_sqrt(best_sum) > __builtin_sqrt(sum[j]);
				if (take) { best_sum = sum[j]; sure_below = band_edge(best_sum); nearest = m; }
			}
		}
	}
	if (i < total) assignment[pt] = nearest;
	}
}

/*
 * The serial arithmetic for the few points a ranking stage could not certify. A lane per point would leave most of
 * the chip idle, so SPLIT lanes (2 for few centroids) share a point: each scans a contiguous range of the centroids (its own 64-byte
 * vector loads from the transposed copy) exactly like the kernel above, and the ranges are merged in ascending
 * order with the serial rule -- the later range wins only with a strictly smaller distance; NaN compares false, so
 * a NaN distance to centroid 0 stays and any other NaN never wins. Ranges that do not start at centroid 0 start
 * from +infinity with no centroid.
 */
template <int LD, int DPAD, int SPLIT>
__global__ void __launch_bounds__(256)
requeued_f64_kernel(const double* __restrict__ data, size_t stride, const double* __restrict__ means_t,
                    uint32_t* __restrict__ assignment, uint32_t dim, uint32_t k, uint32_t kp,
                    const uint32_t* __restrict__ queue, uint32_t queue_stride, const uint32_t* __restrict__ queue_length)
{
	constexpr uint32_t NONE = 0xffffffffu;
	const uint32_t total = *queue_length; /* the points listed in queue[queue_stride * (0 .. total)) */
	const uint32_t per_block = blockDim.x / SPLIT;
	const uint32_t sub = threadIdx.x % SPLIT;
	const uint32_t per = ((kp + SPLIT - 1) / SPLIT + GROUP - 1) / GROUP * GROUP; /* kp is a multiple of GROUP */
	const uint32_t j0 = min(sub * per, kp), j1 = min(j0 + per, kp);
	auto band_edge = [](double s) { return s > 0x1p-900 ? s * (1.0 - 0x1p-49) : 0.0; };
	for (uint32_t first = blockIdx.x * per_block; first < total; first += gridDim.x * per_block) {
		const uint32_t e = first + threadIdx.x / SPLIT;
		const uint32_t pt = queue[(size_t)min(e, total - 1) * queue_stride];
		double x[DPAD > 0 ? DPAD : 1];
		if (DPAD > 0) {
#pragma unroll
			for (int q = 0; q < DPAD; ++q) x[q] = (uint32_t)q < dim ? data[elem<LD>(stride, pt, q)] : 0.0;
		}
		uint32_t nearest = NONE;
		double best_sum = __builtin_inf(), sure_below = __builtin_inf();
		for (uint32_t g = j0; g < j1; g += GROUP) {
			double sum[GROUP];
#pragma unroll
			for (int j = 0; j < GROUP; ++j) sum[j] = 0.0;
			if (DPAD > 0) {
#pragma unroll
				for (int q = 0; q < DPAD; ++q) {
					if ((uint32_t)q < dim) { /* uniform */
						const double* row = means_t + (size_t)q * kp + g;
#pragma unroll
						for (int j = 0; j < GROUP; ++j) {
							double diff = x[q] - row[j];
							double sq = diff * diff;
							sum[j] = sum[j] + sq;
						}
					}
				}
			}
			else {
#pragma unroll 2
				for (uint32_t q = 0; q < dim; ++q) {
					const double xq = data[elem<LD>(stride, pt, q)];
					const double* row = means_t + (size_t)q * kp + g;
#pragma unroll
					for (int j = 0; j < GROUP; ++j) {
						double diff = xq - row[j];
						double sq = diff * diff;
						sum[j] = sum[j] + sq;
					}
				}
			}
#pragma unroll
			for (int j = 0; j < GROUP; ++j) {
				const uint32_t m = g + j;
				if (m == 0) { best_sum = sum[0]; sure_below = band_edge(best_sum); nearest = 0; }
				else if (m < k) {
					bool take = sum[j] < sure_below;
					if (__builtin_expect(!take && sum[j] < best_sum, 0)) take = __builtin_sqrt(best_sum) > __builtin_sqrt(sum[j]);
					if (take) { best_sum = sum[j]; sure_below = band_edge(best_sum); nearest = m; }
				}
			}
		}
		double dist = __builtin_sqrt(best_sum);
		for (int off = 1; off < SPLIT; off <<= 1) { /* lane l now speaks for the ranges of lanes l .. l + 2 off - 1 */
			const double other_dist = __shfl_down(dist, off, SPLIT);
			const uint32_t other = __shfl_down(nearest, off, SPLIT);
			if (sub + off < SPLIT && other != NONE && (nearest == NONE || dist > other_dist)) { dist = other_dist; nearest = other; }
		}
		if (sub == 0 && e < total) assignment[pt] = nearest;
	}
}

/*
 * The same for many centroids: four centroids per lane (a work-group of up to 256 lanes takes the centroids in chunks
 * of four times its size), a batch of 16 queued points in LDS, coordinate by coordinate side by side. For every dimension
 * a lane loads its centroids' coordinates once (coalesced) and applies them to the 16 points: one broadcast LDS read per
 * point serves four multiply-adds (with one centroid per lane the LDS reads, one per multiply-add, bounded the kernel),
 * and the centroids are read once per batch, not once per point. With thresholds from a float sweep the pairs that pass
 * the screen are noted and evaluated afterwards, one lane per pair (N = 1M doubles, d = 256, k = 1024, 9.4 k queued points:
 * 0.78 -> 0.36 ms with both changes; N = 2M, d = 32: 0.105 -> 0.055 ms).
 * The serial choice: the smallest distance by a 64-bit LDS minimum over the bit patterns (distances are non-negative, so
 * the patterns order like the values), then the lowest centroid number among those that hold exactly that distance;
 * without the list, chunks are merged in ascending order with a strict comparison. NaN distances take no part, except
 * that a NaN distance to centroid 0 pins the point there (serial.hpp:21-35).
 */
constexpr int BATCH = 16;
constexpr int BATCH_CPL = 4; /* centroids per lane: one broadcast read of a coordinate serves four multiply-adds */
constexpr int AHEAD = 2; /* dimensions between the request for the centroids' coordinates and their use (1: 13 % slower at d = 256, 4: level) */
constexpr uint32_t THRESHOLD_PARTS = 16; /* lanes that share a row when the thresholds are taken back (fewer in a work-group of fewer than 256) */
constexpr uint32_t PAIR_CAP = 1024;   /* noted pairs per batch; more than that are evaluated on the spot */
constexpr uint32_t PAIR_SHIFT = 28;   /* 16 points of a batch above, the centroid below */
constexpr uint32_t PAIR_MASK = (1u << PAIR_SHIFT) - 1;

template <int LD, bool SCREEN, int CPL>
__global__ void __launch_bounds__(1024 / CPL)
requeued_batch_f64_kernel(const double* __restrict__ data, size_t stride, const double* __restrict__ means_t, const double* __restrict__ norms,
                          uint32_t* __restrict__ assignment, uint32_t dim, uint32_t k, uint32_t kp,
                          const uint32_t* __restrict__ queue, uint32_t queue_stride, const uint32_t* __restrict__ queue_length,
                          const double* __restrict__ frame, const unsigned long long* __restrict__ misc)
{
	extern __shared__ double rows[]; /* dim x BATCH: coordinate q of the batch's points side by side */
	__shared__ unsigned long long chunk_min[BATCH];
	__shared__ uint32_t chunk_arg[BATCH];
	__shared__ double best_dist[BATCH], threshold[BATCH];
	__shared__ uint32_t best_arg[BATCH], pinned[BATCH], point_of[BATCH];
	__shared__ double part_xm[SCREEN ? THRESHOLD_PARTS : 1][BATCH], part_x2[SCREEN ? THRESHOLD_PARTS : 1][BATCH];
	__shared__ uint32_t pair_count, pair_list[SCREEN ? PAIR_CAP : 1]; /* (point of the batch << PAIR_SHIFT) | centroid */
	__shared__ double pair_dist[SCREEN ? PAIR_CAP : 1];
	constexpr uint32_t NONE = 0xffffffffu;
	const uint32_t total = *queue_length;
	for (uint32_t first = blockIdx.x * BATCH; first < total; first += gridDim.x * BATCH) {
		const uint32_t here = min((uint32_t)BATCH, total - first);
		__syncthreads(); /* the previous batch is written out */
		if (threadIdx.x < BATCH) {
			const size_t entry = (size_t)(first + min(threadIdx.x, here - 1)) * queue_stride;
			point_of[threadIdx.x] = queue[entry];
			/* SCREEN: the queue holds (point, threshold) pairs of a float sweep: only a centroid whose ranking value
			 * c^2 - 2 c.x does not exceed the threshold can be the serial choice (the threshold is the sweep's best
			 * value plus its certificate, which covers the sweep's errors; the double ranking value is more accurate) */
			threshold[threadIdx.x] = SCREEN ? (double)__uint_as_float(queue[entry + 1]) : __builtin_inf();
			best_dist[threadIdx.x] = __builtin_inf();
			best_arg[threadIdx.x] = NONE;
			pinned[threadIdx.x] = 0;
		}
		__syncthreads();
		for (uint32_t e = threadIdx.x; e < BATCH * dim; e += blockDim.x) rows[(e % dim) * BATCH + e / dim] = data[elem<LD>(stride, point_of[e / dim], e % dim)];
		if (SCREEN) {
			/* The float sweep ranked x - m against c - m (frame: m, then |m|^2), where the ranking values are those of
			 * the data as given plus sh = 2 x . m - |m|^2; the values below are of the data as given, so the threshold
			 * comes back by sh, with an allowance for the double arithmetic on both sides (certificate.h has the
			 * float version of this): (4 d + 40) 2^-52 (|x|^2 + max |c|^2). */
			__syncthreads(); /* the rows are in place */
			/* x . m and |x|^2 of every point: up to 16 lanes share a row, each with an interleaved part of it (a single lane
			 * per point walked 256 dimensions one LDS round trip at a time) */
			const uint32_t parts = min(THRESHOLD_PARTS, blockDim.x / BATCH);
			if (threadIdx.x < BATCH * parts) {
				const uint32_t b = threadIdx.x % BATCH, part = threadIdx.x / BATCH;
				double xm = 0.0, x2 = 0.0;
				for (uint32_t q = part; q < dim; q += parts) {
					const double v = rows[q * BATCH + b];
					xm = __builtin_fma(v, frame[q], xm);
					x2 = __builtin_fma(v, v, x2);
				}
				part_xm[part][b] = xm;
				part_x2[part][b] = x2;
			}
			__syncthreads();
			if (threadIdx.x < BATCH) {
				double xm = 0.0, x2 = 0.0;
				for (uint32_t part = 0; part < parts; ++part) {
					xm += part_xm[part][threadIdx.x];
					x2 += part_x2[part][threadIdx.x];
				}
				const double c2max = __longlong_as_double((long long)misc[1]);
				const double t = threshold[threadIdx.x] - (2.0 * xm - frame[dim]) + (4.0 * dim + 40.0) * 0x1p-52 * (x2 + c2max);
				threshold[threadIdx.x] = t == t ? t : __builtin_inf(); /* (values the bound does not cover: every centroid is evaluated) */
			}
		}
		/* One pass over the centroids in chunks of blockDim.x * CPL. LISTING (a float sweep gave thresholds): the (point,
		 * centroid) pairs within the threshold -- two or three per point -- are noted in LDS and evaluated afterwards, one
		 * lane each (evaluating on the spot leaves the other lanes of the wavefront waiting through the serial sum, once
		 * per point and centroid of the lane). Otherwise, and when the list overflows (thresholds that cover nothing,
		 * many equal centroids), every lane evaluates its pairs on the spot and the chunks are merged one by one. */
		auto scan = [&](auto listing_tag) {
			constexpr bool LISTING = decltype(listing_tag)::value;
			for (uint32_t base = 0; base < k; base += blockDim.x * CPL) {
				if (!LISTING) {
					__syncthreads(); /* rows are in place; the previous chunk is merged */
					if (threadIdx.x < BATCH) { chunk_min[threadIdx.x] = ~0ull; chunk_arg[threadIdx.x] = NONE; }
				}
				uint32_t j[CPL], jj[CPL]; /* this lane's centroids of the chunk, blockDim.x apart (coalesced loads) */
#pragma unroll
				for (int c = 0; c < CPL; ++c) { j[c] = base + c * blockDim.x + threadIdx.x; jj[c] = min(j[c], kp - 1); }
				double dist[LISTING ? 1 : CPL][LISTING ? 1 : BATCH];
				uint32_t takes_part[CPL]; /* bit b: centroid c of this lane is evaluated for point b */
#pragma unroll
				for (int c = 0; c < CPL; ++c) takes_part[c] = 0;
				if (SCREEN) {
					double dot[CPL][BATCH];
#pragma unroll
					for (int c = 0; c < CPL; ++c)
#pragma unroll
						for (int b = 0; b < BATCH; ++b) dot[c][b] = 0.0;
					/* the centroids' coordinates are requested AHEAD dimensions before they are used (unrolling alone left
					 * every trip waiting for its own loads) */
					double ahead[AHEAD][CPL];
#pragma unroll
					for (int d = 0; d < AHEAD; ++d)
#pragma unroll
						for (int c = 0; c < CPL; ++c) ahead[d][c] = means_t[(size_t)min((uint32_t)d, dim - 1) * kp + jj[c]];
					for (uint32_t q0 = 0; q0 < dim; q0 += AHEAD) {
#pragma unroll
						for (int d = 0; d < AHEAD; ++d) {
							const uint32_t q = q0 + d;
							if (q < dim) {
								double cv[CPL];
#pragma unroll
								for (int c = 0; c < CPL; ++c) {
									cv[c] = ahead[d][c];
									ahead[d][c] = means_t[(size_t)min(q + AHEAD, dim - 1) * kp + jj[c]];
								}
#pragma unroll
								for (int b = 0; b < BATCH; ++b) {
									const double x = rows[q * BATCH + b]; /* one broadcast read serves CPL multiply-adds */
#pragma unroll
									for (int c = 0; c < CPL; ++c) dot[c][b] = __builtin_fma(x, cv[c], dot[c][b]);
								}
							}
						}
					}
#pragma unroll
					for (int c = 0; c < CPL; ++c) {
						const double c2 = norms[jj[c]];
#pragma unroll
						for (int b = 0; b < BATCH; ++b) {
							const bool within = j[c] < k && !(__builtin_fma(-2.0, dot[c][b], c2) > threshold[b]);
							if constexpr (LISTING) {
								if (within) { /* rare */
									const uint32_t slot = atomicAdd(&pair_count, 1u);
									if (slot < PAIR_CAP) pair_list[slot] = ((uint32_t)b << PAIR_SHIFT) | j[c];
								}
							}
							else {
								dist[c][b] = 0.0;
								if (within) { /* rare */
									double sum = 0.0;
#pragma unroll 8
									for (uint32_t q = 0; q < dim; ++q) {
										double diff = rows[q * BATCH + b] - means_t[(size_t)q * kp + jj[c]];
										double sq = diff * diff;
										sum = sum + sq;
									}
									dist[c][b] = __builtin_sqrt(sum);
									takes_part[c] |= 1u << b;
								}
							}
						}
					}
				}
				else if constexpr (!LISTING) {
#pragma unroll
					for (int c = 0; c < CPL; ++c)
#pragma unroll
						for (int b = 0; b < BATCH; ++b) dist[c][b] = 0.0; /* the sums, then their roots */
#pragma unroll 1
					for (uint32_t q = 0; q < dim; ++q) {
						double cv[CPL];
#pragma unroll
						for (int c = 0; c < CPL; ++c) cv[c] = means_t[(size_t)q * kp + jj[c]];
#pragma unroll
						for (int b = 0; b < BATCH; ++b) {
							const double x = rows[q * BATCH + b];
#pragma unroll
							for (int c = 0; c < CPL; ++c) {
								double diff = x - cv[c];
								double sq = diff * diff;
								dist[c][b] = dist[c][b] + sq;
							}
						}
					}
#pragma unroll
					for (int c = 0; c < CPL; ++c) {
#pragma unroll
						for (int b = 0; b < BATCH; ++b) dist[c][b] = __builtin_sqrt(dist[c][b]);
						takes_part[c] = j[c] < k ? 0xffffu : 0u;
					}
				}
				if constexpr (!LISTING) {
					__syncthreads(); /* chunk_min is reset */
#pragma unroll
					for (int c = 0; c < CPL; ++c) {
#pragma unroll
						for (int b = 0; b < BATCH; ++b) {
							if (takes_part[c] & (1u << b)) {
								if (dist[c][b] == dist[c][b]) atomicMin(&chunk_min[b], (unsigned long long)__double_as_longlong(dist[c][b]));
								else if (j[c] == 0) pinned[b] = 1;
							}
						}
					}
					__syncthreads();
#pragma unroll
					for (int c = 0; c < CPL; ++c) {
#pragma unroll
						for (int b = 0; b < BATCH; ++b)
							if ((takes_part[c] & (1u << b)) && dist[c][b] == dist[c][b] && (unsigned long long)__double_as_longlong(dist[c][b]) == chunk_min[b])
								atomicMin(&chunk_arg[b], j[c]);
					}
					__syncthreads();
					if (threadIdx.x < BATCH && chunk_arg[threadIdx.x] != NONE) {
						const double d = __longlong_as_double((long long)chunk_min[threadIdx.x]);
						if (best_arg[threadIdx.x] == NONE || best_dist[threadIdx.x] > d) { best_dist[threadIdx.x] = d; best_arg[threadIdx.x] = chunk_arg[threadIdx.x]; }
					}
				}
			}
		};
		bool listed = false;
		if constexpr (SCREEN) {
			if (k <= PAIR_MASK) {
				if (threadIdx.x == 0) pair_count = 0;
				if (threadIdx.x < BATCH) { chunk_min[threadIdx.x] = ~0ull; chunk_arg[threadIdx.x] = NONE; }
				__syncthreads(); /* rows and thresholds are in place, the list is empty */
				scan(std::true_type{});
				__syncthreads();
				const uint32_t found = pair_count;
				listed = found <= PAIR_CAP;
				if (listed) {
					/* one lane per pair: the serial sum, then the smallest distance per point and the lowest centroid that has it */
					for (uint32_t slot = threadIdx.x; slot < found; slot += blockDim.x) {
						const uint32_t entry = pair_list[slot], b = entry >> PAIR_SHIFT, j = entry & PAIR_MASK;
						double sum = 0.0;
#pragma unroll 8
						for (uint32_t q = 0; q < dim; ++q) {
							double diff = rows[q * BATCH + b] - means_t[(size_t)q * kp + j];
							double sq = diff * diff;
							sum = sum + sq;
						}
						const double d = __builtin_sqrt(sum);
						pair_dist[slot] = d;
						if (d == d) atomicMin(&chunk_min[b], (unsigned long long)__double_as_longlong(d));
						else if (j == 0) pinned[b] = 1;
					}
					__syncthreads();
					for (uint32_t slot = threadIdx.x; slot < found; slot += blockDim.x) {
						const uint32_t entry = pair_list[slot], b = entry >> PAIR_SHIFT, j = entry & PAIR_MASK;
						const double d = pair_dist[slot];
						if (d == d && (unsigned long long)__double_as_longlong(d) == chunk_min[b]) atomicMin(&chunk_arg[b], j);
					}
					__syncthreads();
					if (threadIdx.x < BATCH && chunk_arg[threadIdx.x] != NONE) {
						best_dist[threadIdx.x] = __longlong_as_double((long long)chunk_min[threadIdx.x]);
						best_arg[threadIdx.x] = chunk_arg[threadIdx.x];
					}
				}
			}
		}
		if (!listed) scan(std::false_type{});
		__syncthreads();
		if (threadIdx.x < here)
			assignment[point_of[threadIdx.x]] = (pinned[threadIdx.x] || best_arg[threadIdx.x] == NONE) ? 0u : best_arg[threadIdx.x];
	}
}

/*
 * Ranking sweep: same data flow as above with one FMA per element; see the file header for the certificate.
 * kd = (16 d + 48) 2^-53. The certificate needs |x|^2 + max |c|^2 inside (1e-250, 1e300): above, intermediate values
 * may overflow; below, squares lose bits to underflow; NaN fails both comparisons.
 */
template <int LD, int DPAD, int G, int P>
__global__ void __launch_bounds__(256)
rank_f64_kernel(const double* __restrict__ data, size_t stride, const double* __restrict__ means_t, const double* __restrict__ norms,
                unsigned long long* __restrict__ misc, uint32_t* __restrict__ queue, uint32_t* __restrict__ assignment,
                uint32_t dim, uint32_t k, uint32_t kp, uint32_t n, double kd)
{
	/* P points per lane: a scalar operand is 8 bytes per wavefront instruction here, and the scalar cache supplies
	 * about 2 bytes per cycle and compute unit, a quarter of what four SIMDs issuing one FMA every 4 cycles ask for;
	 * every centroid value fetched is therefore used for P points. */
	uint32_t i[P], pt[P];
	double x[P][DPAD > 0 ? DPAD : 1];
	double x2[P];
#pragma unroll
	for (int p = 0; p < P; ++p) {
		i[p] = (blockIdx.x * P + p) * blockDim.x + threadIdx.x;
		pt[p] = min(i[p], n - 1); /* lanes past the end repeat the last point and store nothing */
		x2[p] = 0.0;
		if (DPAD > 0) {
#pragma unroll
			for (int q = 0; q < DPAD; ++q) {
				x[p][q] = (uint32_t)q < dim ? data[elem<LD>(stride, pt[p], q)] : 0.0;
				x2[p] = __builtin_fma(x[p][q], x[p][q], x2[p]);
			}
		}
		else {
			for (uint32_t q = 0; q < dim; ++q) {
				const double v = data[elem<LD>(stride, pt[p], q)];
				x2[p] = __builtin_fma(v, v, x2[p]);
			}
		}
	}
	double m1[P], m2[P];
	uint32_t i1[P];
#pragma unroll
	for (int p = 0; p < P; ++p) { m1[p] = __builtin_inf(); m2[p] = __builtin_inf(); i1[p] = 0; }
	for (uint32_t g = 0; g < kp; g += G) {
		double dot[P][G];
#pragma unroll
		for (int p = 0; p < P; ++p)
#pragma unroll
			for (int j = 0; j < G; ++j) dot[p][j] = 0.0;
		if (DPAD > 0) {
#pragma unroll
			for (int q = 0; q < DPAD; ++q) {
				if ((uint32_t)q < dim) { /* uniform */
					const double* row = means_t + (size_t)q * kp + g; /* uniform address: scalar loads */
#pragma unroll
					for (int j = 0; j < G; ++j)
#pragma unroll
						for (int p = 0; p < P; ++p) dot[p][j] = __builtin_fma(x[p][q], row[j], dot[p][j]);
				}
			}
		}
		else {
#pragma unroll 2
			for (uint32_t q = 0; q < dim; ++q) {
				double xq[P];
#pragma unroll
				for (int p = 0; p < P; ++p) xq[p] = data[elem<LD>(stride, pt[p], q)];
				const double* row = means_t + (size_t)q * kp + g;
#pragma unroll
				for (int j = 0; j < G; ++j)
#pragma unroll
					for (int p = 0; p < P; ++p) dot[p][j] = __builtin_fma(xq[p], row[j], dot[p][j]);
			}
		}
		const double* c2 = norms + g; /* +inf for the padding: never the smallest */
#pragma unroll
		for (int j = 0; j < G; ++j) {
#pragma unroll
			for (int p = 0; p < P; ++p) {
				const double a = __builtin_fma(-2.0, dot[p][j], c2[j]);
				m2[p] = __builtin_fmin(m2[p], __builtin_fmax(m1[p], a));
				const bool lt = a < m1[p];
				i1[p] = lt ? g + j : i1[p];
				m1[p] = lt ? a : m1[p];
			}
		}
	}
	const double max_c2 = __longlong_as_double((long long)misc[1]);
	const uint32_t lane = threadIdx.x & (WAVE - 1);
#pragma unroll
	for (int p = 0; p < P; ++p) {
		if (i[p] < n) assignment[i[p]] = i1[p];
		const double scale = x2[p] + max_c2;
		const bool certified = (m2[p] - m1[p] > kd * scale) && scale < 1e300 && scale > 1e-250;
		const bool flagged = i[p] < n && !certified;
		const unsigned long long votes = __ballot(flagged);
		if (votes) { /* uniform: one atomic per wavefront */
			uint32_t base = 0;
			if (lane == 0) base = (uint32_t)atomicAdd(&misc[0], (unsigned long long)__popcll(votes));
			base = __builtin_amdgcn_readfirstlane(base);
			if (flagged) queue[base + __popcll(votes & ((1ull << lane) - 1))] = i[p];
		}
	}
}

template <int LD, int LM, bool PRIVATE>
__global__ void __launch_bounds__(256)
update_f64_kernel(const double* __restrict__ data, size_t stride, const uint32_t* __restrict__ assignment,
                  double* __restrict__ means, size_t stride_means, uint32_t* __restrict__ sizes,
                  uint32_t dim, uint32_t k, uint32_t n)
{
	extern __shared__ double sums[]; /* PRIVATE: k * dim doubles, then k counts */
	uint32_t* counts = (uint32_t*)(sums + (size_t)k * dim);
	if (PRIVATE) {
		for (uint32_t e = threadIdx.x; e < k * dim; e += blockDim.x) sums[e] = 0.0;
		for (uint32_t e = threadIdx.x; e < k; e += blockDim.x) counts[e] = 0;
		__syncthreads();
	}
	const size_t total = (size_t)n * dim;
	for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (size_t)gridDim.x * blockDim.x) {
		/* consecutive lanes read consecutive addresses in either layout */
		const uint32_t i = LD == KMX_AOS ? (uint32_t)(e / dim) : (uint32_t)(e % n);
		const uint32_t q = LD == KMX_AOS ? (uint32_t)(e % dim) : (uint32_t)(e / n);
		const uint32_t c = assignment[i];
		const double v = data[elem<LD>(stride, i, q)];
		if (PRIVATE) {
			unsafeAtomicAdd(&sums[(size_t)c * dim + q], v); /* ds_add_f64 */
			if (q == 0) atomicAdd(&counts[c], 1u);
		}
		else {
			unsafeAtomicAdd(&means[elem<LM>(stride_means, c, q)], v); /* global_atomic_add_f64 */
			if (q == 0) atomicAdd(&sizes[c], 1u);
		}
	}
	if (PRIVATE) {
		__syncthreads();
		for (uint32_t e = threadIdx.x; e < k * dim; e += blockDim.x) {
			const double v = sums[e];
			if (v != 0.0) unsafeAtomicAdd(&means[elem<LM>(stride_means, e / dim, e % dim)], v);
		}
		for (uint32_t e = threadIdx.x; e < k; e += blockDim.x)
			if (counts[e]) atomicAdd(&sizes[e], counts[e]);
	}
}

/*
 * Sums that do not fit one private copy: the clusters are split into ranges whose sums fit 32 KB of LDS, and work-group
 * (slice, range) walks its slice of the points in pieces of 8192: first it scans the piece's assignments (4 bytes per
 * point, coalesced) and lists the points of its range in LDS, then all lanes add the listed rows, one lane per
 * element, with LDS atomics. Every row is read from HBM once, by the work-group of its cluster's range; only the
 * assignment vector is read once per range. Listing first keeps all lanes busy in the second step and makes its loads
 * independent of each other (testing the assignment in the adding loop left most lanes idle behind a dependent load).
 */
constexpr uint32_t RANGE_BYTES = 32 * 1024 - 64; /* private sums of one range (with the list: just below 64 KB) */
constexpr uint32_t PIECE_POINTS = 8192;      /* listed per step: 13 bits of position, the rest of the word for the cluster */

template <int LD, int LM>
__global__ void __launch_bounds__(1024)
update_ranges_f64_kernel(const double* __restrict__ data, size_t stride, const uint32_t* __restrict__ assignment,
                         double* __restrict__ means, size_t stride_means, uint32_t* __restrict__ sizes,
                         uint32_t dim, uint32_t k, uint32_t n, uint32_t range_size, uint32_t slices)
{
	extern __shared__ double sums[]; /* range_size * dim doubles, range_size counts, PIECE_POINTS list entries */
	__shared__ uint32_t listed;
	uint32_t* counts = (uint32_t*)(sums + (size_t)range_size * dim);
	uint32_t* list = counts + range_size;
	const uint32_t slice = blockIdx.x % slices, range = blockIdx.x / slices;
	const uint32_t c0 = range * range_size, cn = min(range_size, k - c0);
	for (uint32_t e = threadIdx.x; e < cn * dim; e += blockDim.x) sums[e] = 0.0;
	for (uint32_t e = threadIdx.x; e < cn; e += blockDim.x) counts[e] = 0;
	const uint32_t per_slice = (n + slices - 1) / slices;
	const uint32_t s0 = min(slice * per_slice, n), s1 = min(s0 + per_slice, n);
	for (uint32_t p0 = s0; p0 < s1; p0 += PIECE_POINTS) {
		__syncthreads(); /* sums are zero / the previous piece is added */
		if (threadIdx.x == 0) listed = 0;
		__syncthreads();
		const uint32_t p1 = min(p0 + PIECE_POINTS, s1);
		for (uint32_t i = p0 + threadIdx.x; i < p1; i += blockDim.x) {
			const uint32_t c = assignment[i] - c0;
			if (c < cn) {
				list[atomicAdd(&listed, 1u)] = (i - p0) | (c << 13);
				atomicAdd(&counts[c], 1u);
			}
		}
		__syncthreads();
		const uint32_t members = listed;
		const uint32_t total = members * dim;
#pragma unroll 4
		for (uint32_t e = threadIdx.x; e < total; e += blockDim.x) {
			/* consecutive lanes: consecutive dimensions of a row (AoS) / consecutive listed points of a dimension (SoA) */
			const uint32_t m = LD == KMX_AOS ? e / dim : e % members;
			const uint32_t q = LD == KMX_AOS ? e % dim : e / members;
			const uint32_t entry = list[m];
			unsafeAtomicAdd(&sums[(size_t)(entry >> 13) * dim + q], data[elem<LD>(stride, p0 + (entry & (PIECE_POINTS - 1)), q)]);
		}
	}
	__syncthreads();
	for (uint32_t e = threadIdx.x; e < cn * dim; e += blockDim.x) {
		const double v = sums[e];
		if (v != 0.0) unsafeAtomicAdd(&means[elem<LM>(stride_means, c0 + e / dim, e % dim)], v);
	}
	for (uint32_t e = threadIdx.x; e < cn; e += blockDim.x)
		if (counts[e]) atomicAdd(&sizes[c0 + e], counts[e]);
}

/*
 * The same for AoS rows of 128 dimensions and more: the work-group has one lane per dimension (at most 1024 lanes; longer
 * rows take several dimensions per lane) and all of them add ONE listed row at a time, ROWS_IN_FLIGHT row loads in flight
 * (the last batch of a piece included: loads one after the other wait for HBM each). No two lanes ever meet at an element
 * of the sums, so the additions are plain reads and writes of LDS instead of atomics (an LDS floating-point atomic
 * serialises its lanes): N = 1M doubles, k = 1024: d = 256 0.98 -> 0.54 ms, d = 128 0.41 ms with 8 loads in flight, 0.36 ms
 * with 16 (rows of 512 dimensions: 0.25 ms with 8, 0.27 ms with 16). Pieces of 2048 points keep the list at 8 KB, so that
 * four work-groups share a compute unit; pieces of 4096 and 8192 points measured 25-50 % slower. The ranges differ in their
 * numbers of points (the clusters of a Lloyd iteration are far from equal), so the launch holds twice as many work-groups
 * as are resident and the slices are half as long: at benchmark configuration 4 (N = 1M, d = 256, k = 1024, the assignment of
 * the iteration) 0.55 ms against 0.72 ms with as many as are resident and 1.28 ms with half of that; 16 and 32 per compute unit
 * are no better, and on equal clusters the number makes no difference.
 */
constexpr uint32_t ROWS_PIECE_POINTS = 2048;
constexpr uint32_t ROWS_MIN_DIM = 128;
constexpr uint32_t ROWS_GROUPS_PER_CU = 8; /* work-groups of the launch per compute unit (four are resident) */

template <int LM, int ROWS_IN_FLIGHT>
__global__ void __launch_bounds__(1024)
update_ranges_rows_f64_kernel(const double* __restrict__ data, size_t stride, const uint32_t* __restrict__ assignment,
                              double* __restrict__ means, size_t stride_means, uint32_t* __restrict__ sizes,
                              uint32_t dim, uint32_t k, uint32_t n, uint32_t range_size, uint32_t slices)
{
	extern __shared__ double sums[]; /* range_size * dim doubles, range_size counts, ROWS_PIECE_POINTS list entries */
	__shared__ uint32_t listed;
	uint32_t* counts = (uint32_t*)(sums + (size_t)range_size * dim);
	uint32_t* list = counts + range_size;
	const uint32_t slice = blockIdx.x % slices, range = blockIdx.x / slices;
	const uint32_t c0 = range * range_size, cn = min(range_size, k - c0);
	for (uint32_t e = threadIdx.x; e < cn * dim; e += blockDim.x) sums[e] = 0.0;
	for (uint32_t e = threadIdx.x; e < cn; e += blockDim.x) counts[e] = 0;
	const uint32_t per_slice = (n + slices - 1) / slices;
	const uint32_t s0 = min(slice * per_slice, n), s1 = min(s0 + per_slice, n);
	for (uint32_t p0 = s0; p0 < s1; p0 += ROWS_PIECE_POINTS) {
		__syncthreads(); /* sums are zero / the previous piece is added */
		if (threadIdx.x == 0) listed = 0;
		__syncthreads();
		const uint32_t p1 = min(p0 + ROWS_PIECE_POINTS, s1);
		for (uint32_t i = p0 + threadIdx.x; i < p1; i += blockDim.x) {
			const uint32_t c = assignment[i] - c0;
			if (c < cn) {
				list[atomicAdd(&listed, 1u)] = (i - p0) | (c << 13);
				atomicAdd(&counts[c], 1u);
			}
		}
		__syncthreads();
		const uint32_t members = listed;
		for (uint32_t q = threadIdx.x; q < dim; q += blockDim.x) {
			for (uint32_t m = 0; m < members; m += ROWS_IN_FLIGHT) {
				double v[ROWS_IN_FLIGHT];
				uint32_t at[ROWS_IN_FLIGHT];
#pragma unroll
				for (int i = 0; i < ROWS_IN_FLIGHT; ++i) { /* the last batch repeats its first row where it has no more */
					const uint32_t entry = list[m + i < members ? m + i : m];
					at[i] = (entry >> 13) * dim + q;
					v[i] = data[(size_t)(p0 + (entry & (PIECE_POINTS - 1))) * stride + q];
				}
#pragma unroll
				for (int i = 0; i < ROWS_IN_FLIGHT; ++i) /* in order: two of the rows may belong to one cluster */
					if (m + i < members) sums[at[i]] += v[i];
			}
		}
	}
	__syncthreads();
	for (uint32_t e = threadIdx.x; e < cn * dim; e += blockDim.x) {
		const double v = sums[e];
		if (v != 0.0) unsafeAtomicAdd(&means[elem<LM>(stride_means, c0 + e / dim, e % dim)], v);
	}
	for (uint32_t e = threadIdx.x; e < cn; e += blockDim.x)
		if (counts[e]) atomicAdd(&sizes[c0 + e], counts[e]);
}

/*
 * AoS rows of 17 to 127 dimensions: the listed points of a piece are sorted by cluster (a counting sort in LDS: the
 * listing pass takes each point's rank inside its cluster from the atomic that counts it), the sorted list is cut into
 * equal segments, one per group of G lanes (lane = dimension), and a group adds the rows of its segment in a register,
 * eight row loads in flight, and hands the sum over to the LDS copy -- with an atomic, as a cluster may span segments --
 * only where the cluster changes: one LDS atomic per run of a cluster instead of one per row (an LDS floating-point
 * atomic of a wavefront takes about 70 cycles; they bounded update_ranges_f64_kernel): N = 2M doubles, d = 32, k = 1024:
 * 0.147 -> 0.115 ms (4.4 TB/s with the clearing and the division).
 */
constexpr uint32_t SORTED_PIECE_POINTS = 8192;             /* 13 bits of position in a list entry, the cluster above */
constexpr uint32_t SORTED_RANGE_BYTES = 30 * 1024 - 64;    /* sums of a range: with the sorted list and the counts just below 64 KB */
constexpr int SORTED_IN_FLIGHT = 8;

template <int LM, int G>
__global__ void __launch_bounds__(1024)
update_ranges_sorted_f64_kernel(const double* __restrict__ data, size_t stride, const uint32_t* __restrict__ assignment,
                                double* __restrict__ means, size_t stride_means, uint32_t* __restrict__ sizes,
                                uint32_t dim, uint32_t k, uint32_t n, uint32_t range_size, uint32_t slices)
{
	extern __shared__ double sums[]; /* range_size * dim doubles, range_size counts, range_size places, the sorted list */
	__shared__ uint32_t listed;
	uint32_t* counts = (uint32_t*)(sums + (size_t)range_size * dim);
	uint32_t* place = counts + range_size; /* members of the piece per cluster, then where the cluster's run begins */
	uint32_t* sorted = place + range_size;
	constexpr uint32_t PER_LANE = SORTED_PIECE_POINTS / 1024;
	constexpr uint32_t NOT_MINE = 0xffffffffu;
	const uint32_t slice = blockIdx.x % slices, range = blockIdx.x / slices;
	const uint32_t c0 = range * range_size, cn = min(range_size, k - c0);
	for (uint32_t e = threadIdx.x; e < cn * dim; e += blockDim.x) sums[e] = 0.0;
	for (uint32_t e = threadIdx.x; e < cn; e += blockDim.x) counts[e] = 0;
	const uint32_t per_slice = (n + slices - 1) / slices;
	const uint32_t s0 = min(slice * per_slice, n), s1 = min(s0 + per_slice, n);
	const uint32_t group = threadIdx.x / G, q = threadIdx.x % G;
	constexpr uint32_t GROUPS = 1024 / G;
	for (uint32_t p0 = s0; p0 < s1; p0 += SORTED_PIECE_POINTS) {
		__syncthreads(); /* sums are zero / the previous piece is added */
		for (uint32_t e = threadIdx.x; e < cn; e += blockDim.x) place[e] = 0;
		__syncthreads();
		const uint32_t p1 = min(p0 + SORTED_PIECE_POINTS, s1);
		uint32_t cluster[PER_LANE], rank[PER_LANE];
#pragma unroll
		for (uint32_t u = 0; u < PER_LANE; ++u) {
			const uint32_t i = p0 + u * 1024 + threadIdx.x;
			const uint32_t c = i < p1 ? assignment[i] - c0 : NOT_MINE;
			cluster[u] = c < cn ? c : NOT_MINE;
			rank[u] = 0;
			if (cluster[u] != NOT_MINE) rank[u] = atomicAdd(&place[c], 1u);
		}
		__syncthreads();
		if (threadIdx.x < WAVE) { /* exclusive prefix over the clusters of the range (a few hundred at most) */
			const uint32_t each = (cn + WAVE - 1) / WAVE, from = min(threadIdx.x * each, cn), to = min(from + each, cn);
			uint32_t mine = 0;
			for (uint32_t e = from; e < to; ++e) mine += place[e];
			uint32_t before = mine;
			for (int off = 1; off < WAVE; off <<= 1) {
				const uint32_t other = (uint32_t)__shfl_up((int)before, off);
				if ((int)threadIdx.x >= off) before += other;
			}
			if (threadIdx.x == WAVE - 1) listed = before;
			before -= mine;
			for (uint32_t e = from; e < to; ++e) {
				const uint32_t members = place[e];
				place[e] = before;
				counts[e] += members;
				before += members;
			}
		}
		__syncthreads();
#pragma unroll
		for (uint32_t u = 0; u < PER_LANE; ++u)
			if (cluster[u] != NOT_MINE) sorted[place[cluster[u]] + rank[u]] = (u * 1024 + threadIdx.x) | (cluster[u] << 13);
		__syncthreads();
		const uint32_t members = listed;
		const uint32_t share = (members + GROUPS - 1) / GROUPS;
		const uint32_t m0 = min(group * share, members), m1 = min(m0 + share, members);
		if (q < dim && m0 < m1) {
			double run = 0.0;
			uint32_t current = sorted[m0] >> 13;
			for (uint32_t m = m0; m < m1; m += SORTED_IN_FLIGHT) {
				double v[SORTED_IN_FLIGHT];
				uint32_t c[SORTED_IN_FLIGHT];
#pragma unroll
				for (int i = 0; i < SORTED_IN_FLIGHT; ++i) { /* the last batch repeats its last row where it has no more */
					const uint32_t entry = sorted[min(m + i, m1 - 1)];
					c[i] = entry >> 13;
					v[i] = data[(size_t)(p0 + (entry & (SORTED_PIECE_POINTS - 1))) * stride + q];
				}
#pragma unroll
				for (int i = 0; i < SORTED_IN_FLIGHT; ++i) {
					if (m + i < m1) {
						if (c[i] != current) {
							unsafeAtomicAdd(&sums[(size_t)current * dim + q], run);
							current = c[i];
							run = 0.0;
						}
						run += v[i];
					}
				}
			}
			unsafeAtomicAdd(&sums[(size_t)current * dim + q], run);
		}
	}
	__syncthreads();
	for (uint32_t e = threadIdx.x; e < cn * dim; e += blockDim.x) {
		const double v = sums[e];
		if (v != 0.0) unsafeAtomicAdd(&means[elem<LM>(stride_means, c0 + e / dim, e % dim)], v);
	}
	for (uint32_t e = threadIdx.x; e < cn; e += blockDim.x)
		if (counts[e]) atomicAdd(&sizes[c0 + e], counts[e]);
}

/* serial.hpp:66-72: divide by the member count, empty clusters stay at zero */
template <int LM>
__global__ void __launch_bounds__(256)
divide_means_f64_kernel(double* __restrict__ means, size_t stride_means, const uint32_t* __restrict__ sizes, uint32_t dim, uint32_t k)
{
	const uint32_t e = blockIdx.x * blockDim.x + threadIdx.x;
	if (e >= k * dim) return;
	const uint32_t c = e / dim, q = e % dim;
	const uint32_t size = sizes[c];
	if (size == 0) return;
	double* p = &means[elem<LM>(stride_means, c, q)];
	*p = *p / (double)size;
}

namespace {

int check_layout_f64(const char* who, const char* what, int layout, size_t stride, uint32_t count, uint32_t dim)
{
	if (layout != KMX_AOS && layout != KMX_SOA) return fail(KMX_ERR_INVALID_ARGUMENT, "%s: unknown %s layout %d", who, what, layout);
	if (layout == KMX_AOS && stride < dim) return fail(KMX_ERR_INVALID_ARGUMENT, "%s: %s stride %zu < dim %u", who, what, stride, dim);
	if (layout == KMX_SOA && stride < count) return fail(KMX_ERR_INVALID_ARGUMENT, "%s: %s stride %zu < count %u", who, what, stride, count);
	return KMX_OK;
}

template <int LD>
int launch_assign_f64_ld(int variant, const double* data, size_t stride, uint32_t* assignment, uint32_t dim, uint32_t k, uint32_t kp, uint32_t n,
                         kmx_exec_params* exec, const DeviceInfo& dev, const uint32_t* float_queue, const uint32_t* float_queue_length)
{
	const dim3 block(256), grid((n + 255) / 256);
	exec->block_size = block.x;
	exec->block_count = grid.x;
	unsigned long long* misc = (unsigned long long*)g_misc;
	uint32_t* queue = (uint32_t*)g_queue;
	const uint32_t* exact_queue = queue; /* the queue the exact pass walks: ours (point numbers, length in misc[0], little endian) ... */
	uint32_t exact_stride = 1;
	const uint32_t* exact_length = (const uint32_t*)g_misc;
	if (float_queue) { exact_queue = float_queue; exact_stride = 2; exact_length = float_queue_length; } /* ... or the float sweep's (pairs) */
#define KMX_F64_EXACT(DPAD, G) \
	KMX_LAUNCH_KERNEL((assign_f64_kernel<LD, DPAD, G>), grid, block, 0, stream(), data, stride, g_means_t, assignment, dim, k, kp, n)
	/* queued points: many centroids and rows long enough to pay for the work-group-wide minimum -> batches of points
	 * against one lane per centroid; else 16 lanes (2 for few centroids) share a point */
	/* (without thresholds every pair is evaluated on the spot and every chunk merged across the work-group, which rows of
	 * fewer than 16 dimensions do not pay for; with them the batches win at every width: N = 2M doubles, d = 12, k = 1024,
	 * 40 k queued points: 0.72 -> 0.38 ms per call; N = 4M, d = 4, k = 4096, 33 k points: 1.99 -> 1.64 ms) */
	const bool batched = k >= 256 && dim >= (float_queue ? 2u : 16u) && (size_t)BATCH * dim * sizeof(double) <= 48 * 1024; /* dynamic + static LDS stay below 64 KB */
	const uint32_t batch_threads = std::min<uint32_t>(1024 / BATCH_CPL, ((k + BATCH_CPL - 1) / BATCH_CPL + WAVE - 1) / WAVE * WAVE);
	const dim3 bgrid(std::min<uint32_t>((n + BATCH - 1) / BATCH, dev.compute_units * 2));
	const bool many = k >= 256;
	const dim3 qgrid((uint32_t)std::min<size_t>(((size_t)n * (many ? 16 : 2) + 255) / 256, (size_t)dev.compute_units * 8));
#define KMX_F64_REQUEUED(DPAD) \
	do { \
		if (many) KMX_LAUNCH_KERNEL((requeued_f64_kernel<LD, DPAD, 16>), qgrid, block, 0, stream(), data, stride, g_means_t, assignment, \
		                             dim, k, kp, exact_queue, exact_stride, exact_length); \
		else KMX_LAUNCH_KERNEL((requeued_f64_kernel<LD, DPAD, 2>), qgrid, block, 0, stream(), data, stride, g_means_t, assignment, \
		                        dim, k, kp, exact_queue, exact_stride, exact_length); \
	} while (0)
#define KMX_F64_REQUEUED_BY_DIM() \
	do { \
		if (batched && float_queue) \
			KMX_LAUNCH_KERNEL((requeued_batch_f64_kernel<LD, true, BATCH_CPL>), bgrid, dim3(batch_threads), (size_t)BATCH * dim * sizeof(double), stream(), \
			                   data, stride, g_means_t, g_norms, assignment, dim, k, kp, exact_queue, exact_stride, exact_length, g_frame, misc); \
		else if (batched) \
			KMX_LAUNCH_KERNEL((requeued_batch_f64_kernel<LD, false, BATCH_CPL>), bgrid, dim3(batch_threads), (size_t)BATCH * dim * sizeof(double), stream(), \
			                   data, stride, g_means_t, g_norms, assignment, dim, k, kp, exact_queue, exact_stride, exact_length, g_frame, misc); \
		else if (dim > 32) KMX_F64_REQUEUED(0); \
		else if (dim <= 8) KMX_F64_REQUEUED(8); \
		else if (dim <= 16) KMX_F64_REQUEUED(16); \
		else KMX_F64_REQUEUED(32); \
	} while (0)
	if (variant == KMX_ASSIGN_BASE) {
		if (dim > 32) KMX_F64_EXACT(0, WIDE_GROUP);
		else if (dim <= 8) KMX_F64_EXACT(8, GROUP);
		else if (dim <= 16) KMX_F64_EXACT(16, GROUP);
		else KMX_F64_EXACT(32, GROUP);
		KMX_LAUNCH_CHECK("assign_f64_kernel");
		return KMX_OK;
	}
	if (float_queue) { /* a float sweep has ranked the points and queued the uncertified ones */
		KMX_F64_REQUEUED_BY_DIM();
		KMX_LAUNCH_CHECK("requeued_f64_kernel (points the float sweep did not certify)");
		return KMX_OK;
	}
	const double kd = (16.0 * dim + 48.0) * 0x1p-53;
	constexpr int P = 1; /* points per lane of the ranking sweep (2 measured no faster: fewer wavefronts hide less scalar-load latency) */
	const dim3 rgrid((n + 256 * P - 1) / (256 * P));
#define KMX_F64_RANK(DPAD, G) \
	KMX_LAUNCH_KERNEL((rank_f64_kernel<LD, DPAD, G, P>), rgrid, block, 0, stream(), data, stride, g_means_t, g_norms, misc, queue, assignment, dim, k, kp, n, kd)
	if (dim > 32) KMX_F64_RANK(0, 16);
	else if (dim <= 8) KMX_F64_RANK(8, GROUP);
	else if (dim <= 16) KMX_F64_RANK(16, GROUP);
	else KMX_F64_RANK(32, GROUP);
	KMX_LAUNCH_CHECK("rank_f64_kernel");
	KMX_F64_REQUEUED_BY_DIM();
	KMX_LAUNCH_CHECK("requeued_f64_kernel");
#undef KMX_F64_RANK
#undef KMX_F64_REQUEUED_BY_DIM
#undef KMX_F64_REQUEUED
#undef KMX_F64_EXACT
	return KMX_OK;
}

/* clusters per range of update_ranges_sorted_f64_kernel (0: a row does not fit) */
static uint32_t sorted_range_size(uint32_t k, uint32_t dim)
{
	return (uint32_t)std::min<size_t>(k, SORTED_RANGE_BYTES / ((size_t)dim * sizeof(double) + 2 * sizeof(uint32_t)));
}

template <int LD, int LM>
int launch_update_f64_t(int variant, const double* data, size_t stride, const uint32_t* assignment, double* means, size_t stride_means,
                        uint32_t* sizes, uint32_t dim, uint32_t k, uint32_t n, kmx_exec_params* exec, const DeviceInfo& dev, bool divide)
{
	const size_t private_bytes = ((size_t)k * dim) * sizeof(double) + (size_t)k * sizeof(uint32_t);
	const bool use_private = variant == KMX_UPDATE_ATOMIC_SHM && private_bytes <= 32 * 1024;
	/* ranges of clusters whose sums fit RANGE_BYTES of LDS (the cluster number must fit the list entry's 19 bits, which it
	 * does: at most RANGE_BYTES / 12 clusters); rows beyond that (dim > 4000) go to global atomics */
	const uint32_t range_size = (uint32_t)std::min<size_t>(k, RANGE_BYTES / ((size_t)dim * sizeof(double) + sizeof(uint32_t)));
	const uint32_t ranges = range_size ? (k + range_size - 1) / range_size : 0;
	const bool use_ranges = variant == KMX_UPDATE_ATOMIC_SHM && !use_private && range_size > 0 && ranges <= 256;
	const dim3 block(256);
	const size_t total = (size_t)n * dim;
	/* a work-group with private sums should add at least 16 times as many elements as it has sums to clear and flush */
	const size_t per_group = use_private ? std::max<size_t>(256, 16 * (size_t)k * dim) : 256;
	const uint32_t wanted = (uint32_t)std::min<size_t>((total + per_group - 1) / per_group, (size_t)dev.compute_units * (use_private ? 8 : 32));
	const dim3 grid(std::max<uint32_t>(wanted, 1));
	exec->block_size = block.x;
	exec->block_count = grid.x;
	if (n > 0 && use_ranges && LD == KMX_AOS && dim >= ROWS_MIN_DIM) {
		const size_t range_bytes = (size_t)range_size * dim * sizeof(double) + (size_t)range_size * sizeof(uint32_t) + ROWS_PIECE_POINTS * sizeof(uint32_t);
		const dim3 lanes(std::min<uint32_t>(1024, (dim + WAVE - 1) / WAVE * WAVE)); /* one per dimension */
		const size_t per_slice = std::max<size_t>(1024, 16 * (size_t)range_size * dim);
		const uint32_t slices = (uint32_t)std::max<size_t>(1, std::min<size_t>((total + per_slice - 1) / per_slice, std::max<size_t>(1, (size_t)dev.compute_units * ROWS_GROUPS_PER_CU / ranges)));
		exec->block_size = lanes.x;
		exec->block_count = slices * ranges;
		if (dim <= 256)
			KMX_LAUNCH_KERNEL((update_ranges_rows_f64_kernel<LM, 16>), dim3(slices * ranges), lanes, range_bytes, stream(),
			                   data, stride, assignment, means, stride_means, sizes, dim, k, n, range_size, slices);
		else
			KMX_LAUNCH_KERNEL((update_ranges_rows_f64_kernel<LM, 8>), dim3(slices * ranges), lanes, range_bytes, stream(),
			                   data, stride, assignment, means, stride_means, sizes, dim, k, n, range_size, slices);
		KMX_LAUNCH_CHECK("update_ranges_rows_f64_kernel");
	}
	else if (n > 0 && use_ranges && LD == KMX_AOS && dim > 16 && variant == KMX_UPDATE_ATOMIC_SHM && sorted_range_size(k, dim) > 0) {
		const uint32_t sorted_size = sorted_range_size(k, dim), sorted_ranges = (k + sorted_size - 1) / sorted_size;
		const size_t range_bytes = (size_t)sorted_size * dim * sizeof(double) + 2 * (size_t)sorted_size * sizeof(uint32_t) + SORTED_PIECE_POINTS * sizeof(uint32_t);
		const size_t per_slice = std::max<size_t>(1024, 16 * (size_t)sorted_size * dim);
		const uint32_t slices = (uint32_t)std::max<size_t>(1, std::min<size_t>((total + per_slice - 1) / per_slice, std::max<size_t>(1, (size_t)dev.compute_units * 2 / sorted_ranges))); /* as many as are resident (twice and four times as many: 8 and 20 % slower) */
		exec->block_size = 1024;
		exec->block_count = slices * sorted_ranges;
#define KMX_SORTED_F64(G) \
		KMX_LAUNCH_KERNEL((update_ranges_sorted_f64_kernel<LM, G>), dim3(slices * sorted_ranges), dim3(1024), range_bytes, stream(), \
		                   data, stride, assignment, means, stride_means, sizes, dim, k, n, sorted_size, slices)
		if (dim <= 32) KMX_SORTED_F64(32);
		else if (dim <= 64) KMX_SORTED_F64(64);
		else KMX_SORTED_F64(128);
#undef KMX_SORTED_F64
		KMX_LAUNCH_CHECK("update_ranges_sorted_f64_kernel");
	}
	else if (n > 0 && use_ranges) {
		const size_t range_bytes = (size_t)range_size * dim * sizeof(double) + (size_t)range_size * sizeof(uint32_t) + PIECE_POINTS * sizeof(uint32_t);
		const dim3 wide(1024);
		const size_t per_slice = std::max<size_t>(1024, 16 * (size_t)range_size * dim);
		const uint32_t slices = (uint32_t)std::max<size_t>(1, std::min<size_t>((total + per_slice - 1) / per_slice, std::max<size_t>(1, (size_t)dev.compute_units * 2 / ranges)));
		exec->block_count = slices * ranges;
		KMX_LAUNCH_KERNEL((update_ranges_f64_kernel<LD, LM>), dim3(slices * ranges), wide, range_bytes, stream(),
		                   data, stride, assignment, means, stride_means, sizes, dim, k, n, range_size, slices);
		KMX_LAUNCH_CHECK("update_ranges_f64_kernel");
	}
	else if (n > 0) {
		if (use_private)
			KMX_LAUNCH_KERNEL((update_f64_kernel<LD, LM, true>), grid, block, private_bytes, stream(),
			                   data, stride, assignment, means, stride_means, sizes, dim, k, n);
		else
			KMX_LAUNCH_KERNEL((update_f64_kernel<LD, LM, false>), grid, block, 0, stream(),
			                   data, stride, assignment, means, stride_means, sizes, dim, k, n);
		KMX_LAUNCH_CHECK("update_f64_kernel");
	}
	if (!divide) return KMX_OK; /* the update micro-benchmark wants the sums */
	KMX_LAUNCH_KERNEL((divide_means_f64_kernel<LM>), dim3((k * dim + 255) / 256), dim3(256), 0, stream(), means, stride_means, sizes, dim, k);
	KMX_LAUNCH_CHECK("divide_means_f64_kernel");
	return KMX_OK;
}

} // namespace

int release_f64_workspace()
{
	g_prepared = PreparedPoints();
	double** buffers[] = { &g_means_t, &g_norms, &g_queue, &g_misc, &g_data32, &g_means32, &g_frame };
	size_t* caps[] = { &g_means_t_cap, &g_norms_cap, &g_queue_cap, &g_misc_cap, &g_data32_cap, &g_means32_cap, &g_frame_cap };
	for (size_t b = 0; b < sizeof(buffers) / sizeof(buffers[0]); ++b) {
		if (*buffers[b]) KMX_HIP(hipFree(*buffers[b]));
		*buffers[b] = nullptr;
		*caps[b] = 0;
	}
	return KMX_OK;
}

/* The announced points are about to change or go away: [dst, dst + bytes) is being written or released. If it touches
 * them, the float copy must not outlive them -- hipMalloc readily hands the same address out again, and the sweeps
 * would rank the new contents against the old copy. bytes = 0: extent unknown, anything at or below the points counts. */
void forget_prepared_points_f64(const void* dst, size_t bytes)
{
	if (!g_prepared.data || !dst) return;
	const size_t extent = g_prepared.layout == KMX_AOS ? (size_t)(g_prepared.n - 1) * g_prepared.stride + g_prepared.dim
	                                                   : (size_t)(g_prepared.dim - 1) * g_prepared.stride + g_prepared.n;
	const uintptr_t lo = (uintptr_t)g_prepared.data, hi = lo + extent * sizeof(double);
	const uintptr_t a = (uintptr_t)dst;
	const bool touches = bytes == 0 ? a < hi : (a < hi && a + bytes > lo);
	if (touches) g_prepared = PreparedPoints();
}

/* the frame of these points (g_frame) and the float copy of the moved points (g_data32) */
static int copy_moved_points_f64(const double* data, int layout, size_t stride, uint32_t dim, uint32_t n, const DeviceInfo& dev)
{
	const size_t data_extent = layout == KMX_AOS ? (size_t)(n - 1) * stride + dim : (size_t)(dim - 1) * stride + n;
	int rc = reserve_f64(&g_data32, &g_data32_cap, data_extent / 2 + 1);
	if (rc) return rc;
	rc = reserve_f64(&g_frame, &g_frame_cap, (size_t)dim + 1);
	if (rc) return rc;
	const dim3 grid((uint32_t)std::min<size_t>((data_extent + 1023) / 1024, (size_t)dev.compute_units * 32));
	if (layout == KMX_AOS) {
		KMX_LAUNCH_KERNEL((point_frame_f64_kernel<KMX_AOS>), dim3(1), dim3(256), 0, stream(), data, stride, dim, n, g_frame);
		KMX_LAUNCH_KERNEL((round_moved_to_float_kernel<KMX_AOS>), grid, dim3(256), 0, stream(), data, (float*)g_data32, data_extent, stride, dim, g_frame);
	}
	else {
		KMX_LAUNCH_KERNEL((point_frame_f64_kernel<KMX_SOA>), dim3(1), dim3(256), 0, stream(), data, stride, dim, n, g_frame);
		KMX_LAUNCH_KERNEL((round_moved_to_float_kernel<KMX_SOA>), grid, dim3(256), 0, stream(), data, (float*)g_data32, data_extent, stride, dim, g_frame);
	}
	KMX_LAUNCH_CHECK("round_moved_to_float_kernel");
	return KMX_OK;
}

} // namespace kmx

using namespace kmx;

extern "C" int kmx_prepare_points_f64(const double* data, int layout, size_t stride, uint32_t dim, uint32_t n)
{
	clear_error();
	g_prepared = PreparedPoints(); /* whatever happens below, the old announcement is over */
	if (dim == 0) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_prepare_points_f64: dim must be positive");
	if (n == 0) return KMX_OK;
	if (!data) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_prepare_points_f64: null device pointer");
	int rc = check_layout_f64("kmx_prepare_points_f64", "data", layout, stride, n, dim);
	if (rc) return rc;
	const DeviceInfo* dev = nullptr;
	rc = device_info(&dev);
	if (rc) return rc;
	rc = copy_moved_points_f64(data, layout, stride, dim, n, *dev);
	if (rc) return rc;
	g_prepared.data = data; g_prepared.layout = layout; g_prepared.stride = stride; g_prepared.dim = dim; g_prepared.n = n;
	return KMX_OK;
}

extern "C" int kmx_forget_points_f64(void)
{
	clear_error();
	g_prepared = PreparedPoints();
	return KMX_OK;
}

extern "C" int kmx_assign_f64(int variant,
                              const double* data, int layout, size_t stride,
                              const double* means, int layout_means, size_t stride_means,
                              const uint32_t* last_assignment, uint32_t* assignment,
                              uint32_t dim, uint32_t k, uint32_t n, kmx_exec_params* exec)
{
	clear_error();
	(void)last_assignment;
	if (!exec) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_assign_f64: exec is null");
	if (dim == 0 || k == 0) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_assign_f64: dim and k must be positive");
	if (n == 0) { exec->block_count = 0; return KMX_OK; }
	if (!data || !means || !assignment) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_assign_f64: null device pointer");
	int rc = check_layout_f64("kmx_assign_f64", "data", layout, stride, n, dim);
	if (rc) return rc;
	rc = check_layout_f64("kmx_assign_f64", "means", layout_means, stride_means, k, dim);
	if (rc) return rc;
	if (variant < KMX_ASSIGN_BASE || variant > KMX_ASSIGN_MFMA_BF16X3)
		return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_assign_f64: unknown variant %d", variant);
	const DeviceInfo* dev = nullptr;
	rc = device_info(&dev);
	if (rc) return rc;
	const bool float_ranking = variant == KMX_ASSIGN_MFMA || variant == KMX_ASSIGN_MFMA_BF16X3 || variant == KMX_ASSIGN_BEST;

	const uint32_t kp = round_up_u32(k, WIDE_GROUP);
	rc = reserve_f64(&g_means_t, &g_means_t_cap, (size_t)kp * dim);
	if (rc) return rc;
	rc = reserve_f64(&g_norms, &g_norms_cap, kp);
	if (rc) return rc;
	rc = reserve_f64(&g_queue, &g_queue_cap, float_ranking ? 1 : (size_t)n / 2 + 1);
	if (rc) return rc;
	rc = reserve_f64(&g_misc, &g_misc_cap, 4);
	if (rc) return rc;
	unsigned long long* misc = (unsigned long long*)g_misc;
	KMX_LAUNCH_KERNEL(reset_f64_kernel, dim3(1), dim3(64), 0, stream(), misc);
	KMX_LAUNCH_CHECK("reset_f64_kernel");
	const dim3 pgrid((kp + 255) / 256);
	if (layout_means == KMX_AOS)
		KMX_LAUNCH_KERNEL(prepare_rows_f64_kernel, dim3((kp + 31) / 32), dim3(256), 0, stream(), means, stride_means, g_means_t, g_norms, misc, dim, k, kp);
	else
		KMX_LAUNCH_KERNEL((prepare_means_f64_kernel<KMX_SOA>), pgrid, dim3(256), 0, stream(), means, stride_means, g_means_t, g_norms, misc, dim, k, kp);
	KMX_LAUNCH_CHECK("prepare_means_f64_kernel");

	const uint32_t* float_queue = nullptr;
	const uint32_t* float_queue_length = nullptr;
	if (float_ranking) {
		/* float copies with the layouts and strides of the originals */
		const size_t means_extent = layout_means == KMX_AOS ? (size_t)(k - 1) * stride_means + dim : (size_t)(dim - 1) * stride_means + k;
		rc = reserve_f64(&g_means32, &g_means32_cap, means_extent / 2 + 1);
		if (rc) return rc;
		if (!g_prepared.holds(data, layout, stride, dim, n)) {
			g_prepared = PreparedPoints(); /* the copy is about to hold other points */
			rc = copy_moved_points_f64(data, layout, stride, dim, n, *dev);
			if (rc) return rc;
		}
		/* the centroids in the frame of the points' copy */
		const dim3 mgrid((uint32_t)std::min<size_t>((means_extent + 1023) / 1024, (size_t)dev->compute_units * 32));
		if (layout_means == KMX_AOS)
			KMX_LAUNCH_KERNEL((round_moved_to_float_kernel<KMX_AOS>), mgrid, dim3(256), 0, stream(), means, (float*)g_means32, means_extent, stride_means, dim, g_frame);
		else
			KMX_LAUNCH_KERNEL((round_moved_to_float_kernel<KMX_SOA>), mgrid, dim3(256), 0, stream(), means, (float*)g_means32, means_extent, stride_means, dim, g_frame);
		KMX_LAUNCH_CHECK("round_moved_to_float_kernel");
		Workspace* ws = nullptr;
		rc = workspace(&ws);
		if (rc) return rc;
		AssignArgs a{ (const float*)g_data32, layout, stride, (const float*)g_means32, layout_means, stride_means, assignment, dim, k, n };
		a.kd_extra = 6.0f * 1.1920929e-07f;
		a.ranking_only = true;
		int chosen = -1;
		rc = dispatch_assign(variant, a, exec, ws, *dev, &chosen); /* brackets its sweep for the profile itself */
		if (rc) return rc;
		if (chosen == KMX_ASSIGN_BASE) /* no float sweep fits the shape: evaluate everything on the doubles */
			variant = KMX_ASSIGN_BASE;
		else {
			float_queue = ws->queue;
			float_queue_length = ws->counters;
		}
	}

	if (!float_queue) {
		rc = profile_begin(0);
		if (rc) return rc;
	}
	rc = layout == KMX_AOS ? launch_assign_f64_ld<KMX_AOS>(variant, data, stride, assignment, dim, k, kp, n, exec, *dev, float_queue, float_queue_length)
	                       : launch_assign_f64_ld<KMX_SOA>(variant, data, stride, assignment, dim, k, kp, n, exec, *dev, float_queue, float_queue_length);
	if (rc) return rc;
	if (float_queue) return KMX_OK;
	rc = profile_end(0);
	if (rc) return rc;
	Workspace* ws = nullptr;
	rc = workspace(&ws);
	if (rc) return rc;
	KMX_LAUNCH_KERNEL(publish_queue_length_kernel, dim3(1), dim3(64), 0, stream(), misc, ws->counters, variant == KMX_ASSIGN_LDS_FMA);
	KMX_LAUNCH_CHECK("publish_queue_length_kernel");
	return KMX_OK;
}

static int update_f64_call(const char* who, bool divide, int variant,
                           const double* data, int layout, size_t stride,
                           const uint32_t* assignment,
                           double* means, int layout_means, size_t stride_means,
                           uint32_t* cluster_sizes,
                           uint32_t dim, uint32_t k, uint32_t n, kmx_exec_params* exec)
{
	if (!exec) return fail(KMX_ERR_INVALID_ARGUMENT, "%s: exec is null", who);
	if (dim == 0 || k == 0) return fail(KMX_ERR_INVALID_ARGUMENT, "%s: dim and k must be positive", who);
	if (!means || !cluster_sizes) return fail(KMX_ERR_INVALID_ARGUMENT, "%s: null device pointer", who);
	if (n > 0 && (!data || !assignment)) return fail(KMX_ERR_INVALID_ARGUMENT, "%s: null device pointer", who);
	int rc = check_layout_f64(who, "data", layout, stride, n, dim);
	if (rc) return rc;
	rc = check_layout_f64(who, "means", layout_means, stride_means, k, dim);
	if (rc) return rc;
	if ((variant < KMX_UPDATE_ATOMIC_POINT || variant > KMX_UPDATE_ATOMIC_SHM) && variant != KMX_UPDATE_SERIAL_ORDER)
		return fail(KMX_ERR_INVALID_ARGUMENT, "%s: unknown variant %d (doubles: ATOMIC_POINT, ATOMIC_FINE, ATOMIC_SHM, SERIAL_ORDER)", who, variant);
	if (exec->privatized_copies > 1)
		return fail(KMX_ERR_UNSUPPORTED, "%s: privatized copies in global memory are not built for doubles", who);
	if ((uint64_t)k * dim > 0xffffffffull) return fail(KMX_ERR_UNSUPPORTED, "%s: k * dim does not fit 32 bits", who);
	const DeviceInfo* dev = nullptr;
	rc = device_info(&dev);
	if (rc) return rc;
	if (variant == KMX_UPDATE_SERIAL_ORDER) {
		Workspace* ws = nullptr;
		rc = workspace(&ws);
		if (rc) return rc;
		return launch_update_serial_order<double>(data, layout, stride, assignment, means, layout_means, stride_means, cluster_sizes, dim, k, n, divide, exec, ws, *dev);
	}

	rc = profile_begin(1);
	if (rc) return rc;
#define KMX_F64_UPDATE(LD, LM) \
	launch_update_f64_t<LD, LM>(variant, data, stride, assignment, means, stride_means, cluster_sizes, dim, k, n, exec, *dev, divide)
	if (layout == KMX_AOS) rc = layout_means == KMX_AOS ? KMX_F64_UPDATE(KMX_AOS, KMX_AOS) : KMX_F64_UPDATE(KMX_AOS, KMX_SOA);
	else rc = layout_means == KMX_AOS ? KMX_F64_UPDATE(KMX_SOA, KMX_AOS) : KMX_F64_UPDATE(KMX_SOA, KMX_SOA);
#undef KMX_F64_UPDATE
	if (rc) return rc;
	return profile_end(1);
}

extern "C" int kmx_update_f64(int variant,
                              const double* data, int layout, size_t stride,
                              const uint32_t* assignment,
                              double* means, int layout_means, size_t stride_means,
                              uint32_t* cluster_sizes,
                              uint32_t dim, uint32_t k, uint32_t n, kmx_exec_params* exec)
{
	clear_error();
	return update_f64_call("kmx_update_f64", true, variant, data, layout, stride, assignment, means, layout_means, stride_means, cluster_sizes,
	                       dim, k, n, exec);
}

extern "C" int kmx_bucket_sum_f64(int variant,
                                  const double* data, int layout, size_t stride,
                                  const uint32_t* indices,
                                  double* result, int layout_result, size_t stride_result,
                                  uint32_t dim, uint32_t k, uint32_t n, kmx_exec_params* exec)
{
	clear_error();
	if (k == 0) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_bucket_sum_f64: dim and k must be positive");
	Workspace* ws = nullptr;
	int rc = workspace(&ws);
	if (rc) return rc;
	/* the kernels count members as they go; the counts land in a scratch array */
	rc = reserve_bucket_sizes(ws, k);
	if (rc) return rc;
	rc = kmx_fill_zero_u32(ws->bucket_sizes, k);
	if (rc) return rc;
	return update_f64_call("kmx_bucket_sum_f64", false, variant, data, layout, stride, indices, result, layout_result, stride_result,
	                       ws->bucket_sizes, dim, k, n, exec);
}

extern "C" int kmx_fused_f64(int variant,
                             const double* data, int layout, size_t stride,
                             const double* means_in, double* means_out, int layout_means, size_t stride_means,
                             uint32_t* cluster_sizes,
                             uint32_t dim, uint32_t k, uint32_t n, kmx_exec_params* exec)
{
	clear_error();
	if (variant == KMX_FUSED_ONE_PASS)
		return fail(KMX_ERR_UNSUPPORTED, "kmx_fused_f64: the single-pass kernel is not built for doubles");
	if (variant != KMX_FUSED_TWO_PASS && variant != KMX_FUSED_BEST)
		return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_fused_f64: unknown variant %d", variant);
	Workspace* ws = nullptr;
	int rc = workspace(&ws);
	if (rc) return rc;
	rc = reserve_fused_assignment(ws, std::max<size_t>(n, 1));
	if (rc) return rc;
	/* argument checks of the two halves apply unchanged (their messages name the half that objects) */
	rc = kmx_assign_f64(KMX_ASSIGN_BEST, data, layout, stride, means_in, layout_means, stride_means, nullptr, ws->fused_assignment, dim, k, n, exec);
	if (rc) return rc;
	return kmx_update_f64(KMX_UPDATE_ATOMIC_SHM, data, layout, stride, ws->fused_assignment, means_out, layout_means, stride_means,
	                      cluster_sizes, dim, k, n, exec);
}
