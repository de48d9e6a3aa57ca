/*
 * Assignment with the serial arithmetic, operation for operation:
 *   dist(x, c) = sqrt( (((x0-c0)^2 + (x1-c1)^2) + ...) ), every subtract / multiply / add
 *   rounded separately in fp32, d ascending (reference metric_policies.hpp:23-28,40-44);
 *   argmin with strict comparison from centroid 0, so the lowest index wins equal distances
 *   and NaN distances never win (reference serial.hpp:21-35).
 *
 *   assign_base_kernel  - one lane per point; counterpart of baseAssignmentKernel
 *                         (reference kernels.cu:180-199) and the `hip_base` algorithm.
 *   recheck_kernel,     - the exact pass behind the fast variants (they queue the points whose
 *   recheck_reg_kernel    ranking by |c|^2 - 2x.c is not decided beyond rounding error).
 *
 * Floating-point contraction is switched off for the whole file: a fused multiply-add here
 * would change low-order bits and with them the tie-breaks.
 */
#include "assign_mfma_impl.h"

#pragma clang fp contract(off)

namespace kmx {

template <int LD, int LM>
__device__ __forceinline__ float exact_distance(const float* __restrict__ data, size_t stride, size_t idx,
                                                const float* __restrict__ means, size_t stride_means, size_t m, uint32_t dim)
{
	float sum = 0.0f;
	for (uint32_t d = 0; d < dim; ++d) {
		float diff = data[elem<LD>(stride, idx, d)] - means[elem<LM>(stride_means, m, d)];
		float sq = diff * diff;
		sum = sum + sq;
	}
	return __builtin_sqrtf(sum);
}

template <int LD, int LM>
__global__ void __launch_bounds__(256)
assign_base_kernel(const float* __restrict__ data, size_t stride, const float* __restrict__ means, size_t stride_means,
                   uint32_t* __restrict__ assignment, uint32_t dim, uint32_t k, uint32_t n, uint32_t* __restrict__ counters)
{
	uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x;
	if (idx == 0) counters[0] = 0u; /* nothing is rechecked by this variant */
	if (idx >= n) return;
	float minDist = exact_distance<LD, LM>(data, stride, idx, means, stride_means, 0, dim);
	uint32_t nearest = 0;
	for (uint32_t m = 1; m < k; ++m) {
		float dist = exact_distance<LD, LM>(data, stride, idx, means, stride_means, m, dim);
		if (minDist > dist) {
			minDist = dist;
			nearest = m;
		}
	}
	assignment[idx] = nearest;
}

/*
 * The exact pass behind the fast variants. A queue entry is (point, threshold): the sweep's smallest ranking value
 * a[j] = |c_j|^2 - 2 c_j.x plus its tau. The register kernel (rows up to 64 floats) first SCREENS a centroid with
 * plain fused multiply-adds on the exact centroid copy (the value obeys the sweep's error bound, so a centroid whose
 * value exceeds the threshold has a strictly larger serial distance than the sweep's best one and cannot be the
 * result) and evaluates the serial arithmetic only for the centroids that pass: typically two or three of k. A lane
 * notes up to SCREEN_CAP passing centroids and evaluates them after its scan, so that the wavefront runs the
 * expensive block a few times instead of whenever any of its lanes has a hit; beyond SCREEN_CAP (duplicated
 * centroids, NaN data: `!(a > threshold)` passes everything that is not a number) the lane evaluates on the spot.
 * The kernel for wider rows evaluates every centroid (measured: screening did not pay there, the centroid block is
 * read twice). The merge by (smaller distance, then smaller index) over all evaluated centroids is the serial scan's
 * result: the first centroid attaining the minimum. A NaN distance to centroid 0 pins the point to centroid 0, as
 * `minDist > dist` is then never true (centroid 0 always passes the screen in that case: its ranking value is NaN
 * as well).
 */
constexpr int SCREEN_CAP = 4;

/*
 * Any dimension. A work-group of 256 lanes owns a batch of PB queued points: their coordinates are staged in LDS
 * (rows padded with zeros to a multiple of 4 floats, so that every lane fetches four coordinates with one broadcast
 * 128-bit read), lane t handles centroids t, t+256, ... against all PB points (16 coalesced loads of the transposed
 * centroid block in flight, each value reused PB times) and keeps its own (distance, index) minimum per point.
 * Zero padding is exact: (0-0)^2 = +0 leaves a partial sum unchanged.
 * means_t is the exact transposed copy [dim][kp] written by the pack kernels.
 */
template <int LD, int PB>
__global__ void __launch_bounds__(256)
recheck_kernel(const float* __restrict__ data, size_t stride, const float* __restrict__ means_t, uint32_t kp,
               uint32_t* __restrict__ assignment, uint32_t dim, uint32_t k,
               const uint32_t* __restrict__ queue, const uint32_t* __restrict__ counters)
{
	extern __shared__ float xs[]; /* PB rows of dim4 floats */
	__shared__ float cand_dist[4][PB];
	__shared__ uint32_t cand_idx[4][PB];
	__shared__ uint32_t pinned_mask;
	typedef float f4 __attribute__((ext_vector_type(4)));
	const uint32_t dim4 = (dim + 3) / 4 * 4;
	const uint32_t lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
	const uint32_t count = counters[0];
	const uint32_t batches = (count + PB - 1) / PB;

	for (uint32_t batch = blockIdx.x; batch < batches; batch += gridDim.x) {
		__syncthreads(); /* the previous batch's coordinates and candidates are no longer needed */
		for (uint32_t i = threadIdx.x; i < PB * dim4; i += blockDim.x) {
			const uint32_t p = i / dim4, d = i - p * dim4;
			const uint32_t idx = queue[2 * (size_t)min(batch * PB + p, count - 1)];
			xs[i] = d < dim ? data[elem<LD>(stride, idx, d)] : 0.0f;
		}
		__syncthreads();

		float best[PB];
		uint32_t bestIdx[PB];
		uint32_t pinned = 0;
#pragma unroll
		for (int p = 0; p < PB; ++p) {
			best[p] = __builtin_inff();
			bestIdx[p] = 0xFFFFFFFFu;
		}
		auto evaluate = [&](uint32_t m) {
			float sum[PB];
#pragma unroll
			for (int p = 0; p < PB; ++p) sum[p] = 0.0f;
			for (uint32_t d0 = 0; d0 < dim4; d0 += 16) {
				float c[16];
#pragma unroll
				for (int u = 0; u < 16; ++u) c[u] = d0 + u < dim ? means_t[(size_t)(d0 + u) * kp + m] : 0.0f;
#pragma unroll
				for (int u4 = 0; u4 < 4; ++u4) {
					if (d0 + 4 * u4 < dim4) { /* uniform: whole groups of four padded coordinates */
#pragma unroll
						for (int p = 0; p < PB; ++p) {
							const f4 x = *(const f4*)(xs + p * dim4 + d0 + 4 * u4);
#pragma unroll
							for (int q = 0; q < 4; ++q) {
								float diff = x[q] - c[4 * u4 + q];
								float sq = diff * diff;
								sum[p] = sum[p] + sq;
							}
						}
					}
				}
			}
#pragma unroll
			for (int p = 0; p < PB; ++p) {
				float dist = __builtin_sqrtf(sum[p]);
				if (m == 0 && dist != dist) pinned |= 1u << p;
				if (dist < best[p] || (dist == best[p] && m < bestIdx[p])) {
					best[p] = dist;
					bestIdx[p] = m;
				}
			}
		};
		for (uint32_t m = threadIdx.x; m < k; m += blockDim.x) evaluate(m);
		if (threadIdx.x == 0) pinned_mask = pinned; /* lane 0 handles centroid 0 */
#pragma unroll
		for (int p = 0; p < PB; ++p) {
			for (int off = WAVE / 2; off > 0; off >>= 1) {
				float ob = __shfl_xor(best[p], off);
				uint32_t oi = (uint32_t)__shfl_xor((int)bestIdx[p], off);
				if (ob < best[p] || (ob == best[p] && oi < bestIdx[p])) {
					best[p] = ob;
					bestIdx[p] = oi;
				}
			}
			if (lane == 0) {
				cand_dist[wave][p] = best[p];
				cand_idx[wave][p] = bestIdx[p];
			}
		}
		__syncthreads();
		if (threadIdx.x < PB) {
			const uint32_t p = threadIdx.x;
			float b = cand_dist[0][p];
			uint32_t bi = cand_idx[0][p];
			for (int w = 1; w < 4; ++w) {
				const float ob = cand_dist[w][p];
				const uint32_t oi = cand_idx[w][p];
				if (ob < b || (ob == b && oi < bi)) {
					b = ob;
					bi = oi;
				}
			}
			const uint32_t q = batch * PB + p;
			if (q < count) {
				const bool pin = (pinned_mask >> p) & 1u;
				assignment[queue[2 * (size_t)q]] = (pin || bi == 0xFFFFFFFFu) ? 0u : bi;
			}
		}
	}
}

/*
 * dim <= DPAD <= 64 without LDS: the PB points of a batch live in registers (every lane of the group of L lanes loads
 * the same words, a broadcast), lane t of the group handles centroids t, t+L, ...; all DPAD coordinates of a centroid
 * are requested before the first use, so their latency overlaps. Dimensions beyond dim are fed as x = c = 0: adding
 * (0-0)^2 = +0 leaves every partial sum unchanged, so the padding is exact.
 */
template <int LD, int L, int PB, int DPAD>
__global__ void __launch_bounds__(256)
recheck_reg_kernel(const float* __restrict__ data, size_t stride, const float* __restrict__ means_t, uint32_t kp,
                   uint32_t* __restrict__ assignment, uint32_t dim, uint32_t k,
                   const uint32_t* __restrict__ queue, const uint32_t* __restrict__ counters, uint32_t vec4)
{
	typedef float f4 __attribute__((ext_vector_type(4)));
	constexpr uint32_t GROUPS = 256 / L;
	const uint32_t group = threadIdx.x / L;
	const uint32_t gl = threadIdx.x % L;
	const uint32_t count = counters[0];
	const uint32_t batches = (count + PB - 1) / PB;

	for (uint32_t batch = blockIdx.x * GROUPS + group; batch < batches; batch += gridDim.x * GROUPS) {
		float x[PB][DPAD];
		float thr[PB];
		uint32_t idx[PB];
#pragma unroll
		for (int p = 0; p < PB; ++p) {
			const size_t entry = 2 * (size_t)min(batch * PB + p, count - 1);
			idx[p] = queue[entry];
			thr[p] = __uint_as_float(queue[entry + 1]);
			if (LD == KMX_AOS && vec4) { /* rows of whole, aligned 16-byte pieces: a quarter of the load instructions */
#pragma unroll
				for (int d = 0; d < DPAD; d += 4) {
					f4 v = { 0.0f, 0.0f, 0.0f, 0.0f };
					if ((uint32_t)d < dim) v = *(const f4*)(data + (size_t)idx[p] * stride + d);
					x[p][d] = v.x; x[p][d + 1] = v.y; x[p][d + 2] = v.z; x[p][d + 3] = v.w;
				}
			}
			else {
#pragma unroll
				for (int d = 0; d < DPAD; ++d) x[p][d] = (uint32_t)d < dim ? data[elem<LD>(stride, idx[p], d)] : 0.0f;
			}
		}
		float best[PB];
		uint32_t bestIdx[PB];
		uint32_t pinned = 0;
#pragma unroll
		for (int p = 0; p < PB; ++p) {
			best[p] = __builtin_inff();
			bestIdx[p] = 0xFFFFFFFFu;
		}
		auto evaluate = [&](uint32_t m, const float (&c)[DPAD]) {
			float sum[PB];
#pragma unroll
			for (int p = 0; p < PB; ++p) sum[p] = 0.0f;
#pragma unroll
			for (int d = 0; d < DPAD; ++d) {
#pragma unroll
				for (int p = 0; p < PB; ++p) {
					float diff = x[p][d] - c[d];
					float sq = diff * diff;
					sum[p] = sum[p] + sq;
				}
			}
#pragma unroll
			for (int p = 0; p < PB; ++p) {
				float dist = __builtin_sqrtf(sum[p]);
				if (m == 0 && dist != dist) pinned |= 1u << p;
				if (dist < best[p] || (dist == best[p] && m < bestIdx[p])) {
					best[p] = dist;
					bestIdx[p] = m;
				}
			}
		};
		uint32_t noted[SCREEN_CAP];
		uint32_t notes = 0;
		for (uint32_t m = gl; m < k; m += L) {
			float c[DPAD];
#pragma unroll
			for (int d = 0; d < DPAD; ++d) c[d] = (uint32_t)d < dim ? means_t[(size_t)d * kp + m] : 0.0f;
			float c2 = 0.0f;
			float dot[PB];
#pragma unroll
			for (int p = 0; p < PB; ++p) dot[p] = 0.0f;
#pragma unroll
			for (int d = 0; d < DPAD; ++d) {
				c2 = __builtin_fmaf(c[d], c[d], c2);
#pragma unroll
				for (int p = 0; p < PB; ++p) dot[p] = __builtin_fmaf(c[d], x[p][d], dot[p]);
			}
			bool pass = false;
#pragma unroll
			for (int p = 0; p < PB; ++p) pass = pass || !(__builtin_fmaf(-2.0f, dot[p], c2) > thr[p]);
			if (pass) {
				if (notes < SCREEN_CAP) {
#pragma unroll
					for (int i = 0; i < SCREEN_CAP; ++i)
						if (notes == (uint32_t)i) noted[i] = m;
					++notes;
				}
				else evaluate(m, c);
			}
		}
#pragma unroll
		for (int i = 0; i < SCREEN_CAP; ++i) {
			if ((uint32_t)i < notes) {
				float c[DPAD];
#pragma unroll
				for (int d = 0; d < DPAD; ++d) c[d] = (uint32_t)d < dim ? means_t[(size_t)d * kp + noted[i]] : 0.0f;
				evaluate(noted[i], c);
			}
		}
		pinned = (uint32_t)__shfl((int)pinned, 0, L); /* lane 0 of the group handles centroid 0 */
#pragma unroll
		for (int p = 0; p < PB; ++p) {
			for (int off = L / 2; off > 0; off >>= 1) {
				float ob = __shfl_xor(best[p], off, L);
				uint32_t oi = (uint32_t)__shfl_xor((int)bestIdx[p], off, L);
				if (ob < best[p] || (ob == best[p] && oi < bestIdx[p])) {
					best[p] = ob;
					bestIdx[p] = oi;
				}
			}
			const uint32_t q = batch * PB + p;
			if (gl == 0 && q < count) {
				const bool pin = (pinned >> p) & 1u;
				assignment[idx[p]] = (pin || bestIdx[p] == 0xFFFFFFFFu) ? 0u : bestIdx[p];
			}
		}
	}
}

/*
 * Exact pass with one lane per CENTROID and the queued points as scalar operands, for rows that fit the registers.
 * A work-group of up to 16 wavefronts holds a chunk of up to 1024 centroids, one exact row per lane (read from the
 * transposed exact copy, coalesced), and walks a batch of queue entries: the point of an entry is the same for
 * every lane, so its coordinates and its threshold arrive as scalar loads (one cache fill serves all wavefronts)
 * and feed the multiply-adds directly. A lane whose ranking value does not exceed the threshold evaluates the
 * serial arithmetic for its centroid. The per-point minimum over all lanes and chunks is a 64-bit LDS atomic over
 * (distance bits << 32 | centroid): for non-negative distances the bit pattern orders like the value, equal
 * distances resolve to the smaller index, a NaN never beats a number, and key 0 encodes "NaN distance to
 * centroid 0", which pins the point there as the serial scan does. The sweep's best centroid always passes the
 * screen, so every point gets a key (a point without one -- only NaN coordinates do that -- goes to centroid 0).
 * The batch size adapts to the queue length so that a short queue still spreads over the whole chip.
 * The rows of a batch are first copied to LDS with vector loads (padded with zeros), and the walk reads them from there,
 * four coordinates per broadcast read, instead of through the scalar cache, which delivers about one dword per cycle to
 * the compute units that share it: N = 2M, d = 32, k = 1024, 80 k queued points: 127 -> 109 us; d = 8: 8 % of the call.
 */
/*
 * The points of a batch are scattered rows of the input: a load that misses all the way to HBM takes thousands of
 * cycles. While a batch is worked on, the lanes therefore touch the rows of the batch this work-group takes next with
 * ordinary vector loads (one per 64 bytes of a row), which brings them into the L2 before they are copied to LDS.
 */
template <int LD>
static __device__ __forceinline__ float touch_rows(const float* __restrict__ data, size_t stride, uint32_t dim,
                                                   const uint32_t* __restrict__ queue, uint32_t first, uint32_t points)
{
	const uint32_t parts = (dim + 15) / 16;
	float touched = 0.0f;
	for (uint32_t t = threadIdx.x; t < points * parts; t += blockDim.x)
		touched += data[elem<LD>(stride, queue[2 * (size_t)(first + t / parts)], (t % parts) * 16)];
	return touched;
}

constexpr uint32_t HIT_CAP = 1024;

constexpr uint32_t POINTS_BATCH = 64;

template <int LD, int DPAD, bool FULL, int CPL> /* FULL: dim == DPAD, no guards on the coordinate loads; CPL: centroids per lane */
__global__ void __launch_bounds__(1024)
recheck_points_kernel(const float* __restrict__ data, size_t stride, const float* __restrict__ means_t, const float* __restrict__ norms,
                      uint32_t* __restrict__ assignment, uint32_t dim, uint32_t k, uint32_t kp,
                      const uint32_t* __restrict__ queue, const uint32_t* __restrict__ counters)
{
	__shared__ unsigned long long best_key[POINTS_BATCH];
	__shared__ uint32_t hit_point[DPAD >= 16 ? HIT_CAP : 1], hit_centroid[DPAD >= 16 ? HIT_CAP : 1];
	__shared__ uint32_t hit_count;
	/* the rows of a batch, padded with zeros to DPAD: every lane reads the same coordinates, four per LDS read */
	__shared__ __attribute__((aligned(16))) float batch_rows[POINTS_BATCH * DPAD];
	/* the wavefront number through readfirstlane: the compiler then knows that what depends on it is uniform */
	const uint32_t count = counters[0];
	const uint32_t slots = gridDim.x;
	const uint32_t pb = min(POINTS_BATCH, max(16u, (count + slots - 1) / slots)); /* one batch per work-group while 64 points suffice for that */
	const uint32_t batches = (count + pb - 1) / pb;

	for (uint32_t batch = blockIdx.x; batch < batches; batch += gridDim.x) {
		__syncthreads(); /* the previous batch has been written out */
		if (threadIdx.x < POINTS_BATCH) best_key[threadIdx.x] = ~0ull;
		if (threadIdx.x == 0) hit_count = 0;
		__syncthreads();
		const uint32_t first = batch * pb, here = min(pb, count - first);
		const uint32_t next = (batch + gridDim.x) * pb;
		for (uint32_t t = threadIdx.x; t < here * DPAD; t += blockDim.x) {
			const uint32_t i = t / DPAD, q = t % DPAD;
			batch_rows[t] = (FULL || q < dim) ? data[elem<LD>(stride, queue[2 * (size_t)(first + i)], q)] : 0.0f;
		}
		const float touched = next < count ? touch_rows<LD>(data, stride, dim, queue, next, min(pb, count - next)) : 0.0f;
		__syncthreads(); /* the rows are in place */
		for (uint32_t base = 0; base < k; base += blockDim.x * CPL) {
			/* The scalar cache delivers about one dword per cycle to the compute units that share it, which is half of
			 * what their SIMDs consume when every multiply-add takes a fresh scalar operand: with two centroids per lane
			 * every coordinate of a point is used twice. */
			uint32_t r[CPL];
			float c[CPL][DPAD], c2[CPL];
#pragma unroll
			for (int u = 0; u < CPL; ++u) {
				r[u] = base + u * blockDim.x + threadIdx.x;
				const uint32_t rr = min(r[u], k - 1); /* lanes past the end load a valid row, unconditionally, and never pass the screen */
#pragma unroll
				for (int q = 0; q < DPAD; ++q) c[u][q] = (FULL || (uint32_t)q < dim) ? means_t[(size_t)q * kp + rr] : 0.0f;
				c2[u] = r[u] < k ? norms[norm_at(r[u])] : __builtin_inff();
			}
#pragma unroll 2
			for (uint32_t i = 0; i < here; ++i) {
				const uint32_t pt = queue[2 * (size_t)(first + i)]; /* uniform: scalar loads */
				const float thr = __uint_as_float(queue[2 * (size_t)(first + i) + 1]);
				float x[DPAD < 16 ? DPAD : 4]; /* (short rows are evaluated from these registers below) */
				float dot[CPL];
#pragma unroll
				for (int u = 0; u < CPL; ++u) dot[u] = 0.0f;
#pragma unroll
				for (int q = 0; q < DPAD; q += 4) {
					const f32x4 v = *(const f32x4*)(batch_rows + i * DPAD + q);
					const int at = DPAD < 16 ? q : 0;
					x[at] = v.x; x[at + 1] = v.y; x[at + 2] = v.z; x[at + 3] = v.w;
#pragma unroll
					for (int j = 0; j < 4; ++j) {
#pragma unroll
						for (int u = 0; u < CPL; ++u) dot[u] = __builtin_fmaf(x[at + j], c[u][q + j], dot[u]);
					}
				}
#pragma unroll
				for (int u = 0; u < CPL; ++u) {
					if (r[u] < k && !(__builtin_fmaf(-2.0f, dot[u], c2[u]) > thr)) {
						if constexpr (DPAD >= 16) { /* noted, and evaluated below by one lane per pair */
							const uint32_t slot = atomicAdd(&hit_count, 1u);
							if (slot < HIT_CAP) { hit_point[slot] = i; hit_centroid[slot] = r[u]; }
							else evaluate_pair<LD>(data, stride, means_t, dim, kp, pt, r[u], &best_key[i]);
						} else { /* a short row is evaluated on the spot from the registers */
							float sum = 0.0f;
#pragma unroll
							for (int q = 0; q < DPAD; ++q) { /* padding: (0-0)^2 = +0 leaves the sum unchanged */
								float diff = x[q] - c[u][q];
								float sq = diff * diff;
								sum = sum + sq;
							}
							const float dist = __builtin_sqrtf(sum);
							const unsigned long long key = (r[u] == 0 && dist != dist) ? 0ull : (((unsigned long long)__float_as_uint(dist) << 32) | r[u]);
							atomicMin(&best_key[i], key);
						}
					}
				}
			}
		}
		asm volatile("" :: "v"(touched)); /* the touching loads are not dead code */
		__syncthreads();
		if constexpr (DPAD >= 16) {
			const uint32_t noted = min(hit_count, HIT_CAP);
			for (uint32_t t = threadIdx.x; t < noted; t += blockDim.x) {
				const uint32_t i = hit_point[t];
				evaluate_pair<LD>(data, stride, means_t, dim, kp, queue[2 * (size_t)(first + i)], hit_centroid[t], &best_key[i]);
			}
			__syncthreads();
		}
		if (threadIdx.x < here) {
			const unsigned long long key = best_key[threadIdx.x];
			assignment[queue[2 * (size_t)(first + threadIdx.x)]] = key == ~0ull ? 0u : (uint32_t)key;
		}
	}
}

/*
 * The same scheme for rows too long for the registers: the dimensions go by in slices of 32. A lane keeps the
 * running dot products of its centroid with the 16 points of the batch, loads one slice of its centroid and
 * applies it to the 16 points in turn (their slices are scalar loads). Centroids that pass the screen of a point
 * are noted in an LDS list, and when all centroids are through, one lane per noted (point, centroid) pair evaluates
 * the serial arithmetic from memory: evaluating on the spot would leave 63 lanes of the wavefront waiting for
 * every pair. Pairs beyond the list's capacity (many coincident centroids) are evaluated on the spot.
 */
constexpr int SLICE = 32;
constexpr int SLICED_BATCH = 16;

template <int LD, bool FULL> /* FULL: dim is a multiple of the slice, no guards on the coordinate loads */
__global__ void __launch_bounds__(1024)
recheck_sliced_kernel(const float* __restrict__ data, size_t stride, const float* __restrict__ means_t, const float* __restrict__ norms,
                      uint32_t* __restrict__ assignment, uint32_t dim, uint32_t k, uint32_t kp,
                      const uint32_t* __restrict__ queue, const uint32_t* __restrict__ counters)
{
	__shared__ unsigned long long best_key[SLICED_BATCH];
	__shared__ uint32_t hit_point[HIT_CAP], hit_centroid[HIT_CAP];
	__shared__ uint32_t hit_count;
	const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
	const uint32_t count = counters[0];
	const uint32_t batches = (count + SLICED_BATCH - 1) / SLICED_BATCH;

	for (uint32_t batch = blockIdx.x; batch < batches; batch += gridDim.x) {
		__syncthreads(); /* the previous batch has been written out */
		if (threadIdx.x < SLICED_BATCH) best_key[threadIdx.x] = ~0ull;
		if (threadIdx.x == 0) hit_count = 0;
		__syncthreads();
		const uint32_t first = batch * SLICED_BATCH, here = min((uint32_t)SLICED_BATCH, count - first);
		const uint32_t next = (batch + gridDim.x) * SLICED_BATCH;
		const float touched = next < count ? touch_rows<LD>(data, stride, dim, queue, next, min((uint32_t)SLICED_BATCH, count - next)) : 0.0f;
		/* register i of this wavefront belongs to point at(i) of the batch: another rotation in every wavefront */
		auto at = [&](int i) { return min((uint32_t)(i + wave) % SLICED_BATCH, here - 1); };
		for (uint32_t base = 0; base < k; base += blockDim.x) {
			const uint32_t r = base + threadIdx.x, rr = min(r, k - 1); /* lanes past the end load a valid row, unconditionally, and never pass the screen */
			float dots[SLICED_BATCH];
#pragma unroll
			for (int i = 0; i < SLICED_BATCH; ++i) dots[i] = 0.0f;
			for (uint32_t q0 = 0; q0 < dim; q0 += SLICE) {
				float c[SLICE];
#pragma unroll
				for (int j = 0; j < SLICE; ++j) c[j] = (FULL || q0 + j < dim) ? means_t[(size_t)(q0 + j) * kp + rr] : 0.0f;
#pragma unroll
				for (int i = 0; i < SLICED_BATCH; ++i) {
					const uint32_t pt = queue[2 * (size_t)(first + at(i))]; /* uniform: scalar loads */
					float x[SLICE];
#pragma unroll
					for (int j = 0; j < SLICE; ++j) x[j] = (FULL || q0 + j < dim) ? data[elem<LD>(stride, pt, q0 + j)] : 0.0f;
#pragma unroll
					for (int j = 0; j < SLICE; ++j) dots[i] = __builtin_fmaf(x[j], c[j], dots[i]);
				}
			}
			const float c2 = r < k ? norms[norm_at(r)] : __builtin_inff();
#pragma unroll
			for (int i = 0; i < SLICED_BATCH; ++i) {
				const uint32_t point = at(i);
				const size_t entry = 2 * (size_t)(first + point);
				const float thr = __uint_as_float(queue[entry + 1]);
				/* a batch that is not full has several registers on its last point: the first of them speaks for it */
				const bool mine = (uint32_t)(i + wave) % SLICED_BATCH == point;
				if (mine && r < k && !(__builtin_fmaf(-2.0f, dots[i], c2) > thr)) {
					const uint32_t slot = atomicAdd(&hit_count, 1u);
					if (slot < HIT_CAP) { hit_point[slot] = point; hit_centroid[slot] = r; }
					else evaluate_pair<LD>(data, stride, means_t, dim, kp, queue[entry], r, &best_key[point]);
				}
			}
		}
		asm volatile("" :: "v"(touched)); /* the touching loads are not dead code */
		__syncthreads();
		const uint32_t noted = min(hit_count, HIT_CAP);
		for (uint32_t t = threadIdx.x; t < noted; t += blockDim.x) {
			const uint32_t i = hit_point[t];
			evaluate_pair<LD>(data, stride, means_t, dim, kp, queue[2 * (size_t)(first + i)], hit_centroid[t], &best_key[i]);
		}
		__syncthreads();
		if (threadIdx.x < here) {
			const unsigned long long key = best_key[threadIdx.x];
			assignment[queue[2 * (size_t)(first + threadIdx.x)]] = key == ~0ull ? 0u : (uint32_t)key;
		}
	}
}

template <int LD, int LM>
static int launch_base_t(const AssignArgs& a, kmx_exec_params* exec, uint32_t* counters)
{
	uint32_t block = exec->block_size ? exec->block_size : 256;
	if (block > 256) block = 256;
	block = (block + WAVE - 1) / WAVE * WAVE;
	exec->block_count = (a.n + block - 1) / block;
	int rc = profile_begin(0);
	if (rc) return rc;
	KMX_LAUNCH_KERNEL((assign_base_kernel<LD, LM>), dim3(exec->block_count), dim3(block), 0, stream(),
	                   a.data, a.stride, a.means, a.stride_means, a.assignment, a.dim, a.k, a.n, counters);
	KMX_LAUNCH_CHECK("assign_base_kernel");
	return profile_end(0);
}

int launch_assign_base(const AssignArgs& a, kmx_exec_params* exec)
{
	Workspace* ws = nullptr;
	int rc = workspace(&ws);
	if (rc) return rc;
	if (a.layout == KMX_AOS && a.layout_means == KMX_AOS) return launch_base_t<KMX_AOS, KMX_AOS>(a, exec, ws->counters);
	if (a.layout == KMX_AOS && a.layout_means == KMX_SOA) return launch_base_t<KMX_AOS, KMX_SOA>(a, exec, ws->counters);
	if (a.layout == KMX_SOA && a.layout_means == KMX_AOS) return launch_base_t<KMX_SOA, KMX_AOS>(a, exec, ws->counters);
	return launch_base_t<KMX_SOA, KMX_SOA>(a, exec, ws->counters);
}

template <int LD, int PB>
static int launch_recheck_t(const AssignArgs& a, Workspace* ws, uint32_t kp)
{
	const unsigned block = 256, blocks = 2048;
	const size_t lds = (size_t)PB * ((a.dim + 3) / 4 * 4) * sizeof(float);
	auto kernel = recheck_kernel<LD, PB>;
	if (lds > 48 * 1024) KMX_HIP(hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
	KMX_LAUNCH_KERNEL(kernel, dim3(blocks), dim3(block), lds, stream(),
	                   a.data, a.stride, ws->means_t, kp, a.assignment, a.dim, a.k, ws->queue, ws->counters);
	KMX_LAUNCH_CHECK("recheck_kernel");
	return KMX_OK;
}

template <int LD, int L, int PB, int DPAD>
static int launch_recheck_reg(const AssignArgs& a, Workspace* ws, uint32_t kp)
{
	const uint32_t vec4 = LD == KMX_AOS && a.dim % 4 == 0 && a.stride % 4 == 0 && ((uintptr_t)a.data & 15) == 0;
	KMX_LAUNCH_KERNEL((recheck_reg_kernel<LD, L, PB, DPAD>), dim3(2048), dim3(256), 0, stream(),
	                   a.data, a.stride, ws->means_t, kp, a.assignment, a.dim, a.k, ws->queue, ws->counters, vec4);
	KMX_LAUNCH_CHECK("recheck_reg_kernel");
	return KMX_OK;
}

template <int LD, int L>
static int launch_recheck_dpad(const AssignArgs& a, Workspace* ws, uint32_t kp)
{
	if (a.dim <= 8) return launch_recheck_reg<LD, L, 4, 8>(a, ws, kp);
	if (a.dim <= 16) return launch_recheck_reg<LD, L, 4, 16>(a, ws, kp);
	if (a.dim <= 32) return launch_recheck_reg<LD, L, 4, 32>(a, ws, kp);
	return launch_recheck_reg<LD, L, 2, 64>(a, ws, kp);
}

/* |c|^2 of the centroids as given (a sweep in a moved frame keeps the norms of the moved centroids in ws->norms) */
static const float* exact_norms(const Workspace* ws) { return ws->exact_norms ? ws->exact_norms : ws->norms; }

template <int LD, int DPAD>
static int launch_recheck_points(const AssignArgs& a, Workspace* ws, uint32_t kp)
{
	/* two centroids per lane while their rows fit the registers and the work-group stays large */
	constexpr int CPL = DPAD <= 32 ? 2 : 1;
	const bool two = CPL == 2 && a.k > 512;
	const uint32_t threads = std::min<uint32_t>(1024, round_up(two ? (a.k + 1) / 2 : a.k, WAVE));
	const dim3 grid(DPAD <= 32 ? 512 : 256); /* two work-groups fit a compute unit while the rows of a lane take at most 64 registers */
#define KMX_RECHECK_POINTS(FULL, C) \
	KMX_LAUNCH_KERNEL((recheck_points_kernel<LD, DPAD, FULL, C>), grid, dim3(threads), 0, stream(), \
	                   a.data, a.stride, ws->means_t, exact_norms(ws), a.assignment, a.dim, a.k, kp, ws->queue, ws->counters)
	if (a.dim == DPAD) { if (two) KMX_RECHECK_POINTS(true, CPL); else KMX_RECHECK_POINTS(true, 1); }
	else { if (two) KMX_RECHECK_POINTS(false, CPL); else KMX_RECHECK_POINTS(false, 1); }
#undef KMX_RECHECK_POINTS
	KMX_LAUNCH_CHECK("recheck_points_kernel");
	return KMX_OK;
}

template <int LD>
static int launch_recheck_sliced(const AssignArgs& a, Workspace* ws, uint32_t kp)
{
	const uint32_t threads = std::min<uint32_t>(1024, round_up(a.k, WAVE));
	const dim3 grid(256);
	if (a.dim % SLICE == 0)
		KMX_LAUNCH_KERNEL((recheck_sliced_kernel<LD, true>), grid, dim3(threads), 0, stream(),
		                   a.data, a.stride, ws->means_t, exact_norms(ws), a.assignment, a.dim, a.k, kp, ws->queue, ws->counters);
	else
		KMX_LAUNCH_KERNEL((recheck_sliced_kernel<LD, false>), grid, dim3(threads), 0, stream(),
		                   a.data, a.stride, ws->means_t, exact_norms(ws), a.assignment, a.dim, a.k, kp, ws->queue, ws->counters);
	KMX_LAUNCH_CHECK("recheck_sliced_kernel");
	return KMX_OK;
}

template <int LD>
static int launch_recheck_l(const AssignArgs& a, Workspace* ws, uint32_t kp)
{
	/* rows that fit the registers, many centroids: one lane per centroid, the points as scalar operands */
	if (a.k >= 128 && a.dim <= 32) {
		switch ((a.dim + 3) / 4) {
		case 1: return launch_recheck_points<LD, 4>(a, ws, kp);
		case 2: return launch_recheck_points<LD, 8>(a, ws, kp);
		case 3: return launch_recheck_points<LD, 12>(a, ws, kp);
		case 4: return launch_recheck_points<LD, 16>(a, ws, kp);
		case 5: return launch_recheck_points<LD, 20>(a, ws, kp);
		case 6: return launch_recheck_points<LD, 24>(a, ws, kp);
		case 7: return launch_recheck_points<LD, 28>(a, ws, kp);
		default: return launch_recheck_points<LD, 32>(a, ws, kp);
		}
	}
	if (a.k >= 128 && a.dim > 64) return launch_recheck_sliced<LD>(a, ws, kp);
	if (a.k >= 128 && a.dim <= 64) {
		switch ((a.dim + 7) / 8) {
		case 5: return launch_recheck_points<LD, 40>(a, ws, kp);
		case 6: return launch_recheck_points<LD, 48>(a, ws, kp);
		case 7: return launch_recheck_points<LD, 56>(a, ws, kp);
		default: return launch_recheck_points<LD, 64>(a, ws, kp);
		}
	}
	if (a.dim <= 64) {
		if (a.k >= 48) return launch_recheck_dpad<LD, 64>(a, ws, kp);
		if (a.k >= 24) return launch_recheck_dpad<LD, 32>(a, ws, kp);
		return launch_recheck_dpad<LD, 16>(a, ws, kp);
	}
	if ((size_t)a.dim * 8 * sizeof(float) <= 64 * 1024) return launch_recheck_t<LD, 8>(a, ws, kp);
	return launch_recheck_t<LD, 1>(a, ws, kp);
}

/*
 * SoA points and the lane-per-centroid kernels: a point's coordinates are `stride` apart, so every coordinate would be a
 * scalar load of its own from a cache line of its own, repeated by every wavefront of the work-group (measured: 97 ms
 * for 370 k points of 256 dimensions against 4.6 ms for AoS rows). The rows of the queued points are therefore copied
 * once, with vector loads, into a compact AoS block that has a queue of its own (entry e: row e, the threshold of the
 * original entry e); the kernels run on that block and a last kernel copies their results to the points' places.
 * The block holds up to `cap` rows; entries beyond that are left to the kernels reading the SoA points directly.
 */
static size_t g_queued_rows_bytes = (size_t)1 << 30; /* upper bound of the block of copied rows */

void set_queued_rows_limit(size_t bytes) { g_queued_rows_bytes = bytes; }

/* a group of `1 << group_shift` lanes (the smallest power of two that covers the row, at most a wavefront) copies one row */
template <int LD>
__global__ void __launch_bounds__(256)
gather_queued_rows_kernel(const float* __restrict__ data, size_t stride, uint32_t dim, const uint32_t* __restrict__ queue,
                          uint32_t* __restrict__ counters, float* __restrict__ rows, uint32_t* __restrict__ row_queue,
                          unsigned long long* __restrict__ keys, uint32_t cap, uint32_t group_shift)
{
	const uint32_t count = counters[0];
	const uint32_t taken = min(count, cap);
	if (blockIdx.x == 0 && threadIdx.x == 0) { counters[1] = taken; counters[2] = count - taken; }
	const uint32_t group = 1u << group_shift;
	const uint32_t q0 = threadIdx.x & (group - 1);
	const uint32_t groups = (gridDim.x * blockDim.x) >> group_shift;
	for (uint32_t e = (blockIdx.x * blockDim.x + threadIdx.x) >> group_shift; e < taken; e += groups) {
		const uint32_t pt = queue[2 * (size_t)e];
		for (uint32_t q = q0; q < dim; q += group) rows[(size_t)e * dim + q] = data[elem<LD>(stride, pt, q)];
		if (q0 == 0) {
			row_queue[2 * (size_t)e] = e;
			row_queue[2 * (size_t)e + 1] = queue[2 * (size_t)e + 1];
			if (keys) keys[e] = ~0ull; /* no centroid evaluated yet */
		}
	}
}

__global__ void __launch_bounds__(256)
scatter_row_results_kernel(const uint32_t* __restrict__ queue, const uint32_t* __restrict__ counters,
                           const uint32_t* __restrict__ row_assignment, uint32_t* __restrict__ assignment)
{
	const uint32_t taken = counters[1];
	for (uint32_t e = blockIdx.x * blockDim.x + threadIdx.x; e < taken; e += gridDim.x * blockDim.x)
		assignment[queue[2 * (size_t)e]] = row_assignment[e];
}

/* the pairs the screen noted: a wavefront per work item of the screen (same partition), a lane per pair */
__global__ void __launch_bounds__(256)
evaluate_pairs_kernel(const float* __restrict__ rows, uint32_t dim, const float* __restrict__ means_t, uint32_t kp,
                      const uint32_t* __restrict__ pairs, const uint32_t* __restrict__ item_pairs, const uint32_t* __restrict__ row_count,
                      uint32_t unit_rows, uint32_t screen_waves, unsigned long long* __restrict__ keys)
{
	const ScreenItems work = screen_items(row_count[0], unit_rows, kp / TILE, screen_waves);
	const uint32_t slice = SCREEN_SLICE_PER_ROW * unit_rows;
	const uint32_t lane = threadIdx.x & (WAVE - 1);
	const uint32_t waves = gridDim.x * (blockDim.x / WAVE);
	for (uint32_t item = (blockIdx.x * blockDim.x + threadIdx.x) / WAVE; item < work.items; item += waves) {
		const uint32_t noted = item_pairs[item];
		const uint32_t* mine = pairs + 2 * (size_t)item * slice;
		for (uint32_t t = lane; t < noted; t += WAVE) {
			const uint32_t row = mine[2 * t];
			evaluate_pair<KMX_AOS>(rows, dim, means_t, dim, kp, row, mine[2 * t + 1], &keys[row]);
		}
	}
}

/* a row no centroid was evaluated for (every distance a NaN, or nothing within the threshold, which only values the
 * sweep does not cover produce) stays where the serial scan leaves it: at centroid 0 */
__global__ void __launch_bounds__(256)
scatter_row_keys_kernel(const uint32_t* __restrict__ queue, const uint32_t* __restrict__ counters,
                        const unsigned long long* __restrict__ keys, uint32_t* __restrict__ assignment)
{
	const uint32_t taken = counters[1];
	for (uint32_t e = blockIdx.x * blockDim.x + threadIdx.x; e < taken; e += gridDim.x * blockDim.x) {
		const unsigned long long key = keys[e];
		assignment[queue[2 * (size_t)e]] = key == ~0ull ? 0u : (uint32_t)key;
	}
}

static uint32_t row_group_shift(uint32_t dim)
{
	uint32_t shift = 0;
	while (shift < 6 && (1u << shift) < dim) ++shift;
	return shift;
}

static uint32_t queued_rows_cap(const AssignArgs& a)
{
	return (uint32_t)std::min<size_t>(a.n, std::max<size_t>(1024, g_queued_rows_bytes / ((size_t)a.dim * sizeof(float))));
}

uint32_t screened_rows_cap(const AssignArgs& a)
{
	return std::min<uint32_t>(queued_rows_cap(a), 4u << 20); /* the pair list takes 32 bytes per row */
}

int launch_recheck_screened(const AssignArgs& a, Workspace* ws, uint32_t kp, const DeviceInfo& dev)
{
	const uint32_t cap = screened_rows_cap(a);
	const uint32_t unit_rows = screen_unit_rows(a.dim);
	const uint32_t items_max = screen_items_max(cap, unit_rows);
	const size_t slice_words = 2 * (size_t)SCREEN_SLICE_PER_ROW * unit_rows;
	int rc = reserve_queued_rows(ws, cap, a.dim, items_max + items_max * slice_words);
	if (rc) return rc;
	const uint32_t group_shift = row_group_shift(a.dim);
	uint32_t* row_queue = ws->queued_index;
	unsigned long long* keys = (unsigned long long*)(ws->queued_index + 2 * (size_t)cap);
	uint32_t* item_pairs = ws->queued_index + 4 * (size_t)cap;
	uint32_t* pairs = item_pairs + items_max;
	if (a.layout == KMX_AOS)
		KMX_LAUNCH_KERNEL((gather_queued_rows_kernel<KMX_AOS>), dim3(1024), dim3(256), 0, stream(),
		                   a.data, a.stride, a.dim, ws->queue, ws->counters, ws->queued_rows, row_queue, keys, cap, group_shift);
	else
		KMX_LAUNCH_KERNEL((gather_queued_rows_kernel<KMX_SOA>), dim3(1024), dim3(256), 0, stream(),
		                   a.data, a.stride, a.dim, ws->queue, ws->counters, ws->queued_rows, row_queue, keys, cap, group_shift);
	KMX_LAUNCH_CHECK("gather_queued_rows_kernel");
	uint32_t screen_waves = 0;
	rc = launch_screen_bf16(ws->queued_rows, ws, row_queue, ws->counters + 1, pairs, item_pairs, keys, a.dim, a.k, kp, dev, &screen_waves);
	if (rc) return rc;
	KMX_LAUNCH_KERNEL(evaluate_pairs_kernel, dim3(1024), dim3(256), 0, stream(),
	                   ws->queued_rows, a.dim, ws->means_t, kp, pairs, item_pairs, ws->counters + 1, unit_rows, screen_waves, keys);
	KMX_LAUNCH_CHECK("evaluate_pairs_kernel");
	KMX_LAUNCH_KERNEL(scatter_row_keys_kernel, dim3(512), dim3(256), 0, stream(), ws->queue, ws->counters, keys, a.assignment);
	KMX_LAUNCH_CHECK("scatter_row_keys_kernel");
	if (cap == a.n) return KMX_OK; /* every point has a row: nothing can be left over */
	Workspace rest = *ws; /* the launchers only read the pointers */
	rest.queue = ws->queue + 2 * (size_t)cap; rest.counters = ws->counters + 2;
	return a.layout == KMX_AOS ? launch_recheck_l<KMX_AOS>(a, &rest, kp) : launch_recheck_l<KMX_SOA>(a, &rest, kp);
}

int launch_recheck(const AssignArgs& a, Workspace* ws, uint32_t kp)
{
	if ((size_t)a.dim * sizeof(float) * 16 > 160 * 1024)
		return fail(KMX_ERR_UNSUPPORTED, "assign: dim %u is too large for the exact pass", a.dim);
	if (a.layout == KMX_AOS) return launch_recheck_l<KMX_AOS>(a, ws, kp);
	if (a.k < 128) return launch_recheck_l<KMX_SOA>(a, ws, kp); /* these kernels stage the points in LDS with vector loads */

	const uint32_t cap = queued_rows_cap(a);
	int rc = reserve_queued_rows(ws, cap, a.dim, 0);
	if (rc) return rc;
	const uint32_t group_shift = row_group_shift(a.dim);
	uint32_t* row_queue = ws->queued_index;
	uint32_t* row_assignment = ws->queued_index + 2 * (size_t)cap;
	KMX_LAUNCH_KERNEL((gather_queued_rows_kernel<KMX_SOA>), dim3(2048), dim3(256), 0, stream(),
	                   a.data, a.stride, a.dim, ws->queue, ws->counters, ws->queued_rows, row_queue, (unsigned long long*)nullptr, cap, group_shift);
	KMX_LAUNCH_CHECK("gather_queued_rows_kernel");
	AssignArgs rows = a;
	rows.data = ws->queued_rows; rows.layout = KMX_AOS; rows.stride = a.dim; rows.assignment = row_assignment; rows.n = cap;
	Workspace view = *ws; /* the launchers only read the pointers */
	view.queue = row_queue; view.counters = ws->counters + 1;
	rc = launch_recheck_l<KMX_AOS>(rows, &view, kp);
	if (rc) return rc;
	KMX_LAUNCH_KERNEL(scatter_row_results_kernel, dim3(512), dim3(256), 0, stream(), ws->queue, ws->counters, row_assignment, a.assignment);
	KMX_LAUNCH_CHECK("scatter_row_results_kernel");
	if (cap == a.n) return KMX_OK; /* every point has a row: nothing can be left over */
	view.queue = ws->queue + 2 * (size_t)cap; view.counters = ws->counters + 2;
	return launch_recheck_l<KMX_SOA>(a, &view, kp);
}

} // namespace kmx
