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
#include "kmx_internal.h"

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
                   const uint32_t* __restrict__ queue, const uint32_t* __restrict__ counters)
{
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
#pragma unroll
			for (int d = 0; d < DPAD; ++d) x[p][d] = (uint32_t)d < dim ? data[elem<LD>(stride, idx[p], d)] : 0.0f;
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

template <int LD, int LM>
static int launch_base_t(const AssignArgs& a, kmx_exec_params* exec, uint32_t* counters)
{
	uint32_t block = exec->block_size ? exec->block_size : 256;
	if (block > 256) block = 256;
	block = (block + WAVE - 1) / WAVE * WAVE;
	exec->block_count = (a.n + block - 1) / block;
	int rc = profile_begin(0);
	if (rc) return rc;
	hipLaunchKernelGGL((assign_base_kernel<LD, LM>), dim3(exec->block_count), dim3(block), 0, stream(),
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
	hipLaunchKernelGGL(kernel, dim3(blocks), dim3(block), lds, stream(),
	                   a.data, a.stride, ws->means_t, kp, a.assignment, a.dim, a.k, ws->queue, ws->counters);
	KMX_LAUNCH_CHECK("recheck_kernel");
	return KMX_OK;
}

template <int LD, int L, int PB, int DPAD>
static int launch_recheck_reg(const AssignArgs& a, Workspace* ws, uint32_t kp)
{
	hipLaunchKernelGGL((recheck_reg_kernel<LD, L, PB, DPAD>), dim3(2048), dim3(256), 0, stream(),
	                   a.data, a.stride, ws->means_t, kp, a.assignment, a.dim, a.k, ws->queue, ws->counters);
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

template <int LD>
static int launch_recheck_l(const AssignArgs& a, Workspace* ws, uint32_t kp)
{
	if (a.dim <= 64) {
		if (a.k >= 48) return launch_recheck_dpad<LD, 64>(a, ws, kp);
		if (a.k >= 24) return launch_recheck_dpad<LD, 32>(a, ws, kp);
		return launch_recheck_dpad<LD, 16>(a, ws, kp);
	}
	if ((size_t)a.dim * 8 * sizeof(float) <= 64 * 1024) return launch_recheck_t<LD, 8>(a, ws, kp);
	return launch_recheck_t<LD, 1>(a, ws, kp);
}

int launch_recheck(const AssignArgs& a, Workspace* ws, uint32_t kp)
{
	if ((size_t)a.dim * sizeof(float) * 16 > 160 * 1024)
		return fail(KMX_ERR_UNSUPPORTED, "assign: dim %u is too large for the exact pass", a.dim);
	if (a.layout == KMX_AOS) return launch_recheck_l<KMX_AOS>(a, ws, kp);
	return launch_recheck_l<KMX_SOA>(a, ws, kp);
}

} // namespace kmx
