/*
 * Assignment with the serial arithmetic, operation for operation:
 *   dist(x, c) = sqrt( (((x0-c0)^2 + (x1-c1)^2) + ...) ), every subtract / multiply / add
 *   rounded separately in fp32, d ascending (reference metric_policies.hpp:23-28,40-44);
 *   argmin with strict comparison from centroid 0, so the lowest index wins equal distances
 *   and NaN distances never win (reference serial.hpp:21-35).
 *
 *   assign_base_kernel  - one lane per point; counterpart of baseAssignmentKernel
 *                         (reference kernels.cu:180-199) and the `hip_base` algorithm.
 *   recheck_kernel      - one wavefront per queued point; the exact pass behind the fast
 *                         variants (they queue the points whose ranking by |c|^2 - 2x.c is
 *                         not decided beyond rounding error).
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
 * One wavefront per queued point. Lane l evaluates centroids l, l+64, ... in ascending order and
 * keeps its own (distance, index) minimum; the 64 candidates are merged by (smaller distance, then
 * smaller index), which is the serial scan's result: the first centroid attaining the minimum.
 * A NaN distance to centroid 0 pins the point to centroid 0, as `minDist > dist` is then never true.
 */
template <int LD, int LM>
__global__ void __launch_bounds__(256)
recheck_kernel(const float* __restrict__ data, size_t stride, const float* __restrict__ means, size_t stride_means,
               uint32_t* __restrict__ assignment, uint32_t dim, uint32_t k,
               const uint32_t* __restrict__ queue, const uint32_t* __restrict__ counters)
{
	const uint32_t lane = threadIdx.x & (WAVE - 1);
	const uint32_t wave = (blockIdx.x * blockDim.x + threadIdx.x) / WAVE;
	const uint32_t waves = gridDim.x * blockDim.x / WAVE;
	const uint32_t count = counters[0];

	for (uint32_t q = wave; q < count; q += waves) {
		const uint32_t idx = queue[q];
		float best = __builtin_inff();
		uint32_t bestIdx = 0xFFFFFFFFu;
		for (uint32_t m = lane; m < k; m += WAVE) {
			float dist = exact_distance<LD, LM>(data, stride, idx, means, stride_means, m, dim);
			if (dist < best || (dist == best && m < bestIdx)) {
				best = dist;
				bestIdx = m;
			}
		}
		/* is the distance to centroid 0 NaN? (every lane repeats that one sum; the point index is wave-uniform) */
		float d0 = exact_distance<LD, LM>(data, stride, idx, means, stride_means, 0, dim);
		bool pinned = d0 != d0;
		for (int off = WAVE / 2; off > 0; off >>= 1) {
			float ob = __shfl_xor(best, off);
			uint32_t oi = __shfl_xor(bestIdx, off);
			if (ob < best || (ob == best && oi < bestIdx)) {
				best = ob;
				bestIdx = oi;
			}
		}
		if (lane == 0) assignment[idx] = pinned ? 0u : (bestIdx == 0xFFFFFFFFu ? 0u : bestIdx);
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

template <int LD, int LM>
static int launch_recheck_t(const AssignArgs& a, Workspace* ws)
{
	const unsigned block = 256, blocks = 1024;
	hipLaunchKernelGGL((recheck_kernel<LD, LM>), dim3(blocks), dim3(block), 0, stream(),
	                   a.data, a.stride, a.means, a.stride_means, a.assignment, a.dim, a.k, ws->queue, ws->counters);
	KMX_LAUNCH_CHECK("recheck_kernel");
	return KMX_OK;
}

int launch_recheck(const AssignArgs& a, Workspace* ws)
{
	if (a.layout == KMX_AOS && a.layout_means == KMX_AOS) return launch_recheck_t<KMX_AOS, KMX_AOS>(a, ws);
	if (a.layout == KMX_AOS && a.layout_means == KMX_SOA) return launch_recheck_t<KMX_AOS, KMX_SOA>(a, ws);
	if (a.layout == KMX_SOA && a.layout_means == KMX_AOS) return launch_recheck_t<KMX_SOA, KMX_AOS>(a, ws);
	return launch_recheck_t<KMX_SOA, KMX_SOA>(a, ws);
}

} // namespace kmx
