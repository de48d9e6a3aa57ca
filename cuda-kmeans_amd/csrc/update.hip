/*
 * Update step: per-cluster sums and counts of the assigned points, then the divide.
 *
 *   update_point_kernel - one lane per point, global atomics
 *                         (counterpart of updateAtomicPointKernel, reference kernels.cu:726-743)
 *   update_fine_kernel  - one lane per (point, dim) element, global atomics
 *                         (counterpart of updateAtomicFineKernel, reference kernels.cu:770-791)
 *   update_lds_kernel   - the tuned variant (counterpart of updateAtomicShmKernel, reference
 *                         kernels.cu:817-858): every work-group owns a contiguous chunk of points and
 *                         a slice of the dimensions, accumulates the WHOLE k x slice block (and the
 *                         counts) in LDS with ds_add, and flushes one aggregated atomic per non-zero
 *                         element to HBM. Points are read exactly once, fully coalesced.
 *   reduce_copies_kernel / divide_means_kernel
 *                       - counterparts of reducePrivCopiesKernel / divideMeansKernel
 *                         (reference kernels.cu:115-135,149-163); empty clusters keep their zero.
 *
 * Sums are fp32 and their order differs from the serial order (atomics), exactly as in the
 * reference's GPU path; counts are integers and exact.
 */
#include "kmx_internal.h"

#include <algorithm>

namespace kmx {

/* hardware fp32 atomic add without return value (global_atomic_add_f32 / ds_add_f32) */
__device__ __forceinline__ void atomic_add_f32(float* addr, float v) { unsafeAtomicAdd(addr, v); }

template <int LM>
__device__ __forceinline__ float* privatized(float* means, size_t copy_floats, uint32_t copies)
{
	/* replica = (global lane id / wavefront size) % copies, as privatizeResultPointer (reference kernels.cu:104-111) */
	if (copies > 1) means += copy_floats * (((blockDim.x * blockIdx.x + threadIdx.x) / WAVE) % copies);
	return means;
}

template <int LD, int LM>
__global__ void __launch_bounds__(1024)
update_point_kernel(const float* __restrict__ data, size_t stride, const uint32_t* __restrict__ assignment,
                    float* __restrict__ means, size_t stride_means, uint32_t* __restrict__ sizes,
                    uint32_t dim, uint32_t k, uint32_t n, size_t copy_floats, uint32_t copies)
{
	(void)k;
	means = privatized<LM>(means, copy_floats, copies);
	const uint32_t threads = blockDim.x * gridDim.x;
	for (uint32_t idx = threadIdx.x + blockIdx.x * blockDim.x; idx < n; idx += threads) {
		uint32_t target = assignment[idx];
		for (uint32_t d = 0; d < dim; ++d)
			atomic_add_f32(&means[elem<LM>(stride_means, target, d)], data[elem<LD>(stride, idx, d)]);
		atomicAdd(&sizes[target], 1u);
	}
}

template <int LD, int LM>
__global__ void __launch_bounds__(1024)
update_fine_kernel(const float* __restrict__ data, size_t stride, const uint32_t* __restrict__ assignment,
                   float* __restrict__ means, size_t stride_means, uint32_t* __restrict__ sizes,
                   uint32_t dim, uint32_t k, uint32_t n, size_t copy_floats, uint32_t copies)
{
	(void)k;
	means = privatized<LM>(means, copy_floats, copies);
	const size_t threads = (size_t)blockDim.x * gridDim.x;
	const size_t size = (size_t)n * dim;
	for (size_t i = threadIdx.x + (size_t)blockIdx.x * blockDim.x; i < size; i += threads) {
		uint32_t d = (uint32_t)(i % dim);
		uint32_t idx = (uint32_t)(i / dim);
		uint32_t target = assignment[idx];
		atomic_add_f32(&means[elem<LM>(stride_means, target, d)], data[elem<LD>(stride, idx, d)]);
		if (d == 0) atomicAdd(&sizes[target], 1u);
	}
}

/*
 * LDS-privatised update. Grid = (point chunks, dimension slices).
 * LDS: replicas x k x row floats of partial sums (row = slice width, +1 padding for SoA input so that
 * lanes holding different points of one dimension spread over the banks), then replicas x k counts.
 *
 * AoS input: thread t owns dimension (t % slice) of point slot (t / slice); the work-group walks its
 * chunk `slots` points at a time, so consecutive lanes read consecutive floats of consecutive rows.
 * SoA input: thread t owns a point and walks the slice's dimensions; consecutive lanes read
 * consecutive points of one dimension.
 * Replica = point slot % replicas: for small k the slots of one wavefront then add to different
 * copies, which removes the same-address serialisation of hot clusters.
 */
constexpr int UPDATE_UNROLL = 8;

template <int LD, int LM>
__global__ void __launch_bounds__(1024)
update_lds_kernel(const float* __restrict__ data, size_t stride, const uint32_t* __restrict__ assignment,
                  float* __restrict__ means, size_t stride_means, uint32_t* __restrict__ sizes,
                  uint32_t dim, uint32_t k, uint32_t n, uint32_t slice, uint32_t chunk_points, uint32_t replicas)
{
	extern __shared__ float lds[];
	const uint32_t row = LD == KMX_AOS ? slice : slice + 1;
	const uint32_t d0 = blockIdx.y * slice;
	const uint32_t width = min(slice, dim - d0);
	const uint32_t sum_floats = replicas * k * row;
	uint32_t* counts = (uint32_t*)(lds + sum_floats);
	const bool count_here = blockIdx.y == 0;

	for (uint32_t i = threadIdx.x; i < sum_floats + replicas * k; i += blockDim.x) lds[i] = 0.0f;
	__syncthreads();

	const uint32_t p_begin = min((uint64_t)blockIdx.x * chunk_points, (uint64_t)n);
	const uint32_t p_end = min((uint64_t)p_begin + chunk_points, (uint64_t)n);

	if (LD == KMX_AOS) {
		const uint32_t slots = blockDim.x / slice;
		const uint32_t slot = threadIdx.x / slice;
		const uint32_t dd = threadIdx.x - slot * slice;
		if (slot < slots && dd < width) {
			float* acc = lds + (size_t)(slot % replicas) * k * row + dd;
			uint32_t* cnt = counts + (size_t)(slot % replicas) * k;
			const float* src = data + (size_t)d0 + dd;
			uint32_t p = p_begin + slot;
			for (; p + (UPDATE_UNROLL - 1) * slots < p_end; p += UPDATE_UNROLL * slots) {
				float v[UPDATE_UNROLL];
				uint32_t t[UPDATE_UNROLL];
#pragma unroll
				for (int u = 0; u < UPDATE_UNROLL; ++u) {
					v[u] = src[(size_t)(p + u * slots) * stride];
					t[u] = assignment[p + u * slots];
				}
#pragma unroll
				for (int u = 0; u < UPDATE_UNROLL; ++u) {
					atomic_add_f32(acc + (size_t)t[u] * row, v[u]);
					if (count_here && dd == 0) atomicAdd(cnt + t[u], 1u);
				}
			}
			for (; p < p_end; p += slots) {
				float v = src[(size_t)p * stride];
				uint32_t t = assignment[p];
				atomic_add_f32(acc + (size_t)t * row, v);
				if (count_here && dd == 0) atomicAdd(cnt + t, 1u);
			}
		}
	}
	else {
		const uint32_t rep = (threadIdx.x / 4) % replicas;
		float* acc = lds + (size_t)rep * k * row;
		uint32_t* cnt = counts + (size_t)rep * k;
		for (uint32_t p = p_begin + threadIdx.x; p < p_end; p += blockDim.x) {
			uint32_t t = assignment[p];
			if (count_here) atomicAdd(cnt + t, 1u);
			float* dst = acc + (size_t)t * row;
			uint32_t dd = 0;
			for (; dd + UPDATE_UNROLL <= width; dd += UPDATE_UNROLL) {
				float v[UPDATE_UNROLL];
#pragma unroll
				for (int u = 0; u < UPDATE_UNROLL; ++u) v[u] = data[(size_t)(d0 + dd + u) * stride + p];
#pragma unroll
				for (int u = 0; u < UPDATE_UNROLL; ++u) atomic_add_f32(dst + dd + u, v[u]);
			}
			for (; dd < width; ++dd) atomic_add_f32(dst + dd, data[(size_t)(d0 + dd) * stride + p]);
		}
	}
	__syncthreads();

	/* flush: merge the replicas, one atomic per non-zero element */
	for (uint32_t e = threadIdx.x; e < k * width; e += blockDim.x) {
		uint32_t c = e / width, dd = e - c * width;
		float s = 0.0f;
		for (uint32_t r = 0; r < replicas; ++r) s += lds[(size_t)r * k * row + (size_t)c * row + dd];
		if (s != 0.0f) atomic_add_f32(&means[elem<LM>(stride_means, c, d0 + dd)], s);
	}
	if (count_here) {
		for (uint32_t c = threadIdx.x; c < k; c += blockDim.x) {
			uint32_t s = 0;
			for (uint32_t r = 0; r < replicas; ++r) s += counts[(size_t)r * k + c];
			if (s) atomicAdd(&sizes[c], s);
		}
	}
}

template <int LM>
__global__ void __launch_bounds__(256)
reduce_copies_kernel(float* __restrict__ means, size_t stride_means, size_t copy_floats, uint32_t dim, uint32_t k, uint32_t copies)
{
	const uint32_t total = k * dim;
	for (uint32_t i = threadIdx.x + blockIdx.x * blockDim.x; i < total; i += blockDim.x * gridDim.x) {
		uint32_t c = i / dim, d = i - c * dim;
		size_t e = elem<LM>(stride_means, c, d);
		float acc = means[e];
		for (uint32_t r = 1; r < copies; ++r) acc += means[e + r * copy_floats];
		means[e] = acc;
	}
}

template <int LM>
__global__ void __launch_bounds__(256)
divide_means_kernel(float* __restrict__ means, size_t stride_means, const uint32_t* __restrict__ sizes, uint32_t dim, uint32_t k)
{
	const uint32_t total = k * dim;
	for (uint32_t i = threadIdx.x + blockIdx.x * blockDim.x; i < total; i += blockDim.x * gridDim.x) {
		uint32_t c = i / dim, d = i - c * dim;
		uint32_t divisor = sizes[c];
		if (divisor > 0) {
			size_t e = elem<LM>(stride_means, c, d);
			means[e] = means[e] / (float)divisor;
		}
	}
}

static size_t copy_floats_of(const UpdateArgs& u)
{
	/* LAYOUT_MEANS::size(k, dim) with the caller's stride */
	return u.layout_means == KMX_AOS ? (size_t)u.k * u.stride_means : (size_t)u.dim * u.stride_means;
}

template <int LD, int LM>
static int launch_update_t(int variant, const UpdateArgs& u, kmx_exec_params* exec, const DeviceInfo& dev)
{
	uint32_t block = exec->block_size ? exec->block_size : 256;
	block = std::min<uint32_t>((block + WAVE - 1) / WAVE * WAVE, 1024);
	const uint32_t ipt = exec->items_per_thread ? exec->items_per_thread : 1;
	const size_t copy_floats = copy_floats_of(u);
	uint32_t copies = exec->privatized_copies;

	int rc = KMX_OK;
	if (u.n > 0) {
		if ((rc = profile_begin(1))) return rc;
		if (variant == KMX_UPDATE_ATOMIC_SHM) {
			/* LDS budget: exec->shared_mem_bytes if given, else what the device offers a work-group */
			uint32_t budget = exec->shared_mem_bytes ? std::min(exec->shared_mem_bytes, dev.lds_bytes) : dev.lds_bytes;
			const uint32_t pad = LD == KMX_AOS ? 0 : 1;
			const uint32_t words = budget / 4;
			uint32_t slice = 0;
			if (words > u.k) slice = std::min<uint32_t>(u.dim, (words - u.k) / u.k > pad ? (words - u.k) / u.k - pad : 0);
			if (slice >= 32 && slice < u.dim) slice = slice / 32 * 32; /* whole 128-byte lines per point and slice */
			if (slice == 0 || (LD == KMX_AOS && slice > 1024)) {
				variant = KMX_UPDATE_ATOMIC_FINE; /* k too large for LDS privatisation */
				copies = 1;
			}
			else {
				const uint32_t slices = (u.dim + slice - 1) / slice;
				const uint32_t row = slice + pad;
				const uint32_t wg = 1024;
				const uint32_t slots = LD == KMX_AOS ? wg / slice : wg;
				/* replicas only pay for small k: keep them within 16 KB and one per point slot */
				uint32_t replicas = std::max<uint32_t>(1, std::min<uint32_t>({ 16384u / ((row + 1) * u.k * 4), LD == KMX_AOS ? slots : 16u, 16u }));
				const uint32_t lds_bytes = replicas * u.k * (row + 1) * 4;
				const uint32_t wg_per_cu = std::max<uint32_t>(1, std::min<uint32_t>(2, dev.lds_bytes / std::max(lds_bytes, 1u)));
				uint32_t chunks = std::max<uint32_t>(1, dev.compute_units * wg_per_cu / slices);
				uint32_t chunk_points = (u.n + chunks - 1) / chunks;
				const uint32_t quantum = slots * UPDATE_UNROLL;
				chunk_points = (chunk_points + quantum - 1) / quantum * quantum;
				chunks = (u.n + chunk_points - 1) / chunk_points;
				auto kernel = update_lds_kernel<LD, LM>;
				KMX_HIP(hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
				exec->block_count = chunks * slices;
				hipLaunchKernelGGL(kernel, dim3(chunks, slices), dim3(wg), lds_bytes, stream(),
				                   u.data, u.stride, u.assignment, u.means, u.stride_means, u.cluster_sizes,
				                   u.dim, u.k, u.n, slice, chunk_points, replicas);
				KMX_LAUNCH_CHECK("update_lds_kernel");
				copies = 1; /* this variant writes replica 0 only */
			}
		}
		if (variant == KMX_UPDATE_ATOMIC_POINT) {
			uint32_t threads = (u.n + ipt - 1) / ipt;
			exec->block_count = (threads + block - 1) / block;
			hipLaunchKernelGGL((update_point_kernel<LD, LM>), dim3(exec->block_count), dim3(block), 0, stream(),
			                   u.data, u.stride, u.assignment, u.means, u.stride_means, u.cluster_sizes, u.dim, u.k, u.n, copy_floats, copies);
			KMX_LAUNCH_CHECK("update_point_kernel");
		}
		else if (variant == KMX_UPDATE_ATOMIC_FINE) {
			size_t threads = ((size_t)u.n * u.dim + ipt - 1) / ipt;
			size_t blocks = (threads + block - 1) / block;
			exec->block_count = (uint32_t)std::min<size_t>(blocks, 1u << 20);
			hipLaunchKernelGGL((update_fine_kernel<LD, LM>), dim3(exec->block_count), dim3(block), 0, stream(),
			                   u.data, u.stride, u.assignment, u.means, u.stride_means, u.cluster_sizes, u.dim, u.k, u.n, copy_floats, copies);
			KMX_LAUNCH_CHECK("update_fine_kernel");
		}
		if ((rc = profile_end(1))) return rc;
	}

	const uint32_t total = u.k * u.dim;
	const uint32_t blocks = std::min<uint32_t>((total + 255) / 256, 1024);
	if (copies > 1) {
		hipLaunchKernelGGL((reduce_copies_kernel<LM>), dim3(blocks), dim3(256), 0, stream(), u.means, u.stride_means, copy_floats, u.dim, u.k, copies);
		KMX_LAUNCH_CHECK("reduce_copies_kernel");
	}
	hipLaunchKernelGGL((divide_means_kernel<LM>), dim3(blocks), dim3(256), 0, stream(), u.means, u.stride_means, u.cluster_sizes, u.dim, u.k);
	KMX_LAUNCH_CHECK("divide_means_kernel");
	return KMX_OK;
}

int launch_update(int variant, const UpdateArgs& u, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev)
{
	(void)ws;
	if (u.layout == KMX_AOS && u.layout_means == KMX_AOS) return launch_update_t<KMX_AOS, KMX_AOS>(variant, u, exec, dev);
	if (u.layout == KMX_AOS && u.layout_means == KMX_SOA) return launch_update_t<KMX_AOS, KMX_SOA>(variant, u, exec, dev);
	if (u.layout == KMX_SOA && u.layout_means == KMX_AOS) return launch_update_t<KMX_SOA, KMX_AOS>(variant, u, exec, dev);
	return launch_update_t<KMX_SOA, KMX_SOA>(variant, u, exec, dev);
}

} // namespace kmx
