/*
 * Update step: per-cluster sums and counts of the assigned points, then the divide.
 *
 *   update_point_kernel   - one lane per point, global atomics
 *                           (counterpart of updateAtomicPointKernel, reference kernels.cu:726-743)
 *   update_fine_kernel    - one lane per (point, dim) element, global atomics
 *                           (counterpart of updateAtomicFineKernel, reference kernels.cu:770-791)
 *   KMX_UPDATE_ATOMIC_SHM - the tuned variant (counterpart of updateAtomicShmKernel, reference
 *                           kernels.cu:817-858), three kernels chosen by shape. Measured on gfx950: an LDS
 *                           ds_add_f32 costs ~194 cycles per wavefront instruction whatever the address
 *                           pattern (lanes are serialised), ds_add_u32 4.4 cycles, a plain LDS
 *                           read-add-write 8.2 cycles. Floating-point LDS atomics are therefore avoided:
 *       update_private_kernel  small k*dim: every lane group (one lane per dimension) owns a PRIVATE copy
 *                              of the k x dim block in LDS and accumulates with plain read-add-write; the
 *                              copies are merged at the end, one global atomic per element and work-group.
 *                              (update_private_vec_kernel: the same with 16-byte row pieces per lane, for
 *                              a million points or more: N = 16.7M, d = 16, k = 16 in 0.205 instead of 0.250 ms.)
 *       update_sorted_kernel   larger k: the work-group counting-sorts its chunk of points by cluster
 *                              with integer LDS atomics, then lane groups walk the sorted list and sum each
 *                              cluster's rows in registers (no atomics at all); per-chunk sums go to a partial
 *                              buffer with plain coalesced stores and reduce_partials_kernel folds them.
 *       update_lds_kernel      fallback for the shapes/layouts the two above do not take (SoA points):
 *                              LDS-privatised ds_add_f32.
 *     Points are read exactly once in all three.
 *   reduce_copies_kernel / divide_means_kernel
 *                         - counterparts of reducePrivCopiesKernel / divideMeansKernel
 *                           (reference kernels.cu:115-135,149-163); empty clusters keep their zero.
 *
 * Sums are fp32 and their order differs from the serial order, exactly as in the reference's GPU path
 * (atomics); counts are integers and exact.
 */
#include "kmx_internal.h"

#include <algorithm>


namespace kmx {

/* hardware fp32 atomic add without return value (global_atomic_add_f32 / ds_add_f32) */
__device__ __forceinline__ void atomic_add_f32(float* addr, float v) { unsafeAtomicAdd(addr, v); }

/* EMUL: the addition as a compare-and-swap loop (atomicAddEmul of the update micro-benchmark, reference
 * bucketing-cuda/kernels/kernels.cu:46-57), for measuring what the hardware atomic is worth */
template <bool EMUL>
__device__ __forceinline__ void atomic_add_global(float* addr, float v)
{
	if (!EMUL) { unsafeAtomicAdd(addr, v); return; }
	unsigned int* word = (unsigned int*)addr;
	unsigned int old = *word, assumed;
	do {
		assumed = old;
		old = atomicCAS(word, assumed, __float_as_uint(v + __uint_as_float(assumed)));
	} while (assumed != old);
}

template <int LM>
__device__ __forceinline__ float* privatized(float* means, size_t copy_floats, uint32_t copies)
{
	/* replica = (global lane id / wavefront size) % copies, as privatizeResultPointer (reference kernels.cu:104-111) */
	if (copies > 1) means += copy_floats * (((blockDim.x * blockIdx.x + threadIdx.x) / WAVE) % copies);
	return means;
}

template <int LD, int LM, bool EMUL>
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
			atomic_add_global<EMUL>(&means[elem<LM>(stride_means, target, d)], data[elem<LD>(stride, idx, d)]);
		atomicAdd(&sizes[target], 1u);
	}
}

/* one wavefront per point, the lanes stride over its dimensions (atomicWarpKernel of the update micro-benchmark,
 * reference bucketing-cuda/kernels/kernels.cu:234-251, with 64 lanes instead of 32) */
template <int LD, int LM, bool EMUL>
__global__ void __launch_bounds__(1024)
update_warp_kernel(const float* __restrict__ data, size_t stride, const uint32_t* __restrict__ assignment,
                   float* __restrict__ means, size_t stride_means, uint32_t* __restrict__ sizes,
                   uint32_t dim, uint32_t k, uint32_t n, size_t copy_floats, uint32_t copies)
{
	(void)k;
	means = privatized<LM>(means, copy_floats, copies);
	const uint32_t waves = blockDim.x * gridDim.x / WAVE;
	const uint32_t lane = threadIdx.x % WAVE;
	for (uint32_t idx = (threadIdx.x + blockIdx.x * blockDim.x) / WAVE; idx < n; idx += waves) {
		const uint32_t target = assignment[idx];
		for (uint32_t d = lane; d < dim; d += WAVE)
			atomic_add_global<EMUL>(&means[elem<LM>(stride_means, target, d)], data[elem<LD>(stride, idx, d)]);
		if (lane == 0) atomicAdd(&sizes[target], 1u);
	}
}

/* no atomics at all: one lane per element of the result walks all points and adds those of its cluster, in point
 * order (baseKernel of the update micro-benchmark, reference bucketing-cuda/kernels/kernels.cu:163-178); the sums
 * therefore have the bits of the serial loop. O(n k dim): a baseline for small inputs. */
template <int LD, int LM>
__global__ void __launch_bounds__(256)
update_base_kernel(const float* __restrict__ data, size_t stride, const uint32_t* __restrict__ assignment,
                   float* __restrict__ means, size_t stride_means, uint32_t* __restrict__ sizes,
                   uint32_t dim, uint32_t k, uint32_t n)
{
	const uint32_t e = threadIdx.x + blockIdx.x * blockDim.x;
	const uint32_t d = e % dim, c = e / dim;
	if (c >= k) return;
	float sum = 0.0f;
	uint32_t members = 0;
	for (uint32_t i = 0; i < n; ++i) {
		if (assignment[i] != c) continue;
		sum += data[elem<LD>(stride, i, d)];
		++members;
	}
	means[elem<LM>(stride_means, c, d)] = sum;
	if (d == 0) sizes[c] = members;
}

template <int LD, int LM, bool EMUL>
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
		atomic_add_global<EMUL>(&means[elem<LM>(stride_means, target, d)], data[elem<LD>(stride, idx, d)]);
		if (d == 0) atomicAdd(&sizes[target], 1u);
	}
}

/*
 * atomicShm2Kernel of the update micro-benchmark (reference bucketing-cuda/kernels/kernels.cu:381-426): one lane per
 * input element, the WHOLE k x dim block cached in LDS in `lds_copies` private copies (lane t adds to copy t % lds_copies),
 * floating-point LDS atomics; at the end the copies of every element are summed and added to the result with one global
 * atomic per element and work-group. (The reference sums resultCache[i + copy * dim] at :423-426, which is not where
 * copy `copy` of element i was accumulated, (target * copies + copy) * dim + d, unless there is a single copy; here the
 * copies of the element itself are summed.)
 */
template <int LD, int LM>
__global__ void __launch_bounds__(1024)
update_shm2_kernel(const float* __restrict__ data, size_t stride, const uint32_t* __restrict__ assignment,
                   float* __restrict__ means, size_t stride_means, uint32_t* __restrict__ sizes,
                   uint32_t dim, uint32_t k, uint32_t n, size_t copy_floats, uint32_t copies, uint32_t lds_copies)
{
	extern __shared__ float cache[];
	const uint32_t cache_floats = k * dim * lds_copies;
	for (uint32_t i = threadIdx.x; i < cache_floats; i += blockDim.x) cache[i] = 0.0f;
	__syncthreads();
	means = privatized<LM>(means, copy_floats, copies);
	const size_t threads = (size_t)blockDim.x * gridDim.x;
	const size_t size = (size_t)n * dim;
	const uint32_t mine = threadIdx.x % lds_copies;
	for (size_t i = threadIdx.x + (size_t)blockIdx.x * blockDim.x; i < size; i += threads) {
		const uint32_t d = (uint32_t)(i % dim);
		const uint32_t idx = (uint32_t)(i / dim);
		const uint32_t target = assignment[idx];
		atomic_add_f32(&cache[((size_t)target * lds_copies + mine) * dim + d], data[elem<LD>(stride, idx, d)]);
		if (d == 0) atomicAdd(&sizes[target], 1u);
	}
	__syncthreads();
	for (uint32_t i = threadIdx.x; i < k * dim; i += blockDim.x) {
		const uint32_t c = i / dim, d = i % dim;
		float sum = 0.0f;
		for (uint32_t copy = 0; copy < lds_copies; ++copy) sum += cache[((size_t)c * lds_copies + copy) * dim + d];
		atomic_add_f32(&means[elem<LM>(stride_means, c, d)], sum);
	}
}

/*
 * atomicFakeKernel / atomicShmFakeKernel of the update micro-benchmark (reference bucketing-cuda/kernels/kernels.cu:452-469,
 * 495-531): probes of the raw cost of the atomic additions. One lane per input element, the inputs are ignored: element i
 * adds the constant 0.1 to dimension i % dim of bucket (i / dim) % k with a real atomic, in global memory or, for the
 * first `cached` buckets, in LDS (flushed with one global atomic per element and work-group). The result has a closed
 * form: 0.1 * #{point numbers congruent to the bucket modulo k}.
 */
template <int LM, bool EMUL>
__global__ void __launch_bounds__(1024)
update_fake_kernel(float* __restrict__ means, size_t stride_means, uint32_t dim, uint32_t k, uint32_t n, size_t copy_floats, uint32_t copies)
{
	means = privatized<LM>(means, copy_floats, copies);
	const size_t threads = (size_t)blockDim.x * gridDim.x;
	const size_t size = (size_t)n * dim;
	for (size_t i = threadIdx.x + (size_t)blockIdx.x * blockDim.x; i < size; i += threads) {
		const uint32_t d = (uint32_t)(i % dim);
		const uint32_t target = (uint32_t)((i / dim) % k);
		atomic_add_global<EMUL>(&means[elem<LM>(stride_means, target, d)], 0.1f);
	}
}

template <int LM>
__global__ void __launch_bounds__(1024)
update_fake_shm_kernel(float* __restrict__ means, size_t stride_means, uint32_t dim, uint32_t k, uint32_t n, size_t copy_floats, uint32_t copies,
                       uint32_t cached)
{
	extern __shared__ float cache[];
	const uint32_t cache_floats = cached * dim;
	for (uint32_t i = threadIdx.x; i < cache_floats; i += blockDim.x) cache[i] = 0.0f;
	__syncthreads();
	means = privatized<LM>(means, copy_floats, copies);
	const size_t threads = (size_t)blockDim.x * gridDim.x;
	const size_t size = (size_t)n * dim;
	for (size_t i = threadIdx.x + (size_t)blockIdx.x * blockDim.x; i < size; i += threads) {
		const uint32_t d = (uint32_t)(i % dim);
		const uint32_t target = (uint32_t)((i / dim) % k);
		if (target < cached) atomic_add_f32(&cache[(size_t)target * dim + d], 0.1f);
		else atomic_add_f32(&means[elem<LM>(stride_means, target, d)], 0.1f);
	}
	__syncthreads();
	for (uint32_t i = threadIdx.x; i < cache_floats; i += blockDim.x)
		atomic_add_f32(&means[elem<LM>(stride_means, i / dim, i % dim)], cache[i]);
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
constexpr int UPDATE_UNROLL = 16;


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

/*
 * Small k*dim. Lane group = GW lanes (GW = power of two >= dim), lane gl < dim owns dimension gl. Every group
 * has a private block [k*dim sums | k counts] in LDS; consecutive groups take consecutive points, so a
 * wavefront reads 64/GW consecutive rows per step. LDS operations of one wavefront execute in order, so a
 * plain read-add-write is correct even when consecutive points fall into the same cluster. copy_stride is
 * chosen so that the groups of one wavefront start GW banks apart: equal targets (the hot-cluster case) are
 * conflict-free.
 */
template <int LM>
__global__ void __launch_bounds__(256)
update_private_kernel(const float* __restrict__ data, size_t stride, const uint32_t* __restrict__ assignment,
                      float* __restrict__ means, size_t stride_means, uint32_t* __restrict__ sizes,
                      uint32_t dim, uint32_t k, uint32_t n, uint32_t gw, uint32_t copy_stride, uint32_t chunk_points)
{
	extern __shared__ float lds[];
	const uint32_t groups = blockDim.x / gw;
	const uint32_t group = threadIdx.x / gw;
	const uint32_t gl = threadIdx.x - group * gw;
	for (uint32_t i = threadIdx.x; i < groups * copy_stride; i += blockDim.x) lds[i] = 0.0f;
	__syncthreads();

	float* acc = lds + (size_t)group * copy_stride;
	uint32_t* cnt = (uint32_t*)(acc + (size_t)k * dim);
	const uint32_t p_begin = (uint32_t)min((uint64_t)blockIdx.x * chunk_points, (uint64_t)n);
	const uint32_t p_end = (uint32_t)min((uint64_t)p_begin + chunk_points, (uint64_t)n);
	const bool lane_on = gl < dim;
	const float* src = data + (lane_on ? gl : 0);
	uint32_t p = p_begin + group;
	for (; p + (UPDATE_UNROLL - 1) * groups < p_end; p += UPDATE_UNROLL * groups) {
		float v[UPDATE_UNROLL];
		uint32_t t[UPDATE_UNROLL];
#pragma unroll
		for (int u = 0; u < UPDATE_UNROLL; ++u) {
			v[u] = src[(size_t)(p + u * groups) * stride];
			t[u] = assignment[p + u * groups];
		}
#pragma unroll
		for (int u = 0; u < UPDATE_UNROLL; ++u) {
			if (lane_on) acc[t[u] * dim + gl] += v[u];
			if (gl == 0) cnt[t[u]] += 1u;
		}
	}
	for (; p < p_end; p += groups) {
		float v = src[(size_t)p * stride];
		uint32_t t = assignment[p];
		if (lane_on) acc[t * dim + gl] += v;
		if (gl == 0) cnt[t] += 1u;
	}
	__syncthreads();

	for (uint32_t e = threadIdx.x; e < k * dim; e += blockDim.x) {
		float s = 0.0f;
		for (uint32_t g = 0; g < groups; ++g) s += lds[(size_t)g * copy_stride + e];
		const uint32_t c = e / dim, d = e - c * dim;
		if (s != 0.0f) atomic_add_f32(&means[elem<LM>(stride_means, c, d)], s);
	}
	for (uint32_t c = threadIdx.x; c < k; c += blockDim.x) {
		uint32_t s = 0;
		for (uint32_t g = 0; g < groups; ++g) s += ((const uint32_t*)lds)[(size_t)g * copy_stride + (size_t)k * dim + c];
		if (s) atomicAdd(&sizes[c], s);
	}
}

/*
 * The same with 16-byte pieces of a row per lane (dim a multiple of 4, aligned rows): a group is GW4 = dim / 4 lanes (rounded
 * up to a power of two), so a wavefront reads 64 / GW4 consecutive rows with one instruction -- a quarter of the load
 * instructions, and of the loads of the assignment, that one lane per dimension issues. Every group still needs a copy of its
 * own (lanes of one instruction that met in one copy would lose updates), so a work-group of 256 lanes holds 256 / GW4 copies:
 * more LDS per work-group, fewer work-groups per compute unit, the same bytes in flight.
 */
constexpr int UPDATE_UNROLL_VEC = 8; /* row pieces in flight per lane (16 measured the same) */

template <int LM>
__global__ void __launch_bounds__(256)
update_private_vec_kernel(const float* __restrict__ data, size_t stride, const uint32_t* __restrict__ assignment,
                          float* __restrict__ means, size_t stride_means, uint32_t* __restrict__ sizes,
                          uint32_t dim, uint32_t k, uint32_t n, uint32_t gw, uint32_t copy_stride, uint32_t chunk_points)
{
	extern __shared__ __attribute__((aligned(16))) float lds[];
	const uint32_t groups = blockDim.x / gw;
	const uint32_t group = threadIdx.x / gw;
	const uint32_t gl = threadIdx.x - group * gw;
	for (uint32_t i = threadIdx.x; i < groups * copy_stride; i += blockDim.x) lds[i] = 0.0f;
	__syncthreads();

	float* acc = lds + (size_t)group * copy_stride;
	uint32_t* cnt = (uint32_t*)(acc + (size_t)k * dim);
	const uint32_t p_begin = (uint32_t)min((uint64_t)blockIdx.x * chunk_points, (uint64_t)n);
	const uint32_t p_end = (uint32_t)min((uint64_t)p_begin + chunk_points, (uint64_t)n);
	const bool lane_on = gl * 4 < dim;
	const float* src = data + (lane_on ? gl * 4 : 0);
	auto add_row = [&](uint32_t target, const f32x4& v) {
		if (lane_on) {
			f32x4* at = (f32x4*)(acc + target * dim + gl * 4);
			f32x4 a = *at;
			a.x += v.x; a.y += v.y; a.z += v.z; a.w += v.w;
			*at = a;
		}
		if (gl == 0) cnt[target] += 1u;
	};
	uint32_t p = p_begin + group;
	for (; p + (UPDATE_UNROLL_VEC - 1) * groups < p_end; p += UPDATE_UNROLL_VEC * groups) {
		f32x4 v[UPDATE_UNROLL_VEC];
		uint32_t t[UPDATE_UNROLL_VEC];
#pragma unroll
		for (int u = 0; u < UPDATE_UNROLL_VEC; ++u) {
			v[u] = *(const f32x4*)(src + (size_t)(p + u * groups) * stride);
			t[u] = assignment[p + u * groups];
		}
#pragma unroll
		for (int u = 0; u < UPDATE_UNROLL_VEC; ++u) add_row(t[u], v[u]);
	}
	for (; p < p_end; p += groups) add_row(assignment[p], *(const f32x4*)(src + (size_t)p * stride));
	__syncthreads();

	for (uint32_t e = threadIdx.x; e < k * dim; e += blockDim.x) {
		float s = 0.0f;
		for (uint32_t g = 0; g < groups; ++g) s += lds[(size_t)g * copy_stride + e];
		const uint32_t c = e / dim, d = e - c * dim;
		if (s != 0.0f) atomic_add_f32(&means[elem<LM>(stride_means, c, d)], s);
	}
	for (uint32_t c = threadIdx.x; c < k; c += blockDim.x) {
		uint32_t s = 0;
		for (uint32_t g = 0; g < groups; ++g) s += ((const uint32_t*)lds)[(size_t)g * copy_stride + (size_t)k * dim + c];
		if (s) atomicAdd(&sizes[c], s);
	}
}

/*
 * Larger k. Grid = (point chunks, 32-wide dimension slices); work-group = 1024 lanes.
 *   1. histogram of the chunk's assignments with ds_add_rtn_u32 (the returned value is the point's rank
 *      inside its cluster); 2. exclusive scan -> cluster offsets; 3. scatter (cluster << 15 | local index)
 *      into the sorted list; 4. the sorted list is cut into one range per lane group (groups of GW lanes,
 *      lane = dimension), every range the same number of entries; a group walks its range in batches of 8
 *      entries (8 row loads in flight), adds in a register and stores a cluster's row of sums when the cluster
 *      changes -- zero rows for clusters without members, so the partial buffer needs no clearing. The pieces
 *      of a cluster that spans ranges meet in LDS (measured at N = 2M, d = 32, k = 1024: 58 us with ranges of
 *      whole clusters, whose sizes differed by a cluster; 50 us with equal ranges).
 * Per-chunk counts go to a second partial array (dimension slice 0 only), so that nothing has to be zero beforehand.
 * partial layouts: [chunk][cluster][dim] and [chunk][cluster].
 */
constexpr uint32_t SORT_SHIFT = 15; /* local point index bits: chunk_points <= 32768 */
constexpr int SORT_UNROLL = 8;      /* row loads per batch and lane group in the segment-sum phase (two batches in flight; 16 measured slower) */

/* VEC consecutive floats of a row per lane: one 16-byte load when VEC = 4 (needs dim, stride % 4 == 0 and an aligned base). */
template <int VEC> struct RowPart { float v[VEC]; };

template <int VEC>
__device__ __forceinline__ RowPart<VEC> load_part(const float* p)
{
	RowPart<VEC> r;
	if constexpr (VEC == 4) {
		const f32x4 t = *(const f32x4*)p;
		r.v[0] = t.x; r.v[1] = t.y; r.v[2] = t.z; r.v[3] = t.w;
	} else {
#pragma unroll
		for (int i = 0; i < VEC; ++i) r.v[i] = p[i];
	}
	return r;
}

template <int VEC>
__device__ __forceinline__ void store_part(float* p, const RowPart<VEC>& r)
{
	if constexpr (VEC == 4) {
		f32x4 t;
		t.x = r.v[0]; t.y = r.v[1]; t.z = r.v[2]; t.w = r.v[3];
		*(f32x4*)p = t;
	} else {
#pragma unroll
		for (int i = 0; i < VEC; ++i) p[i] = r.v[i];
	}
}

template <int ITEMS, int GW, int VEC, bool WHOLE_ROWS = false>
__global__ void __launch_bounds__(1024)
update_sorted_kernel(const float* __restrict__ data, size_t stride, const uint32_t* __restrict__ assignment,
                     float* __restrict__ partial, uint32_t* __restrict__ partial_counts,
                     uint32_t dim, uint32_t k, uint32_t n, uint32_t chunk_points)
{
	extern __shared__ __attribute__((aligned(16))) uint32_t sm[];
	uint32_t* offsets = sm;                   /* k + 1 words: histogram, then exclusive offsets */
	uint32_t* scratch = sm + k + 1;           /* 32 words */
	uint32_t* sorted = sm + ((k + 36) & ~3u); /* chunk_points words (a multiple of 1024), then the 16-byte rows of `heads` */
	const uint32_t tid = threadIdx.x;
	const uint32_t lane = tid & (WAVE - 1), wave = tid / WAVE;
	const uint32_t p_begin = (uint32_t)min((uint64_t)blockIdx.x * chunk_points, (uint64_t)n);
	const uint32_t count = min(chunk_points, n - p_begin);
	/* The second grid dimension splits the work of a chunk: into slices of 32 dimensions, or (WHOLE_ROWS) into ranges of
	 * clusters, every lane group then reading whole rows -- one contiguous kilobyte at 256 dimensions instead of eight
	 * pieces of 128 bytes fetched by eight work-groups at unrelated times. */
	const uint32_t d0 = WHOLE_ROWS ? 0u : blockIdx.y * 32;
	const uint32_t width = WHOLE_ROWS ? dim : min(32u, dim - d0);

	for (uint32_t i = tid; i <= k; i += 1024) offsets[i] = 0;
	__syncthreads();

	/* 1. histogram + rank */
	uint32_t target[ITEMS], rank[ITEMS];
#pragma unroll
	for (int it = 0; it < ITEMS; ++it) {
		const uint32_t i = it * 1024 + tid;
		target[it] = i < count ? assignment[p_begin + i] : 0xFFFFFFFFu;
	}
#pragma unroll
	for (int it = 0; it < ITEMS; ++it) {
		rank[it] = 0;
		if (target[it] < k) rank[it] = atomicAdd(&offsets[target[it]], 1u);
	}
	__syncthreads();

	/* counts of this chunk: a row of the count partials, every entry written */
	if (blockIdx.y == 0)
		for (uint32_t c = tid; c < k; c += 1024) partial_counts[(size_t)blockIdx.x * k + c] = offsets[c];

	/* 2. exclusive scan of offsets[0..k) in place; offsets[k] = number of entries */
	const uint32_t per = (k + 1023) / 1024;
	const uint32_t b = tid * per;
	uint32_t local = 0;
	for (uint32_t i = 0; i < per; ++i)
		if (b + i < k) local += offsets[b + i];
	uint32_t incl = local;
	for (int off = 1; off < WAVE; off <<= 1) {
		const uint32_t up = (uint32_t)__shfl_up((int)incl, off);
		if (lane >= (uint32_t)off) incl += up;
	}
	if (lane == WAVE - 1) scratch[wave] = incl;
	__syncthreads();
	uint32_t wave_prefix = 0;
	for (uint32_t w = 0; w < wave; ++w) wave_prefix += scratch[w];
	uint32_t run = wave_prefix + incl - local;
	for (uint32_t i = 0; i < per; ++i)
		if (b + i < k) {
			const uint32_t c = offsets[b + i];
			offsets[b + i] = run;
			run += c;
		}
	if (b <= k && k < b + per) offsets[k] = run;        /* the thread that owns the last entries */
	if (tid == 1023 && b + per <= k) offsets[k] = run;   /* k a multiple of 1024: last thread closes the list */
	__syncthreads();

	/* 3. scatter */
#pragma unroll
	for (int it = 0; it < ITEMS; ++it)
		if (target[it] < k) sorted[offsets[target[it]] + rank[it]] = (target[it] << SORT_SHIFT) | (uint32_t)(it * 1024 + tid);
	__syncthreads();

	/* 4. segment sums */
	constexpr uint32_t GROUPS = 1024 / GW;
	const uint32_t group = tid / GW, gl = tid % GW;
	const uint32_t entries = offsets[k];
	const bool lane_on = gl * VEC < width;
	const float* src = data + (size_t)p_begin * stride + d0 + (lane_on ? gl * VEC : 0);
	float* out = partial + ((size_t)blockIdx.x * k) * dim + d0 + gl * VEC;
	constexpr uint32_t LOCAL_MASK = (1u << SORT_SHIFT) - 1u;

	/* the clusters [c_begin, c_stop) and their entries [e_begin, e_stop) that this work-group sums: all of them, or (WHOLE_ROWS)
	 * one of gridDim.y ranges of whole clusters, balanced by entry count */
	uint32_t c_begin = 0, c_stop = k;
	if constexpr (WHOLE_ROWS) {
		auto first_cluster = [&](uint32_t y) -> uint32_t {
			/* smallest c in [0, k] with offsets[c] >= y * entries / gridDim.y */
			if (y >= gridDim.y) return k;
			const uint32_t want = (uint32_t)((uint64_t)y * entries / gridDim.y);
			uint32_t lo = 0, hi = k;
			while (lo < hi) {
				const uint32_t mid = (lo + hi) / 2;
				if (offsets[mid] >= want) hi = mid; else lo = mid + 1;
			}
			return lo;
		};
		c_begin = first_cluster(blockIdx.y);
		c_stop = first_cluster(blockIdx.y + 1);
	}
	const uint32_t e_begin = offsets[c_begin], e_stop = offsets[c_stop];
	auto cluster_at = [&](uint32_t e) -> uint32_t { return e < e_stop ? sorted[e] >> SORT_SHIFT : c_stop; };
	auto range_begin = [&](uint32_t g) -> uint32_t { return e_begin + (uint32_t)((uint64_t)g * (e_stop - e_begin) / GROUPS); };

	/* Lane group g takes the entries [range_begin(g), range_begin(g + 1)): every group the same number of rows, whatever
	 * the cluster sizes (cut at cluster boundaries the ranges differed by a cluster's size, and the last group to finish set
	 * the time of the work-group). A cluster that spans ranges is summed in pieces: the range it starts in keeps its piece in
	 * registers, the ranges it continues in leave theirs in LDS, and after a barrier the first adds them up. */
	uint32_t e = range_begin(group), e_end = range_begin(group + 1);
	uint32_t cur, c_end;       /* cluster whose sum `acc` holds; cluster the range's last flush runs up to */
	bool head_pending = false; /* the first cluster of the range began in an earlier range: its sum goes to `heads` */
	bool tail_open = false;    /* the last cluster of the range goes on in later ranges: its sum waits in `acc` */
	float* heads = (float*)(sorted + chunk_points);     /* GROUPS rows of GW * VEC floats */
	uint32_t* whole = (uint32_t*)(heads + 1024 * VEC); /* GROUPS flags: the range lies inside one cluster that goes on behind it */
	if (gl == 0) whole[group] = 0u;
	if (e < e_end) {
		const uint32_t c_first = cluster_at(e), c_last = cluster_at(e_end - 1);
		head_pending = offsets[c_first] < e;
		tail_open = offsets[c_last + 1] > e_end;
		cur = e == e_begin ? c_begin : c_first; /* the group of the first entry also writes the rows of the empty clusters before it */
		c_end = cluster_at(e_end);              /* ... and every group those behind its last cluster */
	}
	else {
		/* no entry for this group; clusters without any entry still owe a row of zeros each */
		const bool none = e_begin == e_stop;
		cur = none ? c_begin + (uint32_t)((uint64_t)group * (c_stop - c_begin) / GROUPS) : 0u;
		c_end = none ? c_begin + (uint32_t)((uint64_t)(group + 1) * (c_stop - c_begin) / GROUPS) : 0u;
	}
	RowPart<VEC> acc;
#pragma unroll
	for (int i = 0; i < VEC; ++i) acc.v[i] = 0.0f;
	auto flush_to = [&](uint32_t t) {
		while (cur < t) {
			if (head_pending) {
				store_part<VEC>(heads + (size_t)group * (GW * VEC) + gl * VEC, acc);
				head_pending = false;
			}
			else if (lane_on) store_part<VEC>(out + (size_t)cur * dim, acc);
#pragma unroll
			for (int i = 0; i < VEC; ++i) acc.v[i] = 0.0f;
			++cur;
		}
	};
	/* software pipeline: the row loads of the next batch are issued before the current batch is summed */
	uint32_t ent[SORT_UNROLL];
	RowPart<VEC> v[SORT_UNROLL];
	bool have = e + SORT_UNROLL <= e_end;
	if (have) {
#pragma unroll
		for (int u = 0; u < SORT_UNROLL; ++u) ent[u] = sorted[e + u];
#pragma unroll
		for (int u = 0; u < SORT_UNROLL; ++u) v[u] = load_part<VEC>(src + (size_t)(ent[u] & LOCAL_MASK) * stride);
	}
	while (have) {
		e += SORT_UNROLL;
		const bool more = e + SORT_UNROLL <= e_end;
		uint32_t ent_next[SORT_UNROLL];
		RowPart<VEC> v_next[SORT_UNROLL];
		if (more) {
#pragma unroll
			for (int u = 0; u < SORT_UNROLL; ++u) ent_next[u] = sorted[e + u];
#pragma unroll
			for (int u = 0; u < SORT_UNROLL; ++u) v_next[u] = load_part<VEC>(src + (size_t)(ent_next[u] & LOCAL_MASK) * stride);
		}
#pragma unroll
		for (int u = 0; u < SORT_UNROLL; ++u) {
			flush_to(ent[u] >> SORT_SHIFT);
#pragma unroll
			for (int i = 0; i < VEC; ++i) acc.v[i] += v[u].v[i];
		}
		if (more) {
#pragma unroll
			for (int u = 0; u < SORT_UNROLL; ++u) {
				ent[u] = ent_next[u];
				v[u] = v_next[u];
			}
		}
		have = more;
	}
	if (e < e_end) {
		/* the last entries of the range, fewer than a batch: requested together like a batch */
#pragma unroll
		for (int u = 0; u < SORT_UNROLL; ++u) ent[u] = e + u < e_end ? sorted[e + u] : 0xFFFFFFFFu;
#pragma unroll
		for (int u = 0; u < SORT_UNROLL; ++u)
			if (ent[u] != 0xFFFFFFFFu) v[u] = load_part<VEC>(src + (size_t)(ent[u] & LOCAL_MASK) * stride);
#pragma unroll
		for (int u = 0; u < SORT_UNROLL; ++u)
			if (ent[u] != 0xFFFFFFFFu) {
				flush_to(ent[u] >> SORT_SHIFT);
#pragma unroll
				for (int i = 0; i < VEC; ++i) acc.v[i] += v[u].v[i];
			}
	}
	bool collect = false;
	if (tail_open) {
		if (head_pending) {
			/* the whole range lies inside one cluster that began before it and goes on behind it */
			store_part<VEC>(heads + (size_t)group * (GW * VEC) + gl * VEC, acc);
			if (gl == 0) whole[group] = 1u;
		}
		else collect = true;
	}
	else flush_to(c_end);
	__syncthreads();
	if (collect) {
		for (uint32_t g = group + 1; g < GROUPS; ++g) {
			if (range_begin(g) == range_begin(g + 1)) continue;
			const RowPart<VEC> piece = load_part<VEC>(heads + (size_t)g * (GW * VEC) + gl * VEC);
#pragma unroll
			for (int i = 0; i < VEC; ++i) acc.v[i] += piece.v[i];
			if (!whole[g]) break;
		}
		if (lane_on) store_part<VEC>(out + (size_t)cur * dim, acc);
	}
}

/*
 * means[c][d] = (sum over the chunks of partial[chunk][c][d]) / count[c]  (0 for an empty cluster).
 * Block = 64 consecutive elements x 16 chunk shares; every lane keeps up to 16 loads in flight; the shares meet in LDS.
 * Overwrites means: the sorted path needs neither zeroed centroids nor the separate divide kernel.
 * divide = 0 stores the sums themselves.
 */
constexpr uint32_t REDUCE_SHARES = 16;

template <int LM>
__global__ void __launch_bounds__(64 * REDUCE_SHARES)
reduce_partials_kernel(const float* __restrict__ partial, const uint32_t* __restrict__ partial_counts, float* __restrict__ means, size_t stride_means,
                       uint32_t* __restrict__ sizes, uint32_t dim, uint32_t k, uint32_t chunks, uint32_t divide)
{
	__shared__ float part[REDUCE_SHARES][64];
	__shared__ uint32_t part_count[REDUCE_SHARES][64];
	const uint32_t col = threadIdx.x & 63, share = threadIdx.x >> 6;
	const uint32_t shares = blockDim.x >> 6; /* 1 to REDUCE_SHARES: the launcher gives every share at least 8 chunks */
	const uint32_t e = blockIdx.x * 64 + col;
	const size_t kd = (size_t)k * dim;
	const uint32_t per = (chunks + shares - 1) / shares;
	const uint32_t c0 = min(share * per, chunks), c1 = min(c0 + per, chunks);
	/* the clusters the 64 elements of this work-group belong to (at most 64): lane `col` counts cluster cl_lo + col */
	const uint32_t cl_lo = (uint32_t)(((size_t)blockIdx.x * 64) / dim);
	const uint32_t cl_hi = (uint32_t)min((size_t)k - 1, ((size_t)blockIdx.x * 64 + 63) / dim);
	/* the count partials of this lane's cluster are requested first and added up after the sums, so that both sets of
	 * loads are in flight together */
	const bool counting = cl_lo + col <= cl_hi;
	const uint32_t* pc = partial_counts + cl_lo + (counting ? col : 0);
	uint32_t cv[16];
#pragma unroll
	for (int u = 0; u < 16; ++u) cv[u] = (counting && c0 + u < c1) ? pc[(size_t)(c0 + u) * k] : 0u;
	float s = 0.0f;
	if (e < kd) {
		uint32_t c = c0;
		for (; c + 16 <= c1; c += 16) {
			float v[16];
#pragma unroll
			for (int u = 0; u < 16; ++u) v[u] = partial[(size_t)(c + u) * kd + e];
#pragma unroll
			for (int u = 0; u < 16; ++u) s += v[u];
		}
		for (; c < c1; ++c) s += partial[(size_t)c * kd + e];
	}
	uint32_t members = 0;
#pragma unroll
	for (int u = 0; u < 16; ++u) members += cv[u];
	if (counting)
		for (uint32_t c = c0 + 16; c < c1; ++c) members += pc[(size_t)c * k];
	part_count[share][col] = members;
	part[share][col] = s;
	__syncthreads();
	if (share == 0 && e < kd) {
		s = 0.0f;
		for (uint32_t i = 0; i < shares; ++i) s += part[i][col];
		const uint32_t cl = e / dim, d = e - cl * dim;
		uint32_t count = 0;
		for (uint32_t i = 0; i < shares; ++i) count += part_count[i][cl - cl_lo];
		if (d == 0) sizes[cl] = count; /* the work-group that holds the cluster's first element publishes its size */
		means[elem<LM>(stride_means, cl, d)] = !divide ? s : (count ? s / (float)count : 0.0f);
	}
}

/* means (replica 0) and cluster sizes := 0 in one launch, for the kernels that accumulate into them */
__global__ void __launch_bounds__(256)
clear_outputs_kernel(uint32_t* __restrict__ means_words, size_t words, uint32_t* __restrict__ sizes, uint32_t k)
{
	const size_t threads = (size_t)blockDim.x * gridDim.x;
	for (size_t i = threadIdx.x + (size_t)blockIdx.x * blockDim.x; i < words + k; i += threads) {
		if (i < words) means_words[i] = 0u;
		else sizes[i - words] = 0u;
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

/* The tuned variant does not ask for zeroed outputs: the kernels that accumulate into them start with this. */
static int clear_outputs(const UpdateArgs& u)
{
	const size_t words = copy_floats_of(u);
	const uint32_t blocks = (uint32_t)std::min<size_t>((words + u.k + 255) / 256, 1024);
	KMX_LAUNCH_KERNEL(clear_outputs_kernel, dim3(std::max(blocks, 1u)), dim3(256), 0, stream(), (uint32_t*)u.means, words, u.cluster_sizes, u.k);
	KMX_LAUNCH_CHECK("clear_outputs_kernel");
	return KMX_OK;
}

static uint32_t pow2_at_least(uint32_t v)
{
	uint32_t p = 1;
	while (p < v) p <<= 1;
	return p;
}

template <int ITEMS, int LM>
static int launch_sorted(const UpdateArgs& u, Workspace* ws, uint32_t chunks, uint32_t slices, uint32_t chunk_points, uint32_t gw, uint32_t vec, uint32_t lds_bytes, bool whole_rows)
{
	void (*kernel)(const float*, size_t, const uint32_t*, float*, uint32_t*, uint32_t, uint32_t, uint32_t, uint32_t) = nullptr;
	uint32_t* partial_counts = (uint32_t*)(ws->partials + (size_t)chunks * u.k * u.dim);
	if (whole_rows) {
		switch (gw) {
		case 16: kernel = update_sorted_kernel<ITEMS, 16, 4, true>; break;
		case 32: kernel = update_sorted_kernel<ITEMS, 32, 4, true>; break;
		default: kernel = update_sorted_kernel<ITEMS, 64, 4, true>; break;
		}
	}
	else if (vec == 4) {
		switch (gw) {
		case 1: kernel = update_sorted_kernel<ITEMS, 1, 4>; break;
		case 2: kernel = update_sorted_kernel<ITEMS, 2, 4>; break;
		case 4: kernel = update_sorted_kernel<ITEMS, 4, 4>; break;
		default: kernel = update_sorted_kernel<ITEMS, 8, 4>; break;
		}
	} else {
		switch (gw) {
		case 4: kernel = update_sorted_kernel<ITEMS, 4, 1>; break;
		case 8: kernel = update_sorted_kernel<ITEMS, 8, 1>; break;
		case 16: kernel = update_sorted_kernel<ITEMS, 16, 1>; break;
		default: kernel = update_sorted_kernel<ITEMS, 32, 1>; break;
		}
	}
	KMX_HIP(hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
	KMX_LAUNCH_KERNEL(kernel, dim3(chunks, slices), dim3(1024), lds_bytes, stream(),
	                   u.data, u.stride, u.assignment, ws->partials, partial_counts, u.dim, u.k, u.n, chunk_points);
	KMX_LAUNCH_CHECK("update_sorted_kernel");
	const uint32_t total = u.k * u.dim;
	const uint32_t shares = std::max<uint32_t>(1, std::min<uint32_t>(REDUCE_SHARES, chunks / 8));
	KMX_LAUNCH_KERNEL((reduce_partials_kernel<LM>), dim3((total + 63) / 64), dim3(64 * shares), 0, stream(),
	                   ws->partials, partial_counts, u.means, u.stride_means, u.cluster_sizes, u.dim, u.k, chunks, u.divide ? 1u : 0u);
	KMX_LAUNCH_CHECK("reduce_partials_kernel");
	return KMX_OK;
}

/* Picks and launches the kernel of KMX_UPDATE_ATOMIC_SHM. *state: 0 = no LDS variant fits the shape, 1 = sums and
 * counts accumulated (divide still to do), 2 = centroids finished (the sorted path divides while it folds the partials). */
template <int LD, int LM>
static int launch_update_tuned(const UpdateArgs& u, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev, int* state)
{
	*state = 1;
	const uint32_t budget = exec->shared_mem_bytes ? std::min(exec->shared_mem_bytes, dev.lds_bytes) : dev.lds_bytes;

	if (LD == KMX_AOS && u.dim >= 8 && u.dim <= 64 && u.dim % 4 == 0 && u.stride % 4 == 0 && ((uintptr_t)u.data & 15) == 0 && u.n >= (1u << 20)) {
		/* private copies for groups of dim / 4 lanes with 16-byte row pieces (from a million points on: clearing and folding four
		 * times as many copies costs small inputs more than the wider loads save) */
		const uint32_t gw = pow2_at_least(u.dim / 4);
		const uint32_t groups = 256 / gw;
		const uint64_t copy_words = (uint64_t)u.k * (u.dim + 1);
		const uint64_t copy_stride = (copy_words + 31) / 32 * 32 + 4 * gw; /* groups of one 128-byte LDS cycle start 4 gw banks apart */
		const uint64_t lds_bytes = groups * copy_stride * 4;
		if (lds_bytes <= std::min<uint32_t>(budget, 96 * 1024)) {
			const uint32_t wg_per_cu = std::max<uint32_t>(1, std::min<uint32_t>(8, (uint32_t)(dev.lds_bytes / lds_bytes)));
			uint32_t chunks = dev.compute_units * wg_per_cu;
			const uint32_t quantum = groups * UPDATE_UNROLL_VEC;
			uint32_t chunk_points = (u.n + chunks - 1) / chunks;
			chunk_points = (chunk_points + quantum - 1) / quantum * quantum;
			chunks = (u.n + chunk_points - 1) / chunk_points;
			exec->block_count = chunks;
			int rc = clear_outputs(u);
			if (rc) return rc;
			KMX_HIP(hipFuncSetAttribute((const void*)update_private_vec_kernel<LM>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
			KMX_LAUNCH_KERNEL((update_private_vec_kernel<LM>), dim3(chunks), dim3(256), (uint32_t)lds_bytes, stream(),
			                   u.data, u.stride, u.assignment, u.means, u.stride_means, u.cluster_sizes,
			                   u.dim, u.k, u.n, gw, (uint32_t)copy_stride, chunk_points);
			KMX_LAUNCH_CHECK("update_private_vec_kernel");
			return KMX_OK;
		}
	}

	if (LD == KMX_AOS && u.dim <= 64) {
		/* private copies: 256 / gw groups, each k*dim sums + k counts, padded so that groups start gw banks apart */
		const uint32_t gw = pow2_at_least(u.dim);
		const uint32_t groups = 256 / gw;
		const uint64_t copy_words = (uint64_t)u.k * (u.dim + 1);
		const uint64_t copy_stride = (copy_words + 63) / 64 * 64 + gw;
		const uint64_t lds_bytes = groups * copy_stride * 4;
		if (lds_bytes <= std::min<uint32_t>(budget, 96 * 1024)) {
			const uint32_t wg_per_cu = std::max<uint32_t>(1, std::min<uint32_t>(8, (uint32_t)(dev.lds_bytes / lds_bytes)));
			uint32_t chunks = dev.compute_units * wg_per_cu;
			const uint32_t quantum = groups * UPDATE_UNROLL;
			uint32_t chunk_points = (u.n + chunks - 1) / chunks;
			chunk_points = (chunk_points + quantum - 1) / quantum * quantum;
			chunks = (u.n + chunk_points - 1) / chunk_points;
			exec->block_count = chunks;
			int rc = clear_outputs(u);
			if (rc) return rc;
			KMX_LAUNCH_KERNEL((update_private_kernel<LM>), dim3(chunks), dim3(256), (uint32_t)lds_bytes, stream(),
			                   u.data, u.stride, u.assignment, u.means, u.stride_means, u.cluster_sizes,
			                   u.dim, u.k, u.n, gw, (uint32_t)copy_stride, chunk_points);
			KMX_LAUNCH_CHECK("update_private_kernel");
			return KMX_OK;
		}
	}

	if (LD == KMX_AOS && u.k < (1u << (32 - SORT_SHIFT)) && (uint64_t)(u.k + 36) * 4 + 1024 * 4 + 1024 * 5 * 4 <= budget) {
		const uint32_t slices = (u.dim + 31) / 32;
		/* 16-byte row parts where one slice covers the row and its alignment allows it (measured: no gain for sliced rows) */
		const bool aligned4 = u.dim % 4 == 0 && u.stride % 4 == 0 && ((uintptr_t)u.data & 15) == 0;
		/* rows of 33 to 256 dimensions: the work-groups of a chunk take ranges of clusters and read whole rows (measured at
		 * N = 1M, d = 256, k = 1024: 0.29 ms in slices of 32 dimensions) */
		const bool whole_rows = u.dim > 32 && u.dim <= 256 && aligned4;
		/* 16-byte row parts where one slice covers the row and its alignment allows it (measured: no gain for sliced rows) */
		const uint32_t vec = ((u.dim <= 32 && aligned4) || whole_rows) ? 4 : 1;
		const uint32_t gw = whole_rows ? std::max<uint32_t>(16, pow2_at_least(u.dim / 4)) : (u.dim > 16 ? 32 : pow2_at_least(std::max<uint32_t>(u.dim, 4))) / vec;
		const uint32_t pieces_bytes = 1024u * (vec + 1) * 4; /* sums of clusters cut by a range boundary, and a flag per lane group */
		const uint32_t max_points = std::min<uint32_t>(1u << SORT_SHIFT, (budget - (u.k + 36) * 4 - pieces_bytes) / 4 / 1024 * 1024);
		/* one chunk per compute unit; two for rows of at most 16 bytes, whose chunks are bound by the sorting, not by their
		 * traffic (N = 4M, d = 4: k = 256 0.056 -> 0.045 ms, k = 1024 0.057 -> 0.048 ms, k = 4096 0.070 -> 0.066 ms; rows of
		 * 8 and 16 dimensions: no gain, and four per compute unit lose) */
		uint32_t chunks = std::max<uint32_t>(1, dev.compute_units * (u.dim <= 4 ? 2u : 1u) / slices);
		uint32_t chunk_points = (u.n + chunks - 1) / chunks;
		chunk_points = std::min(max_points, (chunk_points + 1023) / 1024 * 1024);
		chunks = (u.n + chunk_points - 1) / chunk_points;
		const uint32_t lds_bytes = (u.k + 36 + chunk_points) * 4 + pieces_bytes;
		int rc = reserve_partials(ws, (size_t)chunks * u.k * u.dim + (size_t)chunks * u.k); /* sums, then counts */
		if (rc) return rc;
		exec->block_count = chunks * slices;
		*state = 2;
		const uint32_t items = chunk_points / 1024;
		if (items <= 4) return launch_sorted<4, LM>(u, ws, chunks, slices, chunk_points, gw, vec, lds_bytes, whole_rows);
		if (items <= 8) return launch_sorted<8, LM>(u, ws, chunks, slices, chunk_points, gw, vec, lds_bytes, whole_rows);
		if (items <= 16) return launch_sorted<16, LM>(u, ws, chunks, slices, chunk_points, gw, vec, lds_bytes, whole_rows);
		return launch_sorted<32, LM>(u, ws, chunks, slices, chunk_points, gw, vec, lds_bytes, whole_rows);
	}

	/* fallback: LDS-privatised floating-point atomics */
	const uint32_t pad = LD == KMX_AOS ? 0 : 1;
	const uint32_t words = budget / 4;
	uint32_t slice = 0;
	if (words > u.k) slice = std::min<uint32_t>(u.dim, (words - u.k) / u.k > pad ? (words - u.k) / u.k - pad : 0);
	if (LD == KMX_AOS) slice = std::min<uint32_t>(slice, 1024);
	if (slice < u.dim) {
		for (uint32_t nice : { 32u, 16u, 8u, 4u })
			if (slice >= nice) { slice = slice / nice * nice; break; }
	}
	int rc = clear_outputs(u);
	if (rc) return rc;
	if (slice == 0) {
		*state = 0;
		return KMX_OK;
	}
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
	KMX_LAUNCH_KERNEL(kernel, dim3(chunks, slices), dim3(wg), lds_bytes, stream(),
	                   u.data, u.stride, u.assignment, u.means, u.stride_means, u.cluster_sizes,
	                   u.dim, u.k, u.n, slice, chunk_points, replicas);
	KMX_LAUNCH_CHECK("update_lds_kernel");
	return KMX_OK;
}

template <int LD, int LM>
static int launch_update_t(int variant, const UpdateArgs& u, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev)
{
	uint32_t block = exec->block_size ? exec->block_size : 256;
	block = std::min<uint32_t>((block + WAVE - 1) / WAVE * WAVE, 1024);
	const uint32_t ipt = exec->items_per_thread ? exec->items_per_thread : 1;
	const size_t copy_floats = copy_floats_of(u);
	uint32_t copies = exec->privatized_copies;
	const bool emulated = (variant & KMX_UPDATE_EMULATED_ATOMICS) != 0;
	variant &= ~KMX_UPDATE_EMULATED_ATOMICS;

	int rc = KMX_OK;
	if (u.n > 0) {
		if ((rc = profile_begin(1))) return rc;
		if (variant == KMX_UPDATE_ATOMIC_SHM) {
			int state = 0;
			rc = launch_update_tuned<LD, LM>(u, exec, ws, dev, &state);
			if (rc) return rc;
			if (state == 2) return profile_end(1); /* nothing left to merge or divide */
			if (state == 1) copies = 1; /* the tuned kernels write replica 0 only */
			else {
				variant = KMX_UPDATE_ATOMIC_FINE; /* k too large for any LDS privatisation */
				copies = 1;
			}
		}
#define KMX_UPDATE_LAUNCH(KERNEL, NAME) \
	do { \
		if (emulated) KMX_LAUNCH_KERNEL((KERNEL<LD, LM, true>), dim3(exec->block_count), dim3(block), 0, stream(), u.data, u.stride, u.assignment, \
		                                 u.means, u.stride_means, u.cluster_sizes, u.dim, u.k, u.n, copy_floats, copies); \
		else KMX_LAUNCH_KERNEL((KERNEL<LD, LM, false>), dim3(exec->block_count), dim3(block), 0, stream(), u.data, u.stride, u.assignment, \
		                        u.means, u.stride_means, u.cluster_sizes, u.dim, u.k, u.n, copy_floats, copies); \
		KMX_LAUNCH_CHECK(NAME); \
	} while (0)
		if (variant == KMX_UPDATE_ATOMIC_POINT) {
			uint32_t threads = (u.n + ipt - 1) / ipt;
			exec->block_count = (threads + block - 1) / block;
			KMX_UPDATE_LAUNCH(update_point_kernel, "update_point_kernel");
		}
		else if (variant == KMX_UPDATE_ATOMIC_WARP) {
			size_t threads = ((size_t)u.n * WAVE + ipt - 1) / ipt;
			exec->block_count = (uint32_t)std::min<size_t>((threads + block - 1) / block, 1u << 20);
			KMX_UPDATE_LAUNCH(update_warp_kernel, "update_warp_kernel");
		}
		else if (variant == KMX_UPDATE_ATOMIC_FINE) {
			size_t threads = ((size_t)u.n * u.dim + ipt - 1) / ipt;
			size_t blocks = (threads + block - 1) / block;
			exec->block_count = (uint32_t)std::min<size_t>(blocks, 1u << 20);
			KMX_UPDATE_LAUNCH(update_fine_kernel, "update_fine_kernel");
		}
		else if (variant == KMX_UPDATE_ATOMIC_SHM2 || variant == KMX_UPDATE_FAKE || variant == KMX_UPDATE_FAKE_SHM) {
			/* the micro-benchmark's launch shape: one lane per input element (or per items_per_thread elements) */
			const size_t threads = ((size_t)u.n * u.dim + ipt - 1) / ipt;
			exec->block_count = (uint32_t)std::min<size_t>((threads + block - 1) / block, 1u << 20);
			const uint32_t budget = exec->shared_mem_bytes ? std::min(exec->shared_mem_bytes, dev.lds_bytes) : dev.lds_bytes;
			if (variant == KMX_UPDATE_ATOMIC_SHM2) {
				const size_t one_copy = (size_t)u.k * u.dim * sizeof(float);
				const uint32_t lds_copies = (uint32_t)std::min<size_t>(budget / one_copy, block);
				if (lds_copies < 1) return fail(KMX_ERR_UNSUPPORTED, "Insufficient shared memory size for given parameters.");
				const uint32_t lds_bytes = (uint32_t)(lds_copies * one_copy);
				auto kernel = update_shm2_kernel<LD, LM>;
				KMX_HIP(hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
				KMX_LAUNCH_KERNEL(kernel, dim3(exec->block_count), dim3(block), lds_bytes, stream(), u.data, u.stride, u.assignment,
				                   u.means, u.stride_means, u.cluster_sizes, u.dim, u.k, u.n, copy_floats, copies, lds_copies);
				KMX_LAUNCH_CHECK("update_shm2_kernel");
			}
			else if (variant == KMX_UPDATE_FAKE) {
				if (emulated) KMX_LAUNCH_KERNEL((update_fake_kernel<LM, true>), dim3(exec->block_count), dim3(block), 0, stream(),
				                                 u.means, u.stride_means, u.dim, u.k, u.n, copy_floats, copies);
				else KMX_LAUNCH_KERNEL((update_fake_kernel<LM, false>), dim3(exec->block_count), dim3(block), 0, stream(),
				                        u.means, u.stride_means, u.dim, u.k, u.n, copy_floats, copies);
				KMX_LAUNCH_CHECK("update_fake_kernel");
			}
			else {
				const uint32_t cached = (uint32_t)std::min<size_t>(budget / (u.dim * sizeof(float)), u.k);
				const uint32_t lds_bytes = cached * u.dim * (uint32_t)sizeof(float);
				auto kernel = update_fake_shm_kernel<LM>;
				KMX_HIP(hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
				KMX_LAUNCH_KERNEL(kernel, dim3(exec->block_count), dim3(block), lds_bytes, stream(),
				                   u.means, u.stride_means, u.dim, u.k, u.n, copy_floats, copies, cached);
				KMX_LAUNCH_CHECK("update_fake_shm_kernel");
			}
		}
		else if (variant == KMX_UPDATE_BASE) {
			exec->block_count = (u.k * u.dim + 255) / 256;
			copies = 1; /* no replicas: every element of the result has one owner */
			KMX_LAUNCH_KERNEL((update_base_kernel<LD, LM>), dim3(exec->block_count), dim3(256), 0, stream(),
			                   u.data, u.stride, u.assignment, u.means, u.stride_means, u.cluster_sizes, u.dim, u.k, u.n);
			KMX_LAUNCH_CHECK("update_base_kernel");
		}
#undef KMX_UPDATE_LAUNCH
		if ((rc = profile_end(1))) return rc;
	}
	else if (variant == KMX_UPDATE_ATOMIC_SHM) {
		if ((rc = clear_outputs(u))) return rc; /* no points: every cluster is empty */
	}

	const uint32_t total = u.k * u.dim;
	const uint32_t blocks = std::min<uint32_t>((total + 255) / 256, 1024);
	if (copies > 1) {
		KMX_LAUNCH_KERNEL((reduce_copies_kernel<LM>), dim3(blocks), dim3(256), 0, stream(), u.means, u.stride_means, copy_floats, u.dim, u.k, copies);
		KMX_LAUNCH_CHECK("reduce_copies_kernel");
	}
	if (u.divide) {
		KMX_LAUNCH_KERNEL((divide_means_kernel<LM>), dim3(blocks), dim3(256), 0, stream(), u.means, u.stride_means, u.cluster_sizes, u.dim, u.k);
		KMX_LAUNCH_CHECK("divide_means_kernel");
	}
	return KMX_OK;
}

/* means[c][d] /= count[c] for the non-empty clusters (divideMeansKernel of the reference, kernels.cu:149-171) */
int launch_divide_means(const UpdateArgs& u)
{
	const uint32_t total = u.k * u.dim;
	const uint32_t blocks = std::min<uint32_t>((total + 255) / 256, 1024);
	if (u.layout_means == KMX_AOS)
		KMX_LAUNCH_KERNEL((divide_means_kernel<KMX_AOS>), dim3(blocks), dim3(256), 0, stream(), u.means, u.stride_means, u.cluster_sizes, u.dim, u.k);
	else
		KMX_LAUNCH_KERNEL((divide_means_kernel<KMX_SOA>), dim3(blocks), dim3(256), 0, stream(), u.means, u.stride_means, u.cluster_sizes, u.dim, u.k);
	KMX_LAUNCH_CHECK("divide_means_kernel");
	return KMX_OK;
}

/*
 * SoA points and the tuned variant: the kernels that read whole rows (sorted chunks, private copies) are 5 to 10 times
 * faster than anything that adds element by element (measured at N = 2M, d = 32, k = 1024: 0.07 ms against 0.68 ms for the
 * LDS atomics), more than a transposition costs. The points are therefore copied into AoS rows first: tiles of
 * 64 points x 32 dimensions through LDS, reads contiguous along the points, writes contiguous along the dimensions.
 * Rows of fewer than 8 dimensions stay with the element-wise kernel (0.11 ms against 0.15 ms at N = 4M, d = 4, k = 4096).
 */
constexpr size_t ROWS_COPY_MAX_BYTES = (size_t)4 << 30; /* larger inputs keep the element-wise kernel */

__global__ void __launch_bounds__(256)
rows_from_soa_kernel(const float* __restrict__ data, size_t stride, float* __restrict__ rows, uint32_t dim, uint32_t n)
{
	__shared__ float tile[32][65];
	const uint32_t tiles_q = (dim + 31) / 32;
	const size_t tiles = (size_t)((n + 63) / 64) * tiles_q;
	for (size_t t = blockIdx.x; t < tiles; t += gridDim.x) {
		const uint32_t p0 = (uint32_t)(t / tiles_q) * 64, q0 = (uint32_t)(t % tiles_q) * 32;
		__syncthreads(); /* the previous tile has been written out */
		for (uint32_t q = threadIdx.x / 64; q < 32; q += 4) {
			const uint32_t p = threadIdx.x % 64;
			if (q0 + q < dim && p0 + p < n) tile[q][p] = data[(size_t)(q0 + q) * stride + p0 + p];
		}
		__syncthreads();
		for (uint32_t p = threadIdx.x / 32; p < 64; p += 8) {
			const uint32_t q = threadIdx.x % 32;
			if (q0 + q < dim && p0 + p < n) rows[(size_t)(p0 + p) * dim + q0 + q] = tile[q][p];
		}
	}
}

/*
 * Scratch memory of kmx_update_f32_noalloc: the per-chunk partial sums and counts of update_sorted_kernel, the only
 * device memory beyond inputs and outputs the update uses with AoS points. One copy per GPU, held until the process
 * ends. In host code the array's name is only a stand-in: its device address on the current device comes from
 * hipGetSymbolAddress, once per device, and that pointer is what the kernels get.
 */
static __device__ __align__(256) float scratch[KMX_UPDATE_NOALLOC_SCRATCH_BYTES / sizeof(float)];

constexpr int NOALLOC_MAX_DEVICES = 64;
static Workspace g_noalloc_ws[NOALLOC_MAX_DEVICES];

int noalloc_workspace(Workspace** ws)
{
	int device = 0;
	KMX_HIP(hipGetDevice(&device));
	if (device < 0 || device >= NOALLOC_MAX_DEVICES) return fail(KMX_ERR_UNSUPPORTED, "kmx_update_f32_noalloc: device %d is beyond the %d devices the library keeps scratch pointers for", device, NOALLOC_MAX_DEVICES);
	Workspace& w = g_noalloc_ws[device];
	if (!w.partials) {
		/* the first look-up on a device loads the library's code and its 64 MiB array there: not under a recording */
		if (recording_graph())
			return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_update_f32_noalloc: the first call on a device sets up its scratch array, which cannot happen while a graph "
			                                      "is recorded: call kmx_set_device, kmx_reserve_f32 or kmx_update_f32_noalloc once before kmx_graph_begin");
		float* ptr = nullptr;
		KMX_HIP(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)));
		if (!ptr) return fail(KMX_ERR_DEVICE, "kmx_update_f32_noalloc: the scratch array has no address on device %d", device);
		w.partials = ptr;
		w.partials_cap = KMX_UPDATE_NOALLOC_SCRATCH_BYTES / sizeof(float);
		w.fixed = true;
	}
	*ws = &w;
	return KMX_OK;
}

int clear_update_outputs(const UpdateArgs& u) { return clear_outputs(u); }

int launch_update(int variant, const UpdateArgs& u, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev)
{
	if (variant == KMX_UPDATE_SERIAL_ORDER)
		return launch_update_serial_order<float>(u.data, u.layout, u.stride, u.assignment, u.means, u.layout_means, u.stride_means, u.cluster_sizes,
		                                         u.dim, u.k, u.n, u.divide, exec, ws, dev);
	/* (the fixed work space has no room for a copy of the points: SoA points then stay with the element-wise kernels) */
	if (!ws->fixed && u.layout == KMX_SOA && (variant & ~KMX_UPDATE_EMULATED_ATOMICS) == KMX_UPDATE_ATOMIC_SHM && u.n > 0 && u.dim >= 8 &&
	    (size_t)u.n * u.dim * sizeof(float) <= ROWS_COPY_MAX_BYTES) {
		int rc = reserve_rows_copy(ws, (size_t)u.n * u.dim);
		if (rc) return rc;
		const size_t tiles = (size_t)((u.n + 63) / 64) * ((u.dim + 31) / 32);
		KMX_LAUNCH_KERNEL(rows_from_soa_kernel, dim3((uint32_t)std::min<size_t>(tiles, (size_t)dev.compute_units * 32)), dim3(256), 0, stream(),
		                   u.data, u.stride, ws->rows_copy, u.dim, u.n);
		KMX_LAUNCH_CHECK("rows_from_soa_kernel");
		UpdateArgs rows = u;
		rows.data = ws->rows_copy; rows.layout = KMX_AOS; rows.stride = u.dim;
		return u.layout_means == KMX_AOS ? launch_update_t<KMX_AOS, KMX_AOS>(variant, rows, exec, ws, dev)
		                                 : launch_update_t<KMX_AOS, KMX_SOA>(variant, rows, exec, ws, dev);
	}
	if (u.layout == KMX_AOS && u.layout_means == KMX_AOS) return launch_update_t<KMX_AOS, KMX_AOS>(variant, u, exec, ws, dev);
	if (u.layout == KMX_AOS && u.layout_means == KMX_SOA) return launch_update_t<KMX_AOS, KMX_SOA>(variant, u, exec, ws, dev);
	if (u.layout == KMX_SOA && u.layout_means == KMX_AOS) return launch_update_t<KMX_SOA, KMX_AOS>(variant, u, exec, ws, dev);
	return launch_update_t<KMX_SOA, KMX_SOA>(variant, u, exec, ws, dev);
}

} // namespace kmx
