/*
 * KMX_UPDATE_SERIAL_ORDER: the update step with the bits of the serial loop, in O(n dim) work.
 *
 * The reference's CPU k-means adds the members of a cluster in ascending point order, one fp32 (or fp64) addition per
 * member and coordinate, starting from zero, and divides by the member count (serial.hpp:44-73). Floating-point
 * addition is not associative, so only that very order gives those very bits -- but the order only matters INSIDE a
 * cluster and coordinate: the k x dim chains are independent. This variant therefore
 *   1. sorts the point numbers by cluster with a STABLE counting sort (points of one cluster stay in ascending order):
 *      per-chunk histograms -> exclusive scan over (cluster, chunk) -> every chunk, one wavefront, walks its points in
 *      order, 64 at a time, and ranks the lanes that share a cluster by their lane number (ballots, no returning
 *      atomics, whose order would be arbitrary);
 *   2. gives every (cluster, coordinate) chain to one lane, which adds the rows of the sorted list one after the other
 *      with plain additions (no fused operations, no tree) and divides like divideMeansKernel.
 * A whole Lloyd run with this update and any assignment variant (all return the serial index) is bit-identical to the
 * reference's serial run. The price is the length of the longest chain: a cluster of m members is m dependent
 * additions, whatever the machine.
 *
 * Kernels: ordered_histogram_kernel, ordered_range_sums_kernel, ordered_offsets_kernel, ordered_starts_kernel,
 * ordered_scatter_kernel, ordered_sum_kernel.
 */
#include "kmx_internal.h"

#include <algorithm>

namespace kmx {

constexpr uint32_t ORDERED_LDS_CLUSTERS = 16384; /* up to here a chunk's counters live in LDS (64 KB per wavefront-sized work-group) */
constexpr uint32_t ORDERED_HIST_WORDS = 1u << 21; /* bound of chunks x k */
constexpr uint32_t ORDERED_MAX_CHUNKS = 4096;

/*
 * Histogram of one chunk of points: hist[chunk][cluster]. One wavefront per chunk, the same chunks as the scatter.
 * IN_LDS: counters in LDS, the row is written out whole (nothing to clear beforehand); otherwise the row in global
 * memory is the counter array (cleared by the launcher) and takes the atomics directly -- it belongs to this wavefront,
 * but two lanes may hold the same cluster.
 */
template <bool IN_LDS>
__global__ void __launch_bounds__(64)
ordered_histogram_kernel(const uint32_t* __restrict__ assignment, uint32_t* __restrict__ hist, uint32_t k, uint32_t n, uint32_t chunk_points)
{
	extern __shared__ uint32_t counters[];
	const uint32_t lane = threadIdx.x;
	uint32_t* row = hist + (size_t)blockIdx.x * k;
	if (IN_LDS) {
		for (uint32_t c = lane; c < k; c += WAVE) counters[c] = 0u;
		__syncthreads();
	}
	const uint32_t begin = blockIdx.x * chunk_points;          /* chunks * chunk_points < 2^32: the launcher keeps n below 2^32 - 2^20 */
	const uint32_t end = min(n, begin + chunk_points);
	for (uint32_t i = begin + lane; i < end; i += WAVE) {
		const uint32_t c = assignment[i];
		if (c >= k) continue; /* not a cluster: the point is left out, as by the scatter */
		if (IN_LDS) atomicAdd(&counters[c], 1u);
		else atomicAdd(&row[c], 1u);
	}
	if (IN_LDS) {
		__syncthreads();
		for (uint32_t c = lane; c < k; c += WAVE) row[c] = counters[c];
	}
}

/* range_sums[r][c] = sum of hist[chunk][c] over the chunks of range r (ranges of `per` chunks): first half of the scan
 * along the chunks, which for few clusters has too few columns to fill the machine with one lane per column */
__global__ void __launch_bounds__(256)
ordered_range_sums_kernel(const uint32_t* __restrict__ hist, uint32_t* __restrict__ range_sums, uint32_t k, uint32_t chunks, uint32_t ranges, uint32_t per)
{
	const size_t e = (size_t)blockIdx.x * 256 + threadIdx.x;
	if (e >= (size_t)ranges * k) return;
	const uint32_t c = (uint32_t)(e % k), r = (uint32_t)(e / k);
	const uint32_t c0 = min(chunks, r * per), c1 = min(chunks, c0 + per);
	uint32_t sum = 0;
	for (uint32_t chunk = c0; chunk < c1; ++chunk) sum += hist[(size_t)chunk * k + c];
	range_sums[e] = sum;
}

/* second half: hist[chunk][c] := number of members of cluster c in the chunks before `chunk` (exclusive scan along the
 * chunks, in place); the lane of the last range publishes the cluster's size */
__global__ void __launch_bounds__(256)
ordered_offsets_kernel(uint32_t* __restrict__ hist, const uint32_t* __restrict__ range_sums, uint32_t* __restrict__ sizes,
                       uint32_t k, uint32_t chunks, uint32_t ranges, uint32_t per)
{
	const size_t e = (size_t)blockIdx.x * 256 + threadIdx.x;
	if (e >= (size_t)ranges * k) return;
	const uint32_t c = (uint32_t)(e % k), r = (uint32_t)(e / k);
	uint32_t running = 0;
	for (uint32_t q = 0; q < r; ++q) running += range_sums[(size_t)q * k + c];
	const uint32_t c0 = min(chunks, r * per), c1 = min(chunks, c0 + per);
	for (uint32_t chunk = c0; chunk < c1; ++chunk) {
		const uint32_t members = hist[(size_t)chunk * k + c];
		hist[(size_t)chunk * k + c] = running;
		running += members;
	}
	if (r + 1 == ranges) sizes[c] = running;
}

/* starts[c] = sizes[0] + ... + sizes[c - 1]: one work-group; every lane scans a contiguous piece, the pieces meet in LDS */
__global__ void __launch_bounds__(1024)
ordered_starts_kernel(const uint32_t* __restrict__ sizes, uint32_t* __restrict__ starts, uint32_t k)
{
	__shared__ uint32_t piece_sum[1024];
	const uint32_t per = (k + 1023) / 1024;
	const uint32_t c0 = min(k, threadIdx.x * per), c1 = min(k, c0 + per);
	uint32_t sum = 0;
	for (uint32_t c = c0; c < c1; ++c) sum += sizes[c];
	piece_sum[threadIdx.x] = sum;
	__syncthreads();
	if (threadIdx.x == 0) {
		uint32_t running = 0;
		for (uint32_t t = 0; t < 1024; ++t) {
			const uint32_t s = piece_sum[t];
			piece_sum[t] = running;
			running += s;
		}
	}
	__syncthreads();
	uint32_t running = piece_sum[threadIdx.x];
	for (uint32_t c = c0; c < c1; ++c) {
		starts[c] = running;
		running += sizes[c];
	}
}

/*
 * sorted[starts[c] + members of c in earlier chunks + rank inside the chunk] = point number. One wavefront per chunk
 * walks its points in ascending order, 64 per step. Inside a step the lanes that share a cluster are ranked by lane
 * number: the lanes still waiting read the cluster of the first of them, a ballot names all lanes with that cluster,
 * a lane's rank is the number of those below it. The cluster's counter then moves on by the size of the group (written
 * by its last lane, after every lane of the group has read it: one wavefront, in program order). The order inside a
 * cluster is therefore the point order, which no returning atomic would promise.
 */
template <bool IN_LDS>
__global__ void __launch_bounds__(64)
ordered_scatter_kernel(const uint32_t* __restrict__ assignment, uint32_t* __restrict__ hist, const uint32_t* __restrict__ starts,
                       uint32_t* __restrict__ sorted, uint32_t k, uint32_t n, uint32_t chunk_points)
{
	extern __shared__ uint32_t counters[];
	const uint32_t lane = threadIdx.x;
	uint32_t* row = hist + (size_t)blockIdx.x * k;
	for (uint32_t c = lane; c < k; c += WAVE) {
		const uint32_t first = starts[c] + row[c];
		if (IN_LDS) counters[c] = first;
		else __hip_atomic_store(&row[c], first, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
	}
	if (!IN_LDS) __threadfence();
	__syncthreads();
	uint32_t* next = IN_LDS ? counters : row;
	const unsigned long long below = (1ull << lane) - 1ull;
	const uint32_t begin = blockIdx.x * chunk_points;
	const uint32_t end = min(n, begin + chunk_points);
	for (uint32_t base = begin; base < end; base += WAVE) {
		const uint32_t i = base + lane;
		const uint32_t c = i < end ? assignment[i] : 0xFFFFFFFFu;
		bool waiting = c < k;
		uint32_t rank = 0, group = 0;
		while (waiting) {
			const uint32_t first = __builtin_amdgcn_readfirstlane(c); /* cluster of the first lane still waiting */
			const unsigned long long same = __ballot(c == first);     /* the waiting lanes with that cluster: all lanes that have it */
			if (c == first) {
				rank = (uint32_t)__popcll(same & below);
				group = (uint32_t)__popcll(same);
				waiting = false;
			}
		}
		if (c < k) {
			/* counters in global memory: read and written past the vector cache, and fenced below, so that the lanes of the
			 * next step see what this step wrote */
			const uint32_t slot = (IN_LDS ? next[c] : __hip_atomic_load(&next[c], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) + rank;
			sorted[slot] = i;
			if (rank + 1 == group) {
				if (IN_LDS) next[c] = slot + 1;
				else __hip_atomic_store(&next[c], slot + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
			}
		}
		if (!IN_LDS) __threadfence();
	}
}

/*
 * One lane per cluster and piece of VEC consecutive coordinates (VEC = 1, or a 16-byte piece of an AoS row): the members'
 * coordinates added one after the other in the order of the sorted list, i.e. in ascending point number, starting from
 * zero like the serial loop (serial.hpp:57-63), then the guarded divide (serial.hpp:65-71). The additions of a
 * coordinate are a chain; what can overlap are the loads: the pieces of UNROLL rows are in flight together, and the
 * point numbers of the next UNROLL rows are requested before the current ones are added (a chain is as many sums as
 * the machine runs at once here, so the time is the latency of a load divided by the loads in flight).
 */
template <typename F, int VEC> struct alignas(sizeof(F) * VEC) OrderedPiece { F v[VEC]; };

template <typename F, int LD, int LM, int VEC, int UNROLL>
__global__ void __launch_bounds__(64)
ordered_sum_kernel(const F* __restrict__ data, size_t stride, const uint32_t* __restrict__ sorted, const uint32_t* __restrict__ starts,
                   const uint32_t* __restrict__ sizes, F* __restrict__ means, size_t stride_means, uint32_t dim, uint32_t k, uint32_t divide)
{
	static_assert(VEC == 1 || LD == KMX_AOS, "pieces of several coordinates are pieces of AoS rows");
	typedef OrderedPiece<F, VEC> piece_t;
	const uint32_t pieces = dim / VEC; /* the launcher picks VEC among the divisors of dim */
	const size_t e = (size_t)blockIdx.x * WAVE + threadIdx.x;
	if (e >= (size_t)k * pieces) return;
	const uint32_t c = (uint32_t)(e / pieces), d = (uint32_t)(e % pieces) * VEC;
	const uint32_t members = sizes[c];
	const uint32_t begin = starts[c], end = begin + members;
	piece_t sum;
#pragma unroll
	for (int i = 0; i < VEC; ++i) sum.v[i] = (F)0;
	if (members) {
		uint32_t point[UNROLL];
#pragma unroll
		for (int u = 0; u < UNROLL; ++u) point[u] = sorted[min(begin + u, end - 1)];
		for (uint32_t j = begin; j < end; j += UNROLL) {
			piece_t v[UNROLL];
#pragma unroll
			for (int u = 0; u < UNROLL; ++u) v[u] = *(const piece_t*)(data + elem<LD>(stride, point[u], d));
#pragma unroll
			for (int u = 0; u < UNROLL; ++u) point[u] = sorted[min(j + UNROLL + u, end - 1)];
#pragma unroll
			for (int u = 0; u < UNROLL; ++u) {
				if (j + u < end) {
#pragma unroll
					for (int i = 0; i < VEC; ++i) sum.v[i] = sum.v[i] + v[u].v[i];
				}
			}
		}
	}
#pragma unroll
	for (int i = 0; i < VEC; ++i)
		means[elem<LM>(stride_means, c, d + i)] = !divide ? sum.v[i] : (members ? sum.v[i] / (F)members : (F)0);
}

/* Work-groups of one wavefront: what bounds this kernel is the number of cache lines a compute unit keeps in flight, so
 * the chains are spread over as many compute units as there are wavefronts (measured at N = 2M, d = 32, k = 1024: 32
 * work-groups of four wavefronts with 16-byte pieces 0.85 ms). The 16-byte pieces, which need a quarter of the lanes, are
 * taken only where they still leave two wavefronts per compute unit. */
template <typename F, int LD, int LM>
static int launch_ordered_sum(const F* data, size_t stride, const uint32_t* sorted, const uint32_t* starts, const uint32_t* sizes,
                              F* means, size_t stride_means, uint32_t dim, uint32_t k, bool divide, const DeviceInfo& dev)
{
	constexpr int WIDE = 16 / sizeof(F);
	const bool fits = LD == KMX_AOS && dim % WIDE == 0 && stride % WIDE == 0 && ((uintptr_t)data & 15) == 0;
	const bool wide = fits && (size_t)k * (dim / WIDE) >= (size_t)2 * WAVE * dev.compute_units;
	const size_t total = (size_t)k * (wide ? dim / WIDE : dim);
	const dim3 grid((uint32_t)((total + WAVE - 1) / WAVE));
	if (wide)
		KMX_LAUNCH_KERNEL((ordered_sum_kernel<F, KMX_AOS, LM, WIDE, 32>), grid, dim3(WAVE), 0, stream(),
		                   data, stride, sorted, starts, sizes, means, stride_means, dim, k, divide ? 1u : 0u);
	else
		KMX_LAUNCH_KERNEL((ordered_sum_kernel<F, LD, LM, 1, 32>), grid, dim3(WAVE), 0, stream(),
		                   data, stride, sorted, starts, sizes, means, stride_means, dim, k, divide ? 1u : 0u);
	KMX_LAUNCH_CHECK("ordered_sum_kernel");
	return KMX_OK;
}

template <typename F>
int launch_update_serial_order(const F* data, int layout, size_t stride, const uint32_t* assignment,
                               F* means, int layout_means, size_t stride_means, uint32_t* cluster_sizes,
                               uint32_t dim, uint32_t k, uint32_t n, bool divide, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev)
{
	if (n > 0xFFFFFFFFu - (1u << 20)) return fail(KMX_ERR_UNSUPPORTED, "the serial-order update takes fewer than 2^32 - 2^20 points");
	if ((uint64_t)k * dim > 0xFFFFFFFFull * WAVE) return fail(KMX_ERR_UNSUPPORTED, "the serial-order update: k * dim is too large for one launch");
	/* chunks: one wavefront each, a multiple of 64 points, few enough that chunks x k counters stay small */
	uint32_t chunks = 0, chunk_points = WAVE;
	if (n > 0) {
		const uint32_t by_memory = std::max<uint32_t>(1, ORDERED_HIST_WORDS / k);
		chunks = std::min<uint32_t>({ by_memory, ORDERED_MAX_CHUNKS, (n + 255) / 256 });
		chunk_points = ((n + chunks - 1) / chunks + WAVE - 1) / WAVE * WAVE;
		chunks = (n + chunk_points - 1) / chunk_points;
	}
	const uint32_t ranges = std::max<uint32_t>(1, std::min<uint32_t>({ 64u, chunks, (16384 + k - 1) / k }));
	const uint32_t per = chunks ? (chunks + ranges - 1) / ranges : 0;
	const size_t hist_words = (size_t)std::max(chunks, 1u) * k, range_words = (size_t)ranges * k;
	int rc = reserve_partials(ws, hist_words + range_words + k + n);
	if (rc) return rc;
	uint32_t* hist = (uint32_t*)ws->partials;
	uint32_t* range_sums = hist + hist_words;
	uint32_t* starts = range_sums + range_words;
	uint32_t* sorted = starts + k;
	const bool in_lds = k <= ORDERED_LDS_CLUSTERS;
	const uint32_t lds_bytes = in_lds ? k * 4 : 0;

	if ((rc = profile_begin(1))) return rc;
	exec->block_count = chunks;
	if (chunks > 0) {
		if (in_lds) {
			KMX_HIP(hipFuncSetAttribute((const void*)ordered_histogram_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
			KMX_LAUNCH_KERNEL((ordered_histogram_kernel<true>), dim3(chunks), dim3(WAVE), lds_bytes, stream(), assignment, hist, k, n, chunk_points);
		}
		else {
			rc = kmx_fill_zero_u32(hist, hist_words);
			if (rc) return rc;
			KMX_LAUNCH_KERNEL((ordered_histogram_kernel<false>), dim3(chunks), dim3(WAVE), 0, stream(), assignment, hist, k, n, chunk_points);
		}
		KMX_LAUNCH_CHECK("ordered_histogram_kernel");
	}
	const uint32_t scan_blocks = (uint32_t)((range_words + 255) / 256);
	KMX_LAUNCH_KERNEL(ordered_range_sums_kernel, dim3(scan_blocks), dim3(256), 0, stream(), hist, range_sums, k, chunks, ranges, per);
	KMX_LAUNCH_CHECK("ordered_range_sums_kernel");
	KMX_LAUNCH_KERNEL(ordered_offsets_kernel, dim3(scan_blocks), dim3(256), 0, stream(), hist, range_sums, cluster_sizes, k, chunks, ranges, per);
	KMX_LAUNCH_CHECK("ordered_offsets_kernel");
	KMX_LAUNCH_KERNEL(ordered_starts_kernel, dim3(1), dim3(1024), 0, stream(), cluster_sizes, starts, k);
	KMX_LAUNCH_CHECK("ordered_starts_kernel");
	if (chunks > 0) {
		if (in_lds) {
			KMX_HIP(hipFuncSetAttribute((const void*)ordered_scatter_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
			KMX_LAUNCH_KERNEL((ordered_scatter_kernel<true>), dim3(chunks), dim3(WAVE), lds_bytes, stream(), assignment, hist, starts, sorted, k, n, chunk_points);
		}
		else
			KMX_LAUNCH_KERNEL((ordered_scatter_kernel<false>), dim3(chunks), dim3(WAVE), 0, stream(), assignment, hist, starts, sorted, k, n, chunk_points);
		KMX_LAUNCH_CHECK("ordered_scatter_kernel");
	}
	if (layout == KMX_AOS && layout_means == KMX_AOS) rc = launch_ordered_sum<F, KMX_AOS, KMX_AOS>(data, stride, sorted, starts, cluster_sizes, means, stride_means, dim, k, divide, dev);
	else if (layout == KMX_AOS) rc = launch_ordered_sum<F, KMX_AOS, KMX_SOA>(data, stride, sorted, starts, cluster_sizes, means, stride_means, dim, k, divide, dev);
	else if (layout_means == KMX_AOS) rc = launch_ordered_sum<F, KMX_SOA, KMX_AOS>(data, stride, sorted, starts, cluster_sizes, means, stride_means, dim, k, divide, dev);
	else rc = launch_ordered_sum<F, KMX_SOA, KMX_SOA>(data, stride, sorted, starts, cluster_sizes, means, stride_means, dim, k, divide, dev);
	if (rc) return rc;
	return profile_end(1);
}

template int launch_update_serial_order<float>(const float*, int, size_t, const uint32_t*, float*, int, size_t, uint32_t*, uint32_t, uint32_t, uint32_t, bool, kmx_exec_params*, Workspace*, const DeviceInfo&);
template int launch_update_serial_order<double>(const double*, int, size_t, const uint32_t*, double*, int, size_t, uint32_t*, uint32_t, uint32_t, uint32_t, bool, kmx_exec_params*, Workspace*, const DeviceInfo&);

} // namespace kmx
