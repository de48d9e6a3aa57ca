/*
 * The Lloyd iteration on doubles: kmx_assign_f64, kmx_update_f64, kmx_fused_f64.
 *
 * The reference instantiates every algorithm with F = double when its command line says --double
 * (experimental/k-means/k-means/k-means.cpp:341-342; kernels.cu:1200-1261 instantiates the kernels for both types).
 *
 * Assignment. gfx950 executes v_fma_f64 / v_add_f64 / v_mul_f64 at the rate of the plain fp32 instructions, so the
 * serial arithmetic itself -- diff, square, add, in ascending dimension, sqrt, strict comparison from centroid 0
 * (serial.hpp:21-35, metric_policies.hpp:17-47) -- is evaluated for every (point, centroid) pair: no ranking by a
 * cheaper expression, no certification, no second pass, and the result is the serial one by construction.
 * One lane per point; the centroids come eight at a time from a transposed copy ([dim][k rounded up to 8], written
 * by a small kernel first), where the eight values of one dimension are one 64-byte scalar load and feed the
 * subtractions as scalar operands. Rows of up to 32 doubles stay in registers for the whole sweep; longer rows are
 * re-read per group of eight centroids (L1/L2 hits).
 *   bound: 3 fp64 instructions (subtract, multiply, add: the serial code has no fused multiply-add) per point,
 *   centroid and dimension, one wavefront instruction per 4 cycles and SIMD: half of the fp64 peak, which counts FMAs.
 *   Measured at N = 2M, d = 32, k = 1024: 9 ms, 28 % of the peak, 57 % of that instruction bound.
 *
 * Update. One lane per element of the input (coalesced in either layout), as in the reference's updateAtomicFineKernel
 * (kernels.cu:770-809), with fp64 atomics, which gfx950 has natively in LDS and in L2: a work-group first adds into a
 * private copy of the sums in LDS when k * d doubles fit 32 KB and flushes it with one global atomic per element;
 * otherwise the lanes add to global memory directly. Counts are integer atomics issued by the lane of dimension 0.
 * The order of the additions is not the serial one (it is not in the reference's kernels either).
 */
#include "kmx_internal.h"

#include <algorithm>

#pragma clang fp contract(off) /* every multiply and add rounds separately, as in the serial code */

namespace kmx {

constexpr int GROUP = 8;       /* centroids per step: 8 doubles = one s_load_dwordx16 */
constexpr int WIDE_GROUP = 32; /* the same for rows that are re-read per step */

static inline uint32_t round_up_u32(uint32_t v, uint32_t m) { return (v + m - 1) / m * m; }

/* work space of the double-precision calls: transposed centroids; owned by this file, released by kmx_shutdown
 * through release_f64_workspace() */
static double* g_means_t = nullptr;
static size_t g_means_t_cap = 0;

template <int LM>
__global__ void __launch_bounds__(256)
transpose_means_f64_kernel(const double* __restrict__ means, size_t stride_means, double* __restrict__ means_t,
                           uint32_t dim, uint32_t k, uint32_t kp)
{
	const size_t total = (size_t)dim * kp;
	for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += (size_t)gridDim.x * blockDim.x) {
		const uint32_t q = (uint32_t)(e / kp), j = (uint32_t)(e % kp);
		means_t[e] = j < k ? means[elem<LM>(stride_means, j, q)] : 0.0;
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
	const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
	const uint32_t pt = min(i, n - 1); /* lanes past the end repeat the last point and store nothing */
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
	if (i < n) assignment[i] = nearest;
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
                         kmx_exec_params* exec)
{
	const dim3 block(256), grid((n + 255) / 256);
	exec->block_size = block.x;
	exec->block_count = grid.x;
	exec->shared_mem_bytes = 0;
#define KMX_F64_LAUNCH(DPAD, G) \
	hipLaunchKernelGGL((assign_f64_kernel<LD, DPAD, G>), grid, block, 0, stream(), data, stride, g_means_t, assignment, dim, k, kp, n)
	if (variant == KMX_ASSIGN_BASE) KMX_F64_LAUNCH(0, GROUP);
	else if (dim > 32) KMX_F64_LAUNCH(0, WIDE_GROUP);
	else if (dim <= 8) KMX_F64_LAUNCH(8, GROUP);
	else if (dim <= 16) KMX_F64_LAUNCH(16, GROUP);
	else KMX_F64_LAUNCH(32, GROUP);
#undef KMX_F64_LAUNCH
	KMX_LAUNCH_CHECK("assign_f64_kernel");
	return KMX_OK;
}

template <int LD, int LM>
int launch_update_f64_t(int variant, const double* data, size_t stride, const uint32_t* assignment, double* means, size_t stride_means,
                        uint32_t* sizes, uint32_t dim, uint32_t k, uint32_t n, kmx_exec_params* exec, const DeviceInfo& dev)
{
	const size_t private_bytes = ((size_t)k * dim) * sizeof(double) + (size_t)k * sizeof(uint32_t);
	const bool use_private = variant == KMX_UPDATE_ATOMIC_SHM && private_bytes <= 32 * 1024;
	const dim3 block(256);
	const size_t total = (size_t)n * dim;
	/* a work-group with private sums should add at least 16 times as many elements as it has sums to clear and flush */
	const size_t per_group = use_private ? std::max<size_t>(256, 16 * (size_t)k * dim) : 256;
	const uint32_t wanted = (uint32_t)std::min<size_t>((total + per_group - 1) / per_group, (size_t)dev.compute_units * (use_private ? 8 : 32));
	const dim3 grid(std::max<uint32_t>(wanted, 1));
	exec->block_size = block.x;
	exec->block_count = grid.x;
	exec->shared_mem_bytes = use_private ? (uint32_t)private_bytes : 0;
	if (n > 0) {
		if (use_private)
			hipLaunchKernelGGL((update_f64_kernel<LD, LM, true>), grid, block, private_bytes, stream(),
			                   data, stride, assignment, means, stride_means, sizes, dim, k, n);
		else
			hipLaunchKernelGGL((update_f64_kernel<LD, LM, false>), grid, block, 0, stream(),
			                   data, stride, assignment, means, stride_means, sizes, dim, k, n);
		KMX_LAUNCH_CHECK("update_f64_kernel");
	}
	hipLaunchKernelGGL((divide_means_f64_kernel<LM>), dim3((k * dim + 255) / 256), dim3(256), 0, stream(), means, stride_means, sizes, dim, k);
	KMX_LAUNCH_CHECK("divide_means_f64_kernel");
	return KMX_OK;
}

} // namespace

int release_f64_workspace()
{
	if (g_means_t) KMX_HIP(hipFree(g_means_t));
	g_means_t = nullptr;
	g_means_t_cap = 0;
	return KMX_OK;
}

} // namespace kmx

using namespace kmx;

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
	if (variant != KMX_ASSIGN_BASE && variant != KMX_ASSIGN_BEST)
		return fail(KMX_ERR_UNSUPPORTED, "kmx_assign_f64: only KMX_ASSIGN_BASE and KMX_ASSIGN_BEST are built for doubles (variant %d)", variant);
	const DeviceInfo* dev = nullptr;
	rc = device_info(&dev);
	if (rc) return rc;

	const uint32_t kp = round_up_u32(k, WIDE_GROUP);
	const size_t want = (size_t)kp * dim;
	if (want > g_means_t_cap) {
		rc = reserve_f64(&g_means_t, &g_means_t_cap, want);
		if (rc) return rc;
	}
	const dim3 tgrid((uint32_t)std::min<size_t>((want + 255) / 256, 1024));
	if (layout_means == KMX_AOS)
		hipLaunchKernelGGL((transpose_means_f64_kernel<KMX_AOS>), tgrid, dim3(256), 0, stream(), means, stride_means, g_means_t, dim, k, kp);
	else
		hipLaunchKernelGGL((transpose_means_f64_kernel<KMX_SOA>), tgrid, dim3(256), 0, stream(), means, stride_means, g_means_t, dim, k, kp);
	KMX_LAUNCH_CHECK("transpose_means_f64_kernel");

	rc = profile_begin(0);
	if (rc) return rc;
	rc = layout == KMX_AOS ? launch_assign_f64_ld<KMX_AOS>(variant, data, stride, assignment, dim, k, kp, n, exec)
	                       : launch_assign_f64_ld<KMX_SOA>(variant, data, stride, assignment, dim, k, kp, n, exec);
	if (rc) return rc;
	return profile_end(0);
}

extern "C" int kmx_update_f64(int variant,
                              const double* data, int layout, size_t stride,
                              const uint32_t* assignment,
                              double* means, int layout_means, size_t stride_means,
                              uint32_t* cluster_sizes,
                              uint32_t dim, uint32_t k, uint32_t n, kmx_exec_params* exec)
{
	clear_error();
	if (!exec) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_update_f64: exec is null");
	if (dim == 0 || k == 0) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_update_f64: dim and k must be positive");
	if (!means || !cluster_sizes) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_update_f64: null device pointer");
	if (n > 0 && (!data || !assignment)) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_update_f64: null device pointer");
	int rc = check_layout_f64("kmx_update_f64", "data", layout, stride, n, dim);
	if (rc) return rc;
	rc = check_layout_f64("kmx_update_f64", "means", layout_means, stride_means, k, dim);
	if (rc) return rc;
	if (variant < KMX_UPDATE_ATOMIC_POINT || variant > KMX_UPDATE_ATOMIC_SHM)
		return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_update_f64: unknown variant %d", variant);
	if (exec->privatized_copies > 1)
		return fail(KMX_ERR_UNSUPPORTED, "kmx_update_f64: privatized copies in global memory are not built for doubles");
	if ((uint64_t)k * dim > 0xffffffffull) return fail(KMX_ERR_UNSUPPORTED, "kmx_update_f64: k * dim does not fit 32 bits");
	const DeviceInfo* dev = nullptr;
	rc = device_info(&dev);
	if (rc) return rc;

	rc = profile_begin(1);
	if (rc) return rc;
#define KMX_F64_UPDATE(LD, LM) \
	launch_update_f64_t<LD, LM>(variant, data, stride, assignment, means, stride_means, cluster_sizes, dim, k, n, exec, *dev)
	if (layout == KMX_AOS) rc = layout_means == KMX_AOS ? KMX_F64_UPDATE(KMX_AOS, KMX_AOS) : KMX_F64_UPDATE(KMX_AOS, KMX_SOA);
	else rc = layout_means == KMX_AOS ? KMX_F64_UPDATE(KMX_SOA, KMX_AOS) : KMX_F64_UPDATE(KMX_SOA, KMX_SOA);
#undef KMX_F64_UPDATE
	if (rc) return rc;
	return profile_end(1);
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
