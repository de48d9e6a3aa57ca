/*
 * Assignment on the vector ALUs: one lane per point, the point's coordinates in registers, the packed centroids
 * (-2c rows and |c|^2, the same block pack_means_kernel writes for the MFMA variant) in LDS, read as broadcasts;
 * a[j] = |c_j|^2 - 2 c_j . x by plain v_fma_f32, exact (min, second min, argmin) tracking per lane, and the same
 * certification / recheck queue as the MFMA variant (the bound of a chain of fused multiply-adds: certificate.h).
 *
 * With a handful of centroids (the packed block within 8 KB: k = 16 at d = 16, k = 64 at d = 8) the rows are not staged
 * in LDS at all: they are read with wave-uniform addresses, i.e. as scalar loads through the scalar cache, and feed
 * the multiply-adds as scalar operands. That variant is the fastest sweep for k <= 32 (HBM-bound shapes; measured
 * 0.26 ms against 0.32 ms for the MFMA sweep at N = 16.7 M, d = 16, k = 16).
 *
 * This is the counterpart of the reference's shared-memory kernels (cachedFixedAssignmentKernel /
 * cachedRegsAssignmentKernel, reference kernels.cu:216-273,546-661): centroids cached on chip, distances
 * accumulated in registers. On gfx950 it is the SLOWER path at every shape that was measured: an fp32 MFMA
 * retires two multiply-adds per lane and cycle, a v_fma_f32 one (packed fp32 is not used), and the LDS
 * broadcast reads and the per-pair tracking come on top. It is kept as a selectable variant
 * (KMX_ASSIGN_LDS_FMA, `hip_lds_fma`) so that the choice can be measured; KMX_ASSIGN_BEST picks it only for
 * k <= 32 with the scalar-cache path.
 */
#include "certificate.h"
#include "assign_mfma_impl.h"

namespace kmx {

constexpr uint32_t FMA_WAVES = 4; /* wavefronts per work-group */

template <int DP, int LD, bool SCALAR>
__global__ void __launch_bounds__(FMA_WAVES * WAVE)
assign_lds_fma_kernel(const float* __restrict__ data, size_t stride, const float* __restrict__ packed, const float* __restrict__ norms,
                      uint32_t* __restrict__ assignment, uint32_t* __restrict__ queue, uint32_t* __restrict__ counters,
                      uint32_t dim, uint32_t k, uint32_t kp, uint32_t n, uint32_t chunk_rows, float kd, uint32_t vec4, float kd_unmoved)
{
	/* the frame of the sweep (sweep_frame; the packing kernel moved the centroids): the same words for every lane, so
	 * they arrive as scalar operands */
	const float* __restrict__ frame = norms + plain_frame_offset(kp);
	const float frame_m2 = frame[FRAME_DIMS], frame_norm = frame[FRAME_DIMS + 1];
	constexpr uint32_t RS = DP + ROW_PAD;
	extern __shared__ float lds[];
	__shared__ uint32_t wave_max[FMA_WAVES];
	__shared__ uint32_t flag_list[FMA_WAVES][2 * FLAG_CAP]; /* (point, threshold) pairs */
	const uint32_t lane = threadIdx.x & (WAVE - 1);
	const uint32_t wave = threadIdx.x / WAVE;

	uint32_t cmax = 0;
	for (uint32_t j = threadIdx.x; j < k; j += blockDim.x) cmax = max(cmax, __float_as_uint(norms[norm_at(j)]));
	for (int off = WAVE / 2; off > 0; off >>= 1) cmax = max(cmax, (uint32_t)__shfl_xor((int)cmax, off));
	if (lane == 0) wave_max[wave] = cmax;
	__syncthreads();
	cmax = 0;
	for (uint32_t w = 0; w < FMA_WAVES; ++w) cmax = max(cmax, wave_max[w]);
	const float c2max = __uint_as_float(cmax);

	float* lds_norms = lds + (size_t)(chunk_rows / TILE) * tile_floats(RS);
	const uint32_t chunks = (kp + chunk_rows - 1) / chunk_rows;
	auto stage = [&](uint32_t row0, uint32_t rows) {
		const f32x4* src = (const f32x4*)(packed + packed_row(row0, RS));
		f32x4* dst = (f32x4*)lds;
		const uint32_t vecs = (rows / TILE) * tile_floats(RS) / 4;
		for (uint32_t i = threadIdx.x; i < vecs; i += blockDim.x) dst[i] = src[i];
		const f32x4* nsrc = (const f32x4*)(norms + (size_t)(row0 / TILE) * NORM_TILE);
		f32x4* ndst = (f32x4*)lds_norms;
		const uint32_t nvecs = (rows / TILE) * NORM_TILE / 4;
		for (uint32_t i = threadIdx.x; i < nvecs; i += blockDim.x) ndst[i] = nsrc[i];
	};
	/* SCALAR: a handful of centroids. Their rows are read straight from memory with wave-uniform addresses, which the
	 * compiler turns into scalar loads: the values arrive in scalar registers through the scalar cache and feed the
	 * multiply-adds as scalar operands -- no LDS traffic at all, which is what bounds the LDS variant (one 128-bit
	 * LDS read per four multiply-adds). */
	const bool resident = chunks == 1 || SCALAR;
	if (resident && !SCALAR) {
		stage(0, kp);
		__syncthreads();
	}

	uint32_t flagged = 0; /* wave-uniform */
	auto flush_flags = [&]() {
		__builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
		__builtin_amdgcn_wave_barrier();
		uint32_t slot = 0;
		if (lane == 0) slot = atomicAdd(&counters[0], flagged);
		slot = (uint32_t)__shfl((int)slot, 0);
		for (uint32_t i = lane; i < 2 * flagged; i += WAVE) queue[2 * (size_t)slot + i] = flag_list[wave][i];
		__builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
		__builtin_amdgcn_wave_barrier();
		flagged = 0;
	};

	const uint32_t batch_points = FMA_WAVES * WAVE;
	const uint32_t batches = (n + batch_points - 1) / batch_points;
	for (uint32_t batch = blockIdx.x; batch < batches; batch += gridDim.x) {
		const uint32_t pt = batch * batch_points + threadIdx.x;
		const bool valid = pt < n;
		float x[DP];
		float x2 = 0.0f;
		if (LD == KMX_AOS && vec4) {
			/* rows of whole, aligned 16-byte pieces */
#pragma unroll
			for (int q = 0; q < DP; q += 4) {
				f32x4 v = { 0.0f, 0.0f, 0.0f, 0.0f };
				if (valid && (uint32_t)q < dim) v = *(const f32x4*)(data + (size_t)pt * stride + q);
				x[q] = v.x; x[q + 1] = v.y; x[q + 2] = v.z; x[q + 3] = v.w;
			}
		}
		else {
#pragma unroll
			for (int q = 0; q < DP; ++q) x[q] = (valid && (uint32_t)q < dim) ? data[elem<LD>(stride, pt, q)] : 0.0f;
		}
		float along = 0.0f; /* (x - m) . m */
#pragma unroll
		for (int q = 0; q < DP; ++q) {
			const float m = frame[q];
			x[q] -= m;
			x2 += x[q] * x[q];
			along += x[q] * m;
		}
		float m1 = __builtin_inff(), m2 = __builtin_inff();
		uint32_t best = 0;
		for (uint32_t chunk = 0; chunk < (SCALAR ? 1u : chunks); ++chunk) {
			const uint32_t row0 = chunk * chunk_rows;
			const uint32_t rows = min(chunk_rows, kp - row0);
			if (!resident) {
				__syncthreads();
				stage(row0, rows);
				__syncthreads();
			}
			const uint32_t scan_rows = SCALAR ? k : rows; /* the scalar variant skips the padding rows */
#pragma unroll 4
			for (uint32_t r = 0; r < scan_rows; ++r) {
				/* uniform address: every lane reads the same words */
				const float* row = SCALAR ? packed + packed_row(r, RS) : lds + packed_row(r, RS);
				float a = SCALAR ? norms[norm_at(r)] : lds_norms[norm_at(r)];
#pragma unroll
				for (int q = 0; q < DP; q += 4) {
					const f32x4 c = *(const f32x4*)(row + q);
					a = __builtin_fmaf(c.x, x[q], a);
					a = __builtin_fmaf(c.y, x[q + 1], a);
					a = __builtin_fmaf(c.z, x[q + 2], a);
					a = __builtin_fmaf(c.w, x[q + 3], a);
				}
				m2 = __builtin_amdgcn_fmed3f(m1, m2, a);
				const bool lt = a < m1;
				best = lt ? row0 + r : best;
				m1 = lt ? a : m1;
			}
		}
		const float tau = kd * (x2 + c2max);
		const bool decided = (m2 - m1 > tau) && (x2 + c2max > 1e-30f);
		if (valid) assignment[pt] = best < k ? best : 0u;
		const bool flag = valid && !decided;
		const unsigned long long mask = __ballot(flag);
		if (mask) {
			const uint32_t add = (uint32_t)__builtin_popcountll(mask);
			if (flagged + add > FLAG_CAP) flush_flags();
			if (flag) {
				const uint32_t at = 2 * (flagged + __builtin_popcountll(mask & ((1ull << lane) - 1ull)));
				flag_list[wave][at] = pt;
				/* the exact pass evaluates in the frame of the data (certificate.h) */
				flag_list[wave][at + 1] = kd_unmoved > 0.0f
					? screening_threshold(cert_unmoved_threshold(m1, tau, x2, along, c2max, frame_m2, frame_norm, kd_unmoved), 0.0f)
					: screening_threshold(m1, tau);
			}
			flagged += add;
		}
	}
	if (flagged) flush_flags();
}

static uint32_t fma_dp(uint32_t dim)
{
	for (uint32_t o : { 4u, 8u, 16u, 24u, 32u, 48u, 64u })
		if (dim <= o) return o;
	return 0;
}

/* centroid blocks up to this size are read through the scalar cache instead of LDS */
constexpr uint32_t SCALAR_BLOCK_BYTES = 8 * 1024;

static bool scalar_block(uint32_t dp, uint32_t kp)
{
	return (size_t)(kp / TILE) * (tile_floats(dp + ROW_PAD) + NORM_TILE) * 4 <= SCALAR_BLOCK_BYTES;
}

bool lds_fma_reads_through_scalar_cache(const AssignArgs& a)
{
	const uint32_t dp = fma_dp(a.dim);
	return dp != 0 && scalar_block(dp, round_up(a.k, TILE));
}

bool lds_fma_supports(const AssignArgs& a, const DeviceInfo& dev)
{
	const uint32_t dp = fma_dp(a.dim);
	if (dp == 0) return false;
	return (size_t)(tile_floats(dp + ROW_PAD) + NORM_TILE) * 4 + 8192 <= dev.lds_bytes;
}

template <int DP>
static int launch_fma_dp(const AssignArgs& a, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev, uint32_t kp, float kd)
{
	constexpr uint32_t RS = DP + ROW_PAD;
	uint32_t budget = exec->shared_mem_bytes ? std::min(exec->shared_mem_bytes, dev.lds_bytes) : dev.lds_bytes;
	budget = std::min<uint32_t>(budget, 64 * 1024); /* leave room for several work-groups per CU */
	const uint32_t static_bytes = (2 * FLAG_CAP * FMA_WAVES + 64) * 4;
	const uint32_t tile_bytes = (tile_floats(RS) + NORM_TILE) * 4;
	const bool scalar = scalar_block(DP, kp);
	if (!scalar && budget < static_bytes + tile_bytes) return fail(KMX_ERR_UNSUPPORTED, "assign (LDS/FMA): LDS budget of %u bytes is too small", budget);
	const uint32_t chunk_rows = scalar ? kp : std::min<uint32_t>(kp, (budget - static_bytes) / tile_bytes * TILE);
	const uint32_t lds_bytes = scalar ? 0 : chunk_rows / TILE * tile_bytes;
	const uint32_t batches = (a.n + FMA_WAVES * WAVE - 1) / (FMA_WAVES * WAVE);
	const uint32_t per_cu = std::max<uint32_t>(1, std::min<uint32_t>(8, dev.lds_bytes / (lds_bytes + static_bytes)));
	const uint32_t grid = std::min(batches, dev.compute_units * per_cu);
	exec->block_count = grid;
	void (*kernel)(const float*, size_t, const float*, const float*, uint32_t*, uint32_t*, uint32_t*,
	               uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, float, uint32_t, float) = nullptr;
	const uint32_t vec4 = (a.layout == KMX_AOS && a.dim % 4 == 0 && a.stride % 4 == 0 && ((uintptr_t)a.data % 16) == 0) ? 1u : 0u;
	if (a.layout == KMX_AOS) kernel = scalar ? assign_lds_fma_kernel<DP, KMX_AOS, true> : assign_lds_fma_kernel<DP, KMX_AOS, false>;
	else kernel = scalar ? assign_lds_fma_kernel<DP, KMX_SOA, true> : assign_lds_fma_kernel<DP, KMX_SOA, false>;
	int rc = profile_begin(0);
	if (rc) return rc;
	KMX_LAUNCH_KERNEL(kernel, dim3(grid), dim3(FMA_WAVES * WAVE), lds_bytes, stream(),
	                   a.data, a.stride, ws->packed_means, ws->norms, a.assignment, ws->queue, ws->counters, a.dim, a.k, kp, a.n, chunk_rows, kd, vec4, a.unmoved_thresholds ? cert_kd_unmoved(a.dim) : 0.0f);
	KMX_LAUNCH_CHECK("assign_lds_fma_kernel");
	return profile_end(0);
}

int launch_assign_lds_fma(const AssignArgs& args, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev)
{
	AssignArgs a = args;
	/* the frame moves as in the fp32 MFMA sweep (launch_assign_mfma) */
	a.shift_rows = !a.ranking_only;
	a.unmoved_thresholds = a.shift_rows;
	const uint32_t dp = fma_dp(a.dim);
	const uint32_t kp = round_up(a.k, TILE);
	int rc = launch_pack_means(a, ws, dp, kp, a.shift_rows ? FRAME_MOVED : FRAME_KEPT);
	if (rc) return rc;
	const float kd = cert_kd_fma(a.dim) + (a.shift_rows ? 8.0f * CERT_UNIT : 0.0f) + a.kd_extra;
	switch (dp) {
	case 4: rc = launch_fma_dp<4>(a, exec, ws, dev, kp, kd); break;
	case 8: rc = launch_fma_dp<8>(a, exec, ws, dev, kp, kd); break;
	case 16: rc = launch_fma_dp<16>(a, exec, ws, dev, kp, kd); break;
	case 24: rc = launch_fma_dp<24>(a, exec, ws, dev, kp, kd); break;
	case 32: rc = launch_fma_dp<32>(a, exec, ws, dev, kp, kd); break;
	case 48: rc = launch_fma_dp<48>(a, exec, ws, dev, kp, kd); break;
	case 64: rc = launch_fma_dp<64>(a, exec, ws, dev, kp, kd); break;
	default: return fail(KMX_ERR_UNSUPPORTED, "assign (LDS/FMA): dim %u is not supported", a.dim);
	}
	if (rc) return rc;
	if (a.ranking_only) return KMX_OK; /* the caller resolves the queued points */
	ws->exact_norms = ws->norms + plain_exact_norms_offset(kp);
	rc = launch_recheck(a, ws, kp);
	ws->exact_norms = nullptr;
	return rc;
}

} // namespace kmx
