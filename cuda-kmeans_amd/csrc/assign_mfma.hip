/*
 * Assignment on the matrix cores: v_mfma_f32_32x32x2_f32 tiles of  a[j][i] = |c_j|^2 - 2 c_j . x_i .
 *
 * For one point the ranking of the centroids by a[j] is the ranking by squared distance
 * (|x|^2 is common to all j), so the argmin needs one fused multiply-add per (point, centroid,
 * dim) instead of the subtract/multiply/add of the direct form, and it is a dense contraction.
 *
 * Exactness. The caller is promised the index the serial scan would return (reference
 * serial.hpp:21-35 with metric_policies.hpp:23-28,40-44). The kernel therefore tracks, per point,
 * the smallest and the second smallest a[j]. Let u = 2^-24 and T_j the real squared distance.
 *   - serial sum s_j:      |s_j - T_j|  <= (d+2) u T_j                      (positive terms)
 *   - a_j as computed:     |a_j - (T_j - |x|^2)| <= (d+2) u' (|c_j|^2 + 2|x||c_j|),  u' = 2u allowed
 *                          for the accumulation order / rounding inside the matrix core
 *   - sqrt can merge two sums that differ by a few ulp, which would hand the win to a lower index
 * Putting these together, if  a_(2) - a_(1) > tau  with  tau = (8 d + 64) 2^-23 (|x|^2 + max_j |c_j|^2)
 * then centroid (1) has the strictly smallest serial distance and is the serial result. Every other
 * point (including all NaN / overflow cases, for which the comparison is false) is appended to the
 * recheck queue and re-evaluated by recheck_kernel with the serial arithmetic.
 *
 * Data flow. pack_means_kernel writes the centroids once per call as rows of -2c padded to DP = 2*DPH
 * floats (+4 floats of row padding, which makes the 128-bit LDS reads of 16 consecutive rows hit 64
 * distinct banks) and the norms |c_j|^2 (+inf for padding rows). A work-group copies the packed block
 * (or, if it does not fit, chunks of it) into LDS, then every wavefront keeps P tiles of 32 points in
 * registers as MFMA B-operands for the whole sweep over the centroids. Tile layout: centroids are the
 * rows (M), points the columns (N), so a lane holds 16 centroids of ONE point and the running
 * (min, second min, argmin) is pure per-lane VALU work; the two half-waves (row groups) merge once at
 * the end. The K dimension is split between the half-waves: lanes 0-31 feed dims [0,DPH), lanes 32-63
 * dims [DPH,2DPH), so both operands are read as contiguous 16-byte pieces of a row.
 */
#include "kmx_internal.h"

#include <algorithm>

namespace kmx {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

constexpr uint32_t TILE = 32;       /* centroids per MFMA tile = points per MFMA tile */
constexpr uint32_t ROW_PAD = 4;     /* floats appended to every packed centroid row   */
constexpr uint32_t MFMA_WAVES = 8;  /* wavefronts per work-group                      */
constexpr uint32_t MFMA_P = 4;      /* point tiles per wavefront                      */

__host__ __device__ constexpr uint32_t round_up(uint32_t v, uint32_t m) { return (v + m - 1) / m * m; }

/* supported per-half dimension counts (= MFMA k-steps per tile) */
static uint32_t pick_dph(uint32_t dim)
{
	const uint32_t need = (dim + 1) / 2;
	const uint32_t options[] = { 2, 4, 8, 12, 16, 24, 32 };
	for (uint32_t o : options)
		if (need <= o) return o;
	return 0;
}

template <int LM>
__global__ void __launch_bounds__(256)
pack_means_kernel(const float* __restrict__ means, size_t stride_means, float* __restrict__ packed, float* __restrict__ norms,
                  float* __restrict__ means_t, uint32_t dim, uint32_t k, uint32_t kp, uint32_t dp, uint32_t* __restrict__ counters)
{
	const uint32_t j = blockIdx.x * blockDim.x + threadIdx.x;
	if (j == 0) counters[0] = 0u; /* the recheck queue of this call starts empty */
	if (j >= kp) return;
	const uint32_t rs = dp + ROW_PAD;
	float c2 = 0.0f;
	for (uint32_t q = 0; q < rs; ++q) {
		float v = (j < k && q < dim) ? means[elem<LM>(stride_means, j, q)] : 0.0f;
		c2 += v * v;
		packed[(size_t)j * rs + q] = -2.0f * v;
		if (q < dim) means_t[(size_t)q * kp + j] = v; /* exact copy for the recheck pass */
	}
	norms[j] = j < k ? c2 : __builtin_inff();
}

template <int DPH, int P, int LD, bool VEC, bool STREAM>
__global__ void __launch_bounds__(MFMA_WAVES * WAVE)
assign_mfma_kernel(const float* __restrict__ data, size_t stride, const float* __restrict__ packed, const float* __restrict__ norms,
                   uint32_t* __restrict__ assignment, uint32_t* __restrict__ queue, uint32_t* __restrict__ counters,
                   uint32_t dim, uint32_t k, uint32_t kp, uint32_t n, uint32_t chunk_rows, float kd)
{
	constexpr uint32_t DP = 2 * DPH;
	constexpr uint32_t RS = DP + ROW_PAD;
	extern __shared__ float lds[];
	__shared__ uint32_t wave_max[MFMA_WAVES];

	const uint32_t lane = threadIdx.x & (WAVE - 1);
	const uint32_t wave = threadIdx.x / WAVE;
	const uint32_t col = lane & 31; /* point within a tile (B column) / centroid row fed to A */
	const uint32_t h = lane >> 5;   /* half-wave: K split and the +4 row group of the result    */

	/* max_j |c_j|^2 (bit pattern maximum: propagates NaN and +inf, which then flag every point) */
	uint32_t cmax = 0;
	for (uint32_t j = threadIdx.x; j < k; j += blockDim.x) cmax = max(cmax, __float_as_uint(norms[j]));
	for (int off = WAVE / 2; off > 0; off >>= 1) cmax = max(cmax, (uint32_t)__shfl_xor((int)cmax, off));
	if (lane == 0) wave_max[wave] = cmax;
	__syncthreads();
	cmax = 0;
	for (uint32_t w = 0; w < MFMA_WAVES; ++w) cmax = max(cmax, wave_max[w]);
	const float c2max = __uint_as_float(cmax);

	float* lds_norms = lds + (size_t)chunk_rows * RS;
	const uint32_t chunks = (kp + chunk_rows - 1) / chunk_rows;

	auto stage = [&](uint32_t row0, uint32_t rows) {
		/* flat 16-byte copy of `rows` packed rows and their norms */
		const f32x4* src = (const f32x4*)(packed + (size_t)row0 * RS);
		f32x4* dst = (f32x4*)lds;
		const uint32_t vecs = rows * RS / 4;
		for (uint32_t i = threadIdx.x; i < vecs; i += blockDim.x) dst[i] = src[i];
		for (uint32_t i = threadIdx.x; i < rows; i += blockDim.x) lds_norms[i] = norms[row0 + i];
	};

	if (!STREAM) {
		stage(0, kp);
		__syncthreads();
	}

	const uint32_t points_per_round = MFMA_WAVES * P * TILE;
	const uint32_t rounds = (n + points_per_round - 1) / points_per_round;

	for (uint32_t round = blockIdx.x; round < rounds; round += gridDim.x) {
		const uint32_t base = (round * MFMA_WAVES + wave) * P * TILE;

		/* ---- points of this wavefront -> registers (MFMA B operands), |x|^2 ---- */
		float b[P][DPH];
		float x2[P];
#pragma unroll
		for (int p = 0; p < P; ++p) {
			const uint32_t pt = base + p * TILE + col;
			const bool valid = pt < n;
			if (LD == KMX_AOS) {
				const float* src = data + (size_t)pt * stride + h * DPH;
				if (VEC && DPH % 4 == 0) {
#pragma unroll
					for (int s = 0; s < DPH; s += 4) {
						f32x4 v = { 0.0f, 0.0f, 0.0f, 0.0f };
						if (valid && h * DPH + s < dim) v = *(const f32x4*)(src + s);
						b[p][s] = v.x; b[p][s + 1] = v.y; b[p][s + 2] = v.z; b[p][s + 3] = v.w;
					}
				}
				else if (VEC) {
#pragma unroll
					for (int s = 0; s < DPH; s += 2) {
						f32x2 v = { 0.0f, 0.0f };
						if (valid && h * DPH + s < dim) v = *(const f32x2*)(src + s);
						b[p][s] = v.x; b[p][s + 1] = v.y;
					}
				}
				else {
#pragma unroll
					for (int s = 0; s < DPH; ++s) b[p][s] = (valid && h * DPH + s < dim) ? src[s] : 0.0f;
				}
			}
			else {
#pragma unroll
				for (int s = 0; s < DPH; ++s)
					b[p][s] = (valid && h * DPH + s < dim) ? data[(size_t)(h * DPH + s) * stride + pt] : 0.0f;
			}
			float part = 0.0f;
#pragma unroll
			for (int s = 0; s < DPH; ++s) part += b[p][s] * b[p][s];
			x2[p] = part + __shfl_xor(part, 32);
		}

		float m1[P], m2[P];
		uint32_t best[P];
#pragma unroll
		for (int p = 0; p < P; ++p) {
			m1[p] = __builtin_inff();
			m2[p] = __builtin_inff();
			best[p] = 0;
		}

		/* ---- sweep over the centroids ---- */
		for (uint32_t chunk = 0; chunk < chunks; ++chunk) {
			const uint32_t row0 = chunk * chunk_rows;
			const uint32_t rows = min(chunk_rows, kp - row0);
			if (STREAM) {
				__syncthreads(); /* everyone is done with the previous chunk */
				stage(row0, rows);
				__syncthreads();
			}
			const uint32_t tiles = rows / TILE;
			for (uint32_t tile = 0; tile < tiles; ++tile) {
				/* A operand: this lane's centroid row, its half of the dimensions */
				const float* arow = lds + (size_t)(tile * TILE + col) * RS + h * DPH;
				float a[DPH];
				if (DPH % 4 == 0) {
#pragma unroll
					for (int s = 0; s < DPH; s += 4) {
						f32x4 v = *(const f32x4*)(arow + s);
						a[s] = v.x; a[s + 1] = v.y; a[s + 2] = v.z; a[s + 3] = v.w;
					}
				}
				else {
#pragma unroll
					for (int s = 0; s < DPH; s += 2) {
						f32x2 v = *(const f32x2*)(arow + s);
						a[s] = v.x; a[s + 1] = v.y;
					}
				}
				/* C operand: |c|^2 of the 16 rows this lane receives: rows 8g + 4h + (0..3), g = 0..3 */
				f32x16 cinit;
#pragma unroll
				for (int g = 0; g < 4; ++g) {
					f32x4 v = *(const f32x4*)(lds_norms + tile * TILE + 8 * g + 4 * h);
					cinit[4 * g] = v.x; cinit[4 * g + 1] = v.y; cinit[4 * g + 2] = v.z; cinit[4 * g + 3] = v.w;
				}
				const uint32_t tile_row = row0 + tile * TILE;
#pragma unroll
				for (int p = 0; p < P; ++p) {
					f32x16 acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[0], b[p][0], cinit, 0, 0, 0);
#pragma unroll
					for (int s = 1; s < DPH; ++s) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s], b[p][s], acc, 0, 0, 0);
#pragma unroll
					for (int r = 0; r < 16; ++r) {
						const float v = acc[r];
						const uint32_t cand = tile_row + 8 * (r / 4) + (r % 4); /* + 4h, added after the sweep */
						m2[p] = __builtin_amdgcn_fmed3f(m1[p], m2[p], v);
						best[p] = v < m1[p] ? cand : best[p];
						m1[p] = fminf(m1[p], v);
					}
				}
			}
		}

		/* ---- merge the two half-waves, decide, write ---- */
#pragma unroll
		for (int p = 0; p < P; ++p) {
			uint32_t idx = best[p] + 4 * h;
			const float o1 = __shfl_xor(m1[p], 32);
			const float o2 = __shfl_xor(m2[p], 32);
			const uint32_t oi = (uint32_t)__shfl_xor((int)idx, 32);
			const float second = fminf(fmaxf(m1[p], o1), fminf(m2[p], o2));
			if (o1 < m1[p]) idx = oi;
			const float first = fminf(m1[p], o1);
			const float tau = kd * (x2[p] + c2max);
			const uint32_t pt = base + p * TILE + col;
			const bool mine = h == 0 && pt < n;
			const bool decided = (second - first > tau) && (x2[p] + c2max > 1e-30f);
			if (mine) assignment[pt] = idx < k ? idx : 0u;
			const bool flag = mine && !decided;
			const unsigned long long mask = __ballot(flag);
			if (mask) {
				uint32_t slot = 0;
				if (lane == (uint32_t)__builtin_ctzll(mask)) slot = atomicAdd(&counters[0], (uint32_t)__builtin_popcountll(mask));
				slot = (uint32_t)__shfl((int)slot, __builtin_ctzll(mask));
				if (flag) queue[slot + __builtin_popcountll(mask & ((1ull << lane) - 1ull))] = pt;
			}
		}
	}
}

bool mfma_supports(const AssignArgs& a, const DeviceInfo& dev)
{
	const uint32_t dph = pick_dph(a.dim);
	if (dph == 0) return false;
	/* at least one tile of packed rows (+ norms) must fit the LDS of a work-group */
	return (size_t)TILE * (2 * dph + ROW_PAD + 1) * 4 <= dev.lds_bytes;
}

template <int DPH, int LD, bool VEC>
static int launch_mfma_t(const AssignArgs& a, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev, uint32_t kp, float kd)
{
	constexpr uint32_t RS = 2 * DPH + ROW_PAD;
	uint32_t budget = exec->shared_mem_bytes ? std::min(exec->shared_mem_bytes, dev.lds_bytes) : dev.lds_bytes;
	budget -= 256; /* static LDS of the kernel */
	const uint32_t row_bytes = (RS + 1) * 4;
	uint32_t chunk_rows = std::min<uint32_t>(kp, budget / row_bytes / TILE * TILE);
	if (chunk_rows == 0) return fail(KMX_ERR_UNSUPPORTED, "assign (MFMA): LDS budget of %u bytes is too small", budget);
	const bool stream_mode = chunk_rows < kp;
	const uint32_t lds_bytes = chunk_rows * row_bytes;
	const uint32_t points_per_round = MFMA_WAVES * MFMA_P * TILE;
	const uint32_t rounds = (a.n + points_per_round - 1) / points_per_round;
	const uint32_t grid = std::min(rounds, dev.compute_units);
	exec->block_count = grid;

	int rc = KMX_OK;
	if (stream_mode) {
		auto kernel = assign_mfma_kernel<DPH, MFMA_P, LD, VEC, true>;
		KMX_HIP(hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
		if ((rc = profile_begin(0))) return rc;
		hipLaunchKernelGGL(kernel, dim3(grid), dim3(MFMA_WAVES * WAVE), lds_bytes, stream(),
		                   a.data, a.stride, ws->packed_means, ws->norms, a.assignment, ws->queue, ws->counters,
		                   a.dim, a.k, kp, a.n, chunk_rows, kd);
	}
	else {
		auto kernel = assign_mfma_kernel<DPH, MFMA_P, LD, VEC, false>;
		KMX_HIP(hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
		if ((rc = profile_begin(0))) return rc;
		hipLaunchKernelGGL(kernel, dim3(grid), dim3(MFMA_WAVES * WAVE), lds_bytes, stream(),
		                   a.data, a.stride, ws->packed_means, ws->norms, a.assignment, ws->queue, ws->counters,
		                   a.dim, a.k, kp, a.n, chunk_rows, kd);
	}
	KMX_LAUNCH_CHECK("assign_mfma_kernel");
	return profile_end(0);
}

template <int DPH>
static int launch_mfma_dph(const AssignArgs& a, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev, uint32_t kp, float kd)
{
	if (a.layout == KMX_SOA) return launch_mfma_t<DPH, KMX_SOA, false>(a, exec, ws, dev, kp, kd);
	const uint32_t vec = DPH % 4 == 0 ? 4 : 2;
	const bool aligned = a.dim % vec == 0 && a.stride % vec == 0 && ((uintptr_t)a.data % (vec * 4)) == 0;
	if (aligned) return launch_mfma_t<DPH, KMX_AOS, true>(a, exec, ws, dev, kp, kd);
	return launch_mfma_t<DPH, KMX_AOS, false>(a, exec, ws, dev, kp, kd);
}

int launch_assign_mfma(const AssignArgs& a, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev)
{
	const uint32_t dph = pick_dph(a.dim);
	const uint32_t dp = 2 * dph;
	const uint32_t kp = round_up(a.k, TILE);
	int rc = reserve_packed(ws, (size_t)kp * (dp + ROW_PAD), kp, (size_t)kp * a.dim);
	if (rc) return rc;
	rc = reserve_queue(ws, a.n);
	if (rc) return rc;

	const uint32_t pack_blocks = (kp + 255) / 256;
	if (a.layout_means == KMX_AOS)
		hipLaunchKernelGGL((pack_means_kernel<KMX_AOS>), dim3(pack_blocks), dim3(256), 0, stream(),
		                   a.means, a.stride_means, ws->packed_means, ws->norms, ws->means_t, a.dim, a.k, kp, dp, ws->counters);
	else
		hipLaunchKernelGGL((pack_means_kernel<KMX_SOA>), dim3(pack_blocks), dim3(256), 0, stream(),
		                   a.means, a.stride_means, ws->packed_means, ws->norms, ws->means_t, a.dim, a.k, kp, dp, ws->counters);
	KMX_LAUNCH_CHECK("pack_means_kernel");

	/* tau = kd (|x|^2 + max|c|^2), kd = (8 d + 64) 2^-23 (see the bound at the top of the file) */
	const float kd = (8.0f * (float)a.dim + 64.0f) * 1.1920929e-07f;
	switch (dph) {
	case 2: rc = launch_mfma_dph<2>(a, exec, ws, dev, kp, kd); break;
	case 4: rc = launch_mfma_dph<4>(a, exec, ws, dev, kp, kd); break;
	case 8: rc = launch_mfma_dph<8>(a, exec, ws, dev, kp, kd); break;
	case 12: rc = launch_mfma_dph<12>(a, exec, ws, dev, kp, kd); break;
	case 16: rc = launch_mfma_dph<16>(a, exec, ws, dev, kp, kd); break;
	case 24: rc = launch_mfma_dph<24>(a, exec, ws, dev, kp, kd); break;
	case 32: rc = launch_mfma_dph<32>(a, exec, ws, dev, kp, kd); break;
	default: return fail(KMX_ERR_UNSUPPORTED, "assign (MFMA): dim %u is not supported", a.dim);
	}
	if (rc) return rc;
	return launch_recheck(a, ws, kp);
}

} // namespace kmx
