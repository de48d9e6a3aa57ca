/*
 * Assignment on the matrix cores: v_mfma_f32_32x32x2_f32 tiles of  a[j][i] = |c_j|^2 - 2 c_j . x_i .
 *
 * For one point the ranking of the centroids by a[j] is the ranking by squared distance
 * (|x|^2 is common to all j), so the argmin needs one fused multiply-add per (point, centroid,
 * dim) instead of the subtract/multiply/add of the direct form, and it is a dense contraction.
 *
 * Exactness. The caller is promised the index the serial scan would return (reference
 * serial.hpp:21-35 with metric_policies.hpp:23-28,40-44). The kernel therefore establishes, per point,
 * the smallest a[j] and a lower bound of every other a[j]. Let u = 2^-24 and T_j the real squared distance.
 *   - serial sum s_j:      |s_j - T_j|  <= (d+2) u T_j                      (positive terms)
 *   - a_j as computed:     |a_j - (T_j - |x|^2)| <= (d+2) u' (|c_j|^2 + 2|x||c_j|),  u' = 2u allowed
 *                          for the accumulation order / rounding inside the matrix core
 *   - sqrt can merge two sums that differ by a few ulp, which would hand the win to a lower index
 * Putting these together, if  a_(2) - a_(1) > tau  with  tau = (8 d + 24) 2^-23 (|x|^2 + max_j |c_j|^2)
 * then centroid (1) has the strictly smallest serial distance and is the serial result. Every other
 * point (including all NaN / overflow cases, for which the comparison is false) is appended to the
 * recheck queue and re-evaluated by the recheck kernels with the serial arithmetic.
 *
 * Data flow. pack_means_kernel writes the centroids once per call as rows of -2c padded to DP = 2*DPH
 * floats (+4 floats of row padding, which makes the 128-bit LDS reads of 16 consecutive rows hit 64
 * distinct banks; +4 floats after every tile of 32 rows, which spreads equal rows of different tiles
 * over the banks) and the norms |c_j|^2 (+inf for padding rows; 36 floats per tile for the same reason).
 * A work-group copies the packed block (or, if it does not fit, chunks of it) into LDS, then every
 * wavefront keeps P tiles of 32 points in registers as MFMA B-operands for the whole sweep over the
 * centroids, while the points of its next sweep are already being loaded. Tile layout: centroids are the
 * rows (M), points the columns (N), so a lane holds 16 centroids of ONE point and the running minimum is
 * pure per-lane VALU work; the two half-waves (row groups) merge once at the end. The K dimension is
 * split between the half-waves: lanes 0-31 feed dims [0,DPH), lanes 32-63 dims [DPH,2DPH), so both
 * operands are read as contiguous 16-byte pieces of a row.
 *
 * What the counters said (gfx950): fp32 MFMA and VALU time ADD UP -- VALU work is not hidden behind
 * v_mfma_f32_32x32x2_f32, whatever the occupancy -- and VALU operations cost less in long runs than
 * sprinkled between MFMAs. Hence (1) the per-result work is kept minimal: with many tiles only the
 * minimum of a lane's 16 results is tracked per tile (16 operations instead of 66) and the winning row
 * is recomputed once per sweep; (2) sched_group_barrier groups the MFMAs of a tile and the tracking of
 * the previous tile into few large runs.
 */
#include "certificate.h"
#include "assign_mfma_impl.h"

namespace kmx {

/* supported per-half dimension counts (= MFMA k-steps per tile) */
static uint32_t pick_dph(uint32_t dim)
{
	const uint32_t need = (dim + 1) / 2;
	const uint32_t options[] = { 2, 4, 8, 12, 16, 24, 32, 64, 128 };
	for (uint32_t o : options)
		if (need <= o) return o;
	return 0;
}

/*
 * One wavefront per (padded) centroid row: packed row of -2c (coalesced reads for AoS centroids, coalesced
 * writes), |c|^2 by a wavefront reduction, and the exact transposed copy for the recheck pass.
 */
template <int LM>
__global__ void __launch_bounds__(256)
pack_means_kernel(const float* __restrict__ means, size_t stride_means, float* __restrict__ packed, float* __restrict__ norms,
                  float* __restrict__ means_t, uint32_t dim, uint32_t k, uint32_t kp, uint32_t dp, uint32_t moved, uint32_t* __restrict__ counters)
{
	const uint32_t lane = threadIdx.x & (WAVE - 1);
	const uint32_t j = (blockIdx.x * blockDim.x + threadIdx.x) / WAVE;
	if (blockIdx.x == 0 && threadIdx.x == 0) counters[0] = 0u; /* the recheck queue of this call starts empty */
	/* the frame of the sweep (zeros unless `moved`): the rows are those of c - m, with their norms; the exact pass gets
	 * the centroids and their norms as given */
	__shared__ float frame[FRAME_DIMS];
	sweep_frame<LM>(means, stride_means, dim, k, dp, moved, frame, norms + plain_frame_offset(kp));
	if (j >= kp) return;
	const uint32_t rs = dp + ROW_PAD;
	float* row = packed + packed_row(j, rs);
	const uint32_t row_floats = rs + (j % TILE == TILE - 1 ? TILE_PAD : 0); /* the tile padding follows its last row */
	float c2 = 0.0f, exact2 = 0.0f;
	for (uint32_t q = lane; q < row_floats; q += WAVE) {
		const float exact = (j < k && q < dim) ? means[elem<LM>(stride_means, j, q)] : 0.0f;
		const float v = (j < k && q < dim) ? exact - frame[q] : 0.0f;
		c2 += v * v;
		exact2 += exact * exact;
		row[q] = -2.0f * v;
		if (q < dim) means_t[(size_t)q * kp + j] = exact; /* exact copy for the recheck pass */
	}
	for (int off = WAVE / 2; off > 0; off >>= 1) {
		c2 += __shfl_xor(c2, off);
		exact2 += __shfl_xor(exact2, off);
	}
	if (lane == 0) {
		norms[norm_at(j)] = j < k ? c2 : __builtin_inff();
		norms[plain_exact_norms_offset(kp) + norm_at(j)] = j < k ? exact2 : __builtin_inff();
	}
	if (lane < NORM_TILE - TILE && j % TILE == 0) {
		norms[(j / TILE) * NORM_TILE + TILE + lane] = __builtin_inff();
		norms[plain_exact_norms_offset(kp) + (j / TILE) * NORM_TILE + TILE + lane] = __builtin_inff();
	}
}

bool mfma_supports(const AssignArgs& a, const DeviceInfo& dev)
{
	const uint32_t dph = pick_dph(a.dim);
	if (dph == 0) return false;
	/* at least one tile of packed rows (+ norms) must fit the LDS of a work-group */
	return (size_t)(tile_floats(2 * dph + ROW_PAD) + NORM_TILE) * 4 + 8192 <= dev.lds_bytes;
}

/* one launcher per supported row width, each compiled in its own translation unit (assign_mfma_inst.hip) */
#define KMX_DECLARE_MFMA_LAUNCHER(W) \
	int launch_mfma_##W(const AssignArgs& a, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev, uint32_t kp, float kd);
KMX_DECLARE_MFMA_LAUNCHER(2) KMX_DECLARE_MFMA_LAUNCHER(4) KMX_DECLARE_MFMA_LAUNCHER(8) KMX_DECLARE_MFMA_LAUNCHER(12)
KMX_DECLARE_MFMA_LAUNCHER(16) KMX_DECLARE_MFMA_LAUNCHER(24) KMX_DECLARE_MFMA_LAUNCHER(32) KMX_DECLARE_MFMA_LAUNCHER(64)
KMX_DECLARE_MFMA_LAUNCHER(128)

/* packs the centroids of this call into the work space (rows of dp floats, kp rows) and empties the recheck queue */
int launch_pack_means(const AssignArgs& a, Workspace* ws, uint32_t dp, uint32_t kp, uint32_t moved)
{
	int rc = reserve_packed(ws, (size_t)(kp / TILE) * tile_floats(dp + ROW_PAD), plain_norms_floats(kp), (size_t)kp * a.dim);
	if (rc) return rc;
	rc = reserve_queue(ws, 2 * (size_t)a.n); /* (point, threshold) pairs */
	if (rc) return rc;
	const uint32_t pack_blocks = (kp * WAVE + 255) / 256;
	if (a.layout_means == KMX_AOS)
		KMX_LAUNCH_KERNEL((pack_means_kernel<KMX_AOS>), dim3(pack_blocks), dim3(256), 0, stream(),
		                   a.means, a.stride_means, ws->packed_means, ws->norms, ws->means_t, a.dim, a.k, kp, dp, moved, ws->counters);
	else
		KMX_LAUNCH_KERNEL((pack_means_kernel<KMX_SOA>), dim3(pack_blocks), dim3(256), 0, stream(),
		                   a.means, a.stride_means, ws->packed_means, ws->norms, ws->means_t, a.dim, a.k, kp, dp, moved, ws->counters);
	KMX_LAUNCH_CHECK("pack_means_kernel");
	return KMX_OK;
}

int launch_assign_mfma(const AssignArgs& args, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev)
{
	AssignArgs a = args;
	/* The sweep works in a frame moved to the middle of the centroids (sweep_frame), so that tau scales with the spread of
	 * the data and not with its distance from the origin; the thresholds go to the exact pass in the frame of the data.
	 * (Not for the double path: the float copies of its points are rounded relative to the origin anyway.) */
	a.shift_rows = !a.ranking_only;
	a.unmoved_thresholds = a.shift_rows;
	const uint32_t dph = pick_dph(a.dim);
	const uint32_t dp = 2 * dph;
	const uint32_t kp = round_up(a.k, TILE);
	int rc = launch_pack_means(a, ws, dp, kp, a.shift_rows ? FRAME_MOVED : FRAME_KEPT);
	if (rc) return rc;

	/* tau = kd (|x|^2 + max|c|^2), kd = (8 d + 24) 2^-23 (see the bound at the top of the file), 8 * 2^-23 more for the
	 * roundings of x - m and c - m */
	const float kd = cert_kd_fp32(a.dim) + (a.shift_rows ? 8.0f * CERT_UNIT : 0.0f) + a.kd_extra;
	switch (dph) {
	case 2: rc = launch_mfma_2(a, exec, ws, dev, kp, kd); break;
	case 4: rc = launch_mfma_4(a, exec, ws, dev, kp, kd); break;
	case 8: rc = launch_mfma_8(a, exec, ws, dev, kp, kd); break;
	case 12: rc = launch_mfma_12(a, exec, ws, dev, kp, kd); break;
	case 16: rc = launch_mfma_16(a, exec, ws, dev, kp, kd); break;
	case 24: rc = launch_mfma_24(a, exec, ws, dev, kp, kd); break;
	case 32: rc = launch_mfma_32(a, exec, ws, dev, kp, kd); break;
	case 64: rc = launch_mfma_64(a, exec, ws, dev, kp, kd); break;
	case 128: rc = launch_mfma_128(a, exec, ws, dev, kp, kd); break;
	default: return fail(KMX_ERR_UNSUPPORTED, "assign (MFMA): dim %u is not supported", a.dim);
	}
	if (rc) return rc;
	if (a.ranking_only) return KMX_OK; /* the caller resolves the queued points */
	ws->exact_norms = ws->norms + plain_exact_norms_offset(kp);
	rc = launch_recheck(a, ws, kp);
	ws->exact_norms = nullptr;
	return rc;
}

} // namespace kmx
