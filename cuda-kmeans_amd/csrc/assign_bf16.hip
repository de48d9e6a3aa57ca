/*
 * Assignment on the matrix cores at bf16 rate with fp32-level accuracy: a[j][i] = |c_j|^2 - 2 c_j . x_i as
 * v_mfma_f32_32x32x16_bf16 tiles over SPLIT operands.
 *
 * Every fp32 value v is written as hi + mid + rest with hi = bf16(v), mid = bf16(v - hi) (round to nearest
 * even), |mid| <= 2^-8 |v|, |rest| <= 2^-17 |v|. The contraction keeps the three largest of the four hi/mid products,
 *      c'.x  ~  sum_i  c'hi_i x_mid_i + c'mid_i x_hi_i + c'hi_i x_hi_i ,       c' = -2c,
 * each product exact in fp32 (8 x 8 significant bits), accumulated in fp32 by the matrix core. One block of
 * 16 dimensions costs 3 MFMAs of 8 passes where the fp32 kernel (v_mfma_f32_32x32x2_f32) spends 8 MFMAs of
 * 16 passes: 24 against 128 matrix-core passes per tile and block.
 *
 * Exactness. As in the fp32 kernel the result promised to the caller is the index the serial scan returns
 * (reference serial.hpp:21-35, metric_policies.hpp:23-28,40-44), established by the same certification:
 * a point whose two smallest a[j] are further apart than tau is decided, every other point goes to the
 * recheck queue and is re-evaluated with the serial arithmetic. Only tau differs: it has to cover the products
 * the split drops. certificate.h derives it: tau = kd S + 2.06 * (bound of the dropped products), the bound
 * evaluated from the norms of the parts actually dropped -- max_j |c'mid_j| and max_j |c'rest_j|, which the packing
 * kernel below writes behind the norms, and |xmid| (or |xrest|) of the point -- not from their worst case.
 * The refinement (winning row inside the winning tile) re-evaluates rows with v_dot2c_f32_bf16 on the same
 * three products, so the same bound covers it; the sweep of rows of 17 to 48 dimensions with resident centroids keeps the
 * 16 results of the leading tile in registers instead (the snapshot, assign_bf16_impl.h) and has nothing to re-evaluate.
 *
 * Rows of at most 4 dimensions (PACKED): a block of 16 MFMA slots holds ALL FOUR hi/mid products of every dimension
 * (4 d <= 16), so a tile costs one MFMA instead of three and nothing of (hi + mid)(hi + mid) is dropped; only the
 * remainders of the split are (certificate.h, packed form). With 128 centroids or more these rows are swept in a frame moved
 * to the mean of the centroids (pack_means_bf16_kernel below subtracts it from the centroids, the sweep and the screen of the
 * exact pass from the points): tau scales with |x|^2 + max |c|^2, which the frame makes the spread of the data instead of its
 * distance from the origin.
 *
 * Data flow, tiling, tracking, flag buffering and the recheck hand-over are those of the fp32 kernel
 * (assign_mfma.hip); the packed centroid row holds hi and mid parts of -2c, 4 bytes per dimension as before.
 */
#include "assign_bf16_impl.h"

namespace kmx {

/* supported blocks of 16 dimensions per row */
static uint32_t pick_kb(uint32_t dim)
{
	const uint32_t need = (dim + KBLOCK - 1) / KBLOCK;
	const uint32_t options[] = { 1, 2, 3, 4, 8, 16 };
	for (uint32_t o : options)
		if (need <= o) return o;
	return 0;
}

/*
 * One wavefront per (padded) centroid row: hi/mid parts of -2c in the unit order tile_step_bf16 reads,
 * |c|^2 by a wavefront reduction, and the exact transposed copy for the recheck pass.
 */
template <int LM>
__global__ void __launch_bounds__(256)
pack_means_bf16_kernel(const float* __restrict__ means, size_t stride_means, float* __restrict__ packed, float* __restrict__ norms,
                       float* __restrict__ means_t, uint32_t dim, uint32_t k, uint32_t kp, uint32_t dp, uint32_t packed_slots,
                       uint32_t* __restrict__ counters)
{
	const uint32_t lane = threadIdx.x & (WAVE - 1);
	const uint32_t j = (blockIdx.x * blockDim.x + threadIdx.x) / WAVE;
	if (blockIdx.x == 0 && threadIdx.x == 0) {
		counters[0] = 0u; /* the recheck queue of this call starts empty */
		counters[LISTED_COUNTER] = 0u; /* and so does the list of points the first level of a two-level sweep passes on */
	}
	/* packed rows: the frame of the sweep, the mean of the first centroids (up to 256 of them, one per lane; the finite
	 * coordinates; any vector would do, this one is near the middle of the data). Every work-group computes it, in the same order. */
	__shared__ float frame_parts[4][4];
	float frame[4] = { 0.0f, 0.0f, 0.0f, 0.0f };
	if ((packed_slots & 3u) == 3u) {
		const uint32_t sample = min(k, 256u);
		float sum[4] = { 0.0f, 0.0f, 0.0f, 0.0f };
		for (uint32_t r = threadIdx.x; r < sample; r += 256) {
#pragma unroll
			for (int q = 0; q < 4; ++q) {
				const float v = (uint32_t)q < dim ? means[elem<LM>(stride_means, r, q)] : 0.0f;
				sum[q] += __builtin_fabsf(v) < __builtin_inff() ? v : 0.0f;
			}
		}
		for (int off = WAVE / 2; off > 0; off >>= 1)
			for (int q = 0; q < 4; ++q) sum[q] += __shfl_xor(sum[q], off);
		if (lane == 0)
			for (int q = 0; q < 4; ++q) frame_parts[threadIdx.x / WAVE][q] = sum[q];
		__syncthreads();
		for (int q = 0; q < 4; ++q) frame[q] = (frame_parts[0][q] + frame_parts[1][q] + frame_parts[2][q] + frame_parts[3][q]) / (float)sample;
	}
	if ((packed_slots & 1u) && blockIdx.x == 0) {
#pragma unroll
		for (int q = 0; q < 4; ++q)
			if (threadIdx.x == (uint32_t)q) norms[frame_offset(kp) + q] = frame[q];
	}
	/* unpacked rows: the same for rows of up to FRAME_DIMS dimensions (sweep_frame) */
	__shared__ float wide_frame[FRAME_DIMS];
	if (!(packed_slots & 1u)) sweep_frame<LM>(means, stride_means, dim, k, dp, (packed_slots & 2u) ? FRAME_MOVED : FRAME_KEPT, wide_frame, norms + frame_offset(kp));
	if (j >= kp) return;
	const bool packed_form = (packed_slots & 1u) != 0;
	const uint32_t rs = packed_form ? row_floats<1, true>() : dp + ROW_PAD;
	float* row = packed + packed_row(j, rs);
	__bf16* parts = (__bf16*)row;
	float c2 = 0.0f, mid2 = 0.0f, rest2 = 0.0f; /* |c|^2 (of the moved centroid) and, for the certificate, sum_i c'mid_i^2, sum_i c'rest_i^2 */
	float exact2 = 0.0f; /* unpacked rows: |c|^2 of the centroid as given */
	if (packed_form) {
		/* rows of at most 4 dimensions: slots 0..3 = hi, 4..7 = mid, 8..11 = hi, 12..15 = mid of -2c; inside the tile
		 * the first halves of all rows, then the second halves (packed_half; load_packed_points has the matching order
		 * of the point's parts) */
		if (lane < KBLOCK) {
			const uint32_t q = lane % 4;
			const float exact = (j < k && q < dim) ? means[elem<LM>(stride_means, j, q)] : 0.0f;
			const float v = (j < k && q < dim) ? exact - (q == 0 ? frame[0] : q == 1 ? frame[1] : q == 2 ? frame[2] : frame[3]) : 0.0f;
			__bf16 hi, mid;
			const float rest = split_bf16(-2.0f * v, hi, mid);
			float* tile = packed + (size_t)(j / TILE) * tile_floats(rs);
			((__bf16*)(tile + packed_half(j % TILE, lane / 8)))[lane % 8] = (lane / 4) % 2 == 1 ? mid : hi;
			if (j % TILE == TILE - 1 && lane < TILE_PAD) tile[TILE * rs + lane] = 0.0f;
			if (lane < 4) {
				c2 = v * v;
				exact2 = exact * exact;
				mid2 = (float)mid * (float)mid;
				rest2 = rest * rest;
				if (q < dim) means_t[(size_t)q * kp + j] = exact; /* exact copy for the recheck pass */
			}
		}
	}
	else
	for (uint32_t q = lane; q < dp; q += WAVE) {
		const float exact = (j < k && q < dim) ? means[elem<LM>(stride_means, j, q)] : 0.0f;
		const float v = (j < k && q < dim) ? exact - wide_frame[q] : 0.0f;
		exact2 += exact * exact;
		c2 += v * v;
		__bf16 hi, mid;
		const float rest = split_bf16(-2.0f * v, hi, mid);
		mid2 += (float)mid * (float)mid;
		rest2 += rest * rest;
		/* block q / 16, half-wave (q % 16) / 8: 16-byte unit 4 kb + 2 h (hi), + 1 (mid) */
		const uint32_t unit = 4 * (q / KBLOCK) + 2 * ((q % KBLOCK) / 8);
		parts[8 * unit + q % 8] = hi;
		parts[8 * (unit + 1) + q % 8] = mid;
		if (q < dim) means_t[(size_t)q * kp + j] = exact; /* exact copy for the recheck pass */
	}
	const uint32_t pad_floats = ROW_PAD + (j % TILE == TILE - 1 ? TILE_PAD : 0);
	if (!packed_form && lane < pad_floats) row[dp + lane] = 0.0f;
	for (int off = WAVE / 2; off > 0; off >>= 1) {
		c2 += __shfl_xor(c2, off);
		mid2 += __shfl_xor(mid2, off);
		rest2 += __shfl_xor(rest2, off);
		exact2 += __shfl_xor(exact2, off);
	}
	if (lane == 0) {
		norms[norm_at(j)] = j < k ? c2 : __builtin_inff();
		norms[exact_norms_offset(kp) + norm_at(j)] = j < k ? exact2 : __builtin_inff();
		float* part_norms = norms + split_norms_offset(kp);
		part_norms[j] = mid2;
		part_norms[kp + j] = rest2;
	}
	if (lane < NORM_TILE - TILE && j % TILE == 0) {
		norms[(j / TILE) * NORM_TILE + TILE + lane] = __builtin_inff();
		norms[exact_norms_offset(kp) + (j / TILE) * NORM_TILE + TILE + lane] = __builtin_inff();
	}
}

bool bf16_supports(const AssignArgs& a, const DeviceInfo& dev)
{
	const uint32_t kb = pick_kb(a.dim);
	if (kb == 0) return false;
	/* two tiles (the double-buffered stream of the centroid block) plus the static flag lists must fit */
	return (size_t)(tile_floats(KBLOCK * kb + ROW_PAD) + NORM_TILE) * 4 * 2 + 2 * FLAG_CAP * MFMA_WAVES * 4 + 1024 <= dev.lds_bytes;
}

#define KMX_DECLARE_BF16_LAUNCHER(W) \
	int launch_bf16_##W(const AssignArgs& a, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev, uint32_t kp, float kd);
KMX_DECLARE_BF16_LAUNCHER(1) KMX_DECLARE_BF16_LAUNCHER(2) KMX_DECLARE_BF16_LAUNCHER(3) KMX_DECLARE_BF16_LAUNCHER(4)
KMX_DECLARE_BF16_LAUNCHER(8) KMX_DECLARE_BF16_LAUNCHER(16)

#define KMX_DECLARE_BF16_SCREEN(W) \
	int launch_screen_bf16_##W(const float* rows, const Workspace* ws, const uint32_t* row_queue, const uint32_t* row_count, \
	                           uint32_t* pairs, uint32_t* item_pairs, unsigned long long* keys, uint32_t dim, uint32_t k, uint32_t kp, \
	                           const DeviceInfo& dev, uint32_t* waves);
KMX_DECLARE_BF16_SCREEN(1) KMX_DECLARE_BF16_SCREEN(2) KMX_DECLARE_BF16_SCREEN(3) KMX_DECLARE_BF16_SCREEN(4)
KMX_DECLARE_BF16_SCREEN(8) KMX_DECLARE_BF16_SCREEN(16)

/* rows per work item of the screen: two tiles of 32 while the operands of two tiles fit the registers */
uint32_t screen_unit_rows(uint32_t dim) { return pick_kb(dim) <= 4 ? 2 * TILE : TILE; }

int launch_screen_bf16(const float* rows, const Workspace* ws, const uint32_t* row_queue, const uint32_t* row_count,
                       uint32_t* pairs, uint32_t* item_pairs, unsigned long long* keys, uint32_t dim, uint32_t k, uint32_t kp,
                       const DeviceInfo& dev, uint32_t* waves)
{
#define KMX_SCREEN_CASE(W) case W: return launch_screen_bf16_##W(rows, ws, row_queue, row_count, pairs, item_pairs, keys, dim, k, kp, dev, waves)
	switch (pick_kb(dim)) {
	KMX_SCREEN_CASE(1); KMX_SCREEN_CASE(2); KMX_SCREEN_CASE(3); KMX_SCREEN_CASE(4); KMX_SCREEN_CASE(8); KMX_SCREEN_CASE(16);
	default: return fail(KMX_ERR_UNSUPPORTED, "assign (split-bf16 MFMA): dim %u is not supported", dim);
	}
#undef KMX_SCREEN_CASE
}

int launch_assign_bf16(const AssignArgs& args, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev)
{
	AssignArgs a = args;
	/* wide rows and many centroids: a second sweep screens the queued points (narrow rows fit the registers of the
	 * lane-per-centroid kernels, which then need fewer launches); so do the packed rows, whose sweep queues more points
	 * than the fp32 one and screens a tile with a single MFMA */
	const bool screened = !a.ranking_only && a.k >= 128 && (a.dim > 32 || packed_rows(a.dim));
	/* The sweep works in a frame moved to the middle of the centroids (certificate.h): tau then scales with the spread of
	 * the data instead of its distance from the origin. The screen shares the frame and takes the thresholds as they are
	 * (queue entries beyond its block of copied rows, which other kernels read, get infinite ones); for the other kernels
	 * of the exact pass the sweep takes the thresholds back to the frame of the data. The packed rows move only where the
	 * screen follows; the double path ranks float copies of its points, whose rounding is relative to the origin anyway. */
	a.shift_rows = packed_rows(a.dim) ? screened : !a.ranking_only;
	a.shifted_cap = (a.shift_rows && screened) ? screened_rows_cap(a) : 0xFFFFFFFFu;
	a.unmoved_thresholds = a.shift_rows && !screened;
	const uint32_t kb = pick_kb(a.dim);
	const uint32_t dp = KBLOCK * kb;
	const uint32_t kp = round_up(a.k, TILE);
	const uint32_t rs = packed_rows(a.dim) ? row_floats<1, true>() : dp + ROW_PAD;
	int rc = reserve_packed(ws, (size_t)(kp / TILE) * tile_floats(rs), split_norms_floats(kp), (size_t)kp * a.dim);
	if (rc) return rc;
	rc = reserve_queue(ws, 2 * (size_t)a.n); /* (point, threshold) pairs */
	if (rc) return rc;
	const uint32_t pack_blocks = (kp * WAVE + 255) / 256;
	if (a.layout_means == KMX_AOS)
		KMX_LAUNCH_KERNEL((pack_means_bf16_kernel<KMX_AOS>), dim3(pack_blocks), dim3(256), 0, stream(),
		                   a.means, a.stride_means, ws->packed_means, ws->norms, ws->means_t, a.dim, a.k, kp, dp, (packed_rows(a.dim) ? 1u : 0u) | (a.shift_rows ? 2u : 0u), ws->counters);
	else
		KMX_LAUNCH_KERNEL((pack_means_bf16_kernel<KMX_SOA>), dim3(pack_blocks), dim3(256), 0, stream(),
		                   a.means, a.stride_means, ws->packed_means, ws->norms, ws->means_t, a.dim, a.k, kp, dp, (packed_rows(a.dim) ? 1u : 0u) | (a.shift_rows ? 2u : 0u), ws->counters);
	KMX_LAUNCH_CHECK("pack_means_bf16_kernel");

	/* tau = kd (|x|^2 + max|c|^2) + the bound of the dropped products (certificate.h) */
	const float kd = (packed_rows(a.dim) ? cert_kd_packed(a.dim) : cert_kd_split(a.dim) + (a.shift_rows ? 8.0f * CERT_UNIT : 0.0f)) + a.kd_extra;
	switch (kb) {
	case 1: rc = launch_bf16_1(a, exec, ws, dev, kp, kd); break;
	case 2: rc = launch_bf16_2(a, exec, ws, dev, kp, kd); break;
	case 3: rc = launch_bf16_3(a, exec, ws, dev, kp, kd); break;
	case 4: rc = launch_bf16_4(a, exec, ws, dev, kp, kd); break;
	case 8: rc = launch_bf16_8(a, exec, ws, dev, kp, kd); break;
	case 16: rc = launch_bf16_16(a, exec, ws, dev, kp, kd); break;
	default: return fail(KMX_ERR_UNSUPPORTED, "assign (split-bf16 MFMA): dim %u is not supported", a.dim);
	}
	if (rc) return rc;
	if (a.ranking_only) return KMX_OK; /* the caller resolves the queued points */
	ws->exact_norms = ws->norms + exact_norms_offset(kp);
	rc = screened ? launch_recheck_screened(a, ws, kp, dev) : launch_recheck(a, ws, kp);
	ws->exact_norms = nullptr;
	return rc;
}

} // namespace kmx
