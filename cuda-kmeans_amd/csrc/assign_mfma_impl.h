/*
 * Device code of the MFMA assignment (see assign_mfma.hip for the design notes). Kept in a header because the
 * kernel is instantiated per row width in separate translation units (assign_mfma_inst.hip, one object per
 * KMX_DPH value) so that the instantiations compile in parallel.
 */
#ifndef KMX_ASSIGN_MFMA_IMPL_H
#define KMX_ASSIGN_MFMA_IMPL_H

#include "kmx_internal.h"
#include "certificate.h"

#include <algorithm>

namespace kmx {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

constexpr uint32_t TILE = 32;       /* centroids per MFMA tile = points per MFMA tile */
constexpr uint32_t ROW_PAD = 4;     /* floats appended to every packed centroid row   */
constexpr uint32_t TILE_PAD = 4;    /* floats appended to every packed tile of 32 rows */
constexpr uint32_t NORM_TILE = 36;  /* floats per tile in the norms array (32 + 4 padding) */
constexpr uint32_t MFMA_WAVES = 8;  /* wavefronts per work-group                      */
constexpr uint32_t FLAG_CAP = 128;  /* per-wavefront list of points waiting for the recheck queue */

/*
 * A recheck queue entry is two words: the point index and, as float bits, the screening threshold of the point:
 * the smallest ranking value a[j] the sweep saw plus tau. A centroid whose a[j] exceeds it cannot be the serial
 * result (same argument as for the certification), so the exact pass only evaluates the others. Anything that is
 * not a finite number (NaN, overflow) becomes +inf: every centroid is then evaluated.
 */
__device__ __forceinline__ uint32_t screening_threshold(float first, float tau)
{
	const float t = first + tau;
	return __float_as_uint(__builtin_fabsf(t) < __builtin_inff() ? t : __builtin_inff());
}
constexpr uint32_t COARSE_MIN_TILES = 10; /* from this many centroid tiles on, track per tile and refine */

/*
 * The frame of a sweep: FRAME_DIMS coordinates of the vector m that is subtracted from every point and centroid before
 * the sweep uses them (zeros: the frame of the data), then |m|^2 and an upper bound of |m|. tau scales with
 * |x - m|^2 + max |c - m|^2, so with m in the middle of the data it no longer grows with the distance of the data from
 * the origin (certificate.h).
 */
constexpr uint32_t FRAME_DIMS = 256;
constexpr uint32_t FRAME_FLOATS = FRAME_DIMS + 4;
/* the norms array of the fp32 sweeps: the tiles of |c - m|^2, the frame, the tiles of |c|^2 (for the exact pass) */
__host__ __device__ __forceinline__ size_t plain_frame_offset(uint32_t kp) { return (size_t)(kp / TILE) * NORM_TILE; }
__host__ __device__ __forceinline__ size_t plain_exact_norms_offset(uint32_t kp) { return plain_frame_offset(kp) + FRAME_FLOATS; }
__host__ __device__ __forceinline__ size_t plain_norms_floats(uint32_t kp) { return plain_exact_norms_offset(kp) + (size_t)(kp / TILE) * NORM_TILE; }

/*
 * The frame of a call, for the packing kernels (256 threads): m = the mean of the first 16 centroids, finite coordinates
 * only (any vector would do; this one lies inside the data), a thread per dimension with its 16 loads in flight together;
 * zeros when `moved` is FRAME_KEPT, and with FRAME_MOVED_IF_FAR also when |m|^2 is at most 16 times the mean squared
 * distance of those centroids from m (data about the origin: a kernel that pays for the subtraction per point can then
 * skip it). Every work-group computes it into `m` (LDS, dp <= FRAME_DIMS floats), in the same order; the first one stores
 * it at `stored` with |m|^2 (as computed: it enters the shift of the thresholds) and an upper bound of |m|. Ends with a
 * barrier.
 */
constexpr uint32_t FRAME_KEPT = 0, FRAME_MOVED = 1, FRAME_MOVED_IF_FAR = 2;
template <int LM>
__device__ __forceinline__ void sweep_frame(const float* __restrict__ means, size_t stride_means, uint32_t dim, uint32_t k, uint32_t dp,
                                            uint32_t moved, float* m, float* __restrict__ stored)
{
	constexpr uint32_t SAMPLE = 16;
	const uint32_t sample = min(k, SAMPLE);
	__shared__ float frame_far[2][4]; /* per wavefront: its share of |m|^2 and of the summed squared distances */
	float mine_m2 = 0.0f, mine_spread = 0.0f;
	for (uint32_t q = threadIdx.x; q < dp; q += blockDim.x) {
		float sum = 0.0f;
		if (moved != FRAME_KEPT && q < dim) {
			float v[SAMPLE];
#pragma unroll
			for (uint32_t r = 0; r < SAMPLE; ++r) v[r] = r < sample ? means[elem<LM>(stride_means, r, q)] : 0.0f;
#pragma unroll
			for (uint32_t r = 0; r < SAMPLE; ++r) sum += __builtin_fabsf(v[r]) < __builtin_inff() ? v[r] : 0.0f;
			sum = sum / (float)sample;
			sum = __builtin_fabsf(sum) < __builtin_inff() ? sum : 0.0f; /* (the sum of finite values may overflow) */
			mine_m2 += sum * sum;
#pragma unroll
			for (uint32_t r = 0; r < SAMPLE; ++r)
				if (r < sample && __builtin_fabsf(v[r]) < __builtin_inff()) mine_spread += (v[r] - sum) * (v[r] - sum);
		}
		m[q] = sum;
	}
	if (moved == FRAME_MOVED_IF_FAR) {
		for (int off = 32; off > 0; off >>= 1) {
			mine_m2 += __shfl_xor(mine_m2, off);
			mine_spread += __shfl_xor(mine_spread, off);
		}
		if ((threadIdx.x & 63u) == 0) { frame_far[0][threadIdx.x / 64] = mine_m2; frame_far[1][threadIdx.x / 64] = mine_spread; }
		__syncthreads();
		const float m2 = (frame_far[0][0] + frame_far[0][1]) + (frame_far[0][2] + frame_far[0][3]);
		const float spread = ((frame_far[1][0] + frame_far[1][1]) + (frame_far[1][2] + frame_far[1][3])) / (float)sample;
		if (!(m2 > 16.0f * spread)) /* (the same decision in every work-group: the same numbers in the same order) */
			for (uint32_t q = threadIdx.x; q < dp; q += blockDim.x) m[q] = 0.0f;
	}
	__syncthreads();
	if (blockIdx.x == 0) {
		for (uint32_t q = threadIdx.x; q < dp; q += blockDim.x) stored[q] = m[q];
		if (threadIdx.x < 64) {
			float m2 = 0.0f;
			for (uint32_t q = threadIdx.x; q < dp; q += 64) m2 += m[q] * m[q];
			for (int off = 32; off > 0; off >>= 1) m2 += __shfl_xor(m2, off);
			if (threadIdx.x == 0) {
				stored[FRAME_DIMS] = m2;
				stored[FRAME_DIMS + 1] = __builtin_sqrtf(m2) * 1.0001f;
			}
		}
	}
}

__host__ __device__ constexpr uint32_t round_up(uint32_t v, uint32_t m) { return (v + m - 1) / m * m; }
/* floats of one packed tile / offset of a packed row / offset of a norm */
__host__ __device__ constexpr uint32_t tile_floats(uint32_t rs) { return TILE * rs + TILE_PAD; }
__host__ __device__ __forceinline__ size_t packed_row(uint32_t row, uint32_t rs) { return (size_t)(row / TILE) * tile_floats(rs) + (size_t)(row % TILE) * rs; }
__host__ __device__ __forceinline__ uint32_t norm_at(uint32_t row) { return (row / TILE) * NORM_TILE + (row % TILE); }

/*
 * The serial distance of one (point, centroid) pair -- subtract, multiply, add, every operation rounded separately, in
 * ascending dimension, then the correctly rounded square root (reference metric_policies.hpp:23-28,40-44) -- merged
 * into the point's 64-bit key (distance bits << 32 | centroid) by an atomic minimum: the smallest key is what the
 * serial scan returns (lower index on equal distances; a NaN distance has the largest bit patterns and never wins,
 * except at centroid 0, where the scan starts: key 0). Contraction is off inside this function whatever the
 * translation unit's setting.
 */
template <int LD>
static __device__ __forceinline__ void evaluate_pair(const float* __restrict__ data, size_t stride, const float* __restrict__ means_t,
                                                      uint32_t dim, uint32_t kp, uint32_t pt, uint32_t r, unsigned long long* key_slot)
{
#pragma clang fp contract(off)
	float sum = 0.0f;
#pragma unroll 16
	for (uint32_t q = 0; q < dim; ++q) {
		float diff = data[elem<LD>(stride, pt, q)] - means_t[(size_t)q * kp + r];
		float sq = diff * diff;
		sum = sum + sq;
	}
	const float dist = __builtin_sqrtf(sum);
	const unsigned long long key = (r == 0 && dist != dist) ? 0ull : (((unsigned long long)__float_as_uint(dist) << 32) | r);
	atomicMin(key_slot, key);
}

/*
 * Work items of the screen of the exact pass (screen_bf16_kernel) and of the kernel that evaluates what it notes: a
 * unit of `unit_rows` queued rows, and, when there are fewer units than wavefronts in the launch (as many as the
 * device holds at once), a share of the centroid tiles.
 * Every item owns a slice of SCREEN_SLICE_PER_ROW * unit_rows (row, centroid) pairs of the list and a counter.
 */
constexpr uint32_t SCREEN_WAVES = 4;          /* wavefronts per work-group */
constexpr uint32_t SCREEN_MAX_WAVES = 16384;  /* upper bound of the wavefronts of a launch (as many as are resident at once) */
constexpr uint32_t SCREEN_SLICE_PER_ROW = 4;
struct ScreenItems { uint32_t units, parts, part_tiles, items; };
__host__ __device__ __forceinline__ ScreenItems screen_items(uint32_t rows, uint32_t unit_rows, uint32_t tiles, uint32_t waves)
{
	ScreenItems w;
	w.units = (rows + unit_rows - 1) / unit_rows;
	uint32_t want = w.units ? waves / w.units : 1u;
	if (want < 2u && w.units) {
		/* about as many units as wavefronts, or more: the wavefronts go round ceil(items / waves) times, and the last round
		 * may be nearly empty (1225 units on 1024 wavefronts: two rounds for 1.2 rounds of work). Shares of the tiles make
		 * the rounds shorter: the split with the least rounds of whole sweeps, while the items stay within the bound of
		 * screen_items_max. */
		uint32_t best_rounds = (w.units + waves - 1) / waves * 8u; /* in eighths of a whole sweep */
		want = 1u;
		for (uint32_t p = 2; p <= 8u && p <= tiles && w.units * p <= SCREEN_MAX_WAVES; p *= 2) {
			const uint32_t rounds = (w.units * p + waves - 1) / waves * (8u / p);
			if (rounds < best_rounds) { best_rounds = rounds; want = p; }
		}
	}
	want = want < 1u ? 1u : (want > tiles ? tiles : want);
	w.part_tiles = (tiles + want - 1) / want;
	w.parts = (tiles + w.part_tiles - 1) / w.part_tiles;
	w.items = w.units * w.parts;
	return w;
}
/* upper bound of the number of items for up to `cap` rows */
__host__ __forceinline__ uint32_t screen_items_max(uint32_t cap, uint32_t unit_rows)
{
	const uint32_t units = (cap + unit_rows - 1) / unit_rows;
	return units > SCREEN_MAX_WAVES ? units : SCREEN_MAX_WAVES;
}

/* points of one sweep unit (P tiles of 32 points) -> registers as MFMA B operands; rows beyond n read as zero */
template <int DPH, int P, int LD, bool VEC>
__device__ __forceinline__ void load_points(float (&b)[P][DPH], const float* __restrict__ data, size_t stride,
                                            uint32_t base, uint32_t col, uint32_t h, uint32_t dim, uint32_t n)
{
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
			/* wide rows: the address advances from load to load and the loads are issued in groups of 16, so that
			 * no more than 16 addresses are alive at a time (128 independent 64-bit addresses do not fit the registers) */
			const float* src = data + (size_t)(h * DPH) * stride + pt;
#pragma unroll
			for (int s = 0; s < DPH; ++s) {
				b[p][s] = (valid && h * DPH + s < dim) ? *src : 0.0f;
				src += stride;
				if (DPH > 64 && s % 16 == 15) __builtin_amdgcn_sched_barrier(0);
			}
		}
	}
}

/* min(a, b) as one v_med3_f32: median(a, b, -inf). Unlike fminf() it needs no canonicalisation of the MFMA
 * results, and its result is known to be canonical, so the fminf() tree above it folds into v_min3_f32.
 * neg_inf arrives as a kernel argument: a literal -inf would let the compiler rewrite the median as fminf(). */
__device__ __forceinline__ float min2_raw(float a, float b, float neg_inf) { return __builtin_amdgcn_fmed3f(a, b, neg_inf); }

/* per-lane tracking state of one point: smallest value, a lower bound for all others, where the smallest was seen */
struct Track {
	float m1, m2;
	uint32_t tile; /* tile of m1; with FINE8: 2 * tile + (0: results 0..7, 1: results 8..15) */
	uint32_t loc;  /* fine mode only: row of m1 inside the tile, without the half-wave's +4 */
};

/*
 * COARSE = true, 12 VALU operations per tile and point: the minimum t of the lane's 16 results (a min tree),
 * then over the tiles the smallest t (m1, with its tile) and the second smallest t (m2). Which of the 16
 * rows attained m1, and how close the runner-up inside that tile is, is settled once per sweep by the
 * refinement in the kernel, which recomputes those rows.
 * COARSE and FINE8, 16 operations: the same for the lane's results 0..7 and 8..15 separately (`tile` then holds
 * 2 * tile + group), so that the refinement recomputes 8 rows instead of 16: worth it when a row is long enough
 * for the refinement to cost more than four operations per tile.
 * COARSE = false, 66 operations: exact smallest / second smallest / row over all results; used when the
 * sweep has too few tiles to pay for the refinement.
 */
template <bool COARSE, bool FINE8>
__device__ __forceinline__ void track_tile(const f32x16& acc, Track& s, uint32_t tile, float neg_inf)
{
	if (COARSE) {
		/* Minimum trees in v_minimum3_f32 (two values per instruction; unlike fminf() it needs no canonicalised operands,
		 * so it works on the raw MFMA results). It propagates NaN: a group that contains a NaN result has a NaN minimum,
		 * which is never smaller than m1 and makes the median below return m1, so m2 = m1 and the point is not
		 * certified -- the exact pass then decides it, as it must. */
		auto lowest = [](float a, float b) { return __builtin_elementwise_minimum(a, b); };
		if (FINE8) {
			const float ta = lowest(lowest(lowest(lowest(lowest(lowest(lowest(acc[0], acc[1]), acc[2]), acc[3]), acc[4]), acc[5]), acc[6]), acc[7]); /* results 0..7 */
			const float tb = lowest(lowest(lowest(lowest(lowest(lowest(lowest(acc[8], acc[9]), acc[10]), acc[11]), acc[12]), acc[13]), acc[14]), acc[15]); /* results 8..15 */
			s.m2 = __builtin_amdgcn_fmed3f(s.m1, s.m2, ta); /* second smallest of {m1, m2, ta} as m1 <= m2 */
			const bool lta = ta < s.m1;
			s.tile = lta ? 2 * tile : s.tile;
			s.m1 = lta ? ta : s.m1;
			s.m2 = __builtin_amdgcn_fmed3f(s.m1, s.m2, tb);
			const bool ltb = tb < s.m1;
			s.tile = ltb ? 2 * tile + 1 : s.tile;
			s.m1 = ltb ? tb : s.m1;
		}
		else {
			float t = acc[0];
#pragma unroll
			for (int i = 1; i < 16; ++i) t = lowest(t, acc[i]);
			s.m2 = __builtin_amdgcn_fmed3f(s.m1, s.m2, t); /* second smallest of {m1, m2, t} as m1 <= m2 */
			const bool lt = t < s.m1;
			s.tile = lt ? tile : s.tile;
			s.m1 = lt ? t : s.m1;
		}
	}
	else {
		const float start = s.m1;
#pragma unroll
		for (int r = 0; r < 16; ++r) {
			const float v = acc[r];
			s.m2 = __builtin_amdgcn_fmed3f(s.m1, s.m2, v);
			const bool lt = v < s.m1;
			s.loc = lt ? (uint32_t)(8 * (r / 4) + (r % 4)) : s.loc;
			s.m1 = lt ? v : s.m1;
		}
		s.tile = s.m1 < start ? tile : s.tile;
	}
}

/*
 * One step of the software pipeline: the MFMAs of tile `tile_new` (chunk-local number) into acc_new and the
 * tracking of the previous tile's results in acc_old, which are complete by then: no wavefront ever waits
 * for an MFMA result. sched_group_barrier keeps the MFMAs and the VALU work in GROUPS large runs.
 */
/* rows of at least 16 dimensions: the refinement is worth halving */
template <int DPH> constexpr bool fine8() { return DPH >= 8; }

template <int DPH, int P, bool TRACK, bool COARSE>
__device__ __forceinline__ void tile_step(const float* __restrict__ lds, const float* __restrict__ lds_norms, uint32_t tile_new,
                                          uint32_t col, uint32_t h, const float (&b)[P][DPH],
                                          f32x16 (&acc_new)[P], const f32x16 (&acc_old)[P], uint32_t tile_old,
                                          Track (&st)[P], float neg_inf)
{
	constexpr uint32_t RS = 2 * DPH + ROW_PAD;
	/* A operand: this lane's centroid row, its half of the dimensions */
	const float* arow = lds + (size_t)tile_new * tile_floats(RS) + (size_t)col * RS + h * DPH;
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
		f32x4 v = *(const f32x4*)(lds_norms + tile_new * NORM_TILE + 8 * g + 4 * h);
		cinit[4 * g] = v.x; cinit[4 * g + 1] = v.y; cinit[4 * g + 2] = v.z; cinit[4 * g + 3] = v.w;
	}
#pragma unroll
	for (int p = 0; p < P; ++p) acc_new[p] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[0], b[p][0], cinit, 0, 0, 0);
#pragma unroll
	for (int s = 1; s < DPH; ++s) {
#pragma unroll
		for (int p = 0; p < P; ++p) acc_new[p] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[s], b[p][s], acc_new[p], 0, 0, 0);
	}
	if (TRACK) {
#pragma unroll
		for (int p = 0; p < P; ++p) track_tile<COARSE, fine8<DPH>()>(acc_old[p], st[p], tile_old, neg_inf);
		constexpr int MFMAS = DPH * P;
		constexpr int GROUPS = COARSE ? 1 : (MFMAS >= 4 ? 4 : 1);
		constexpr int VALU_PER_GROUP = ((COARSE ? (fine8<DPH>() ? 16 : 12) : 67) * P + GROUPS - 1) / GROUPS;
		if (DPH <= 32) { /* wider rows: the tracking is a few per cent of the step, the default schedule will do */
#pragma unroll
			for (int i = 0; i < GROUPS; ++i) {
				__builtin_amdgcn_sched_group_barrier(0x008, MFMAS / GROUPS, 0);
				__builtin_amdgcn_sched_group_barrier(0x002, VALU_PER_GROUP, 0);
			}
		}
	}
}

template <int DPH, int P, int LD, bool VEC, bool STREAM, bool COARSE, bool PREFETCH>
__global__ void __launch_bounds__(MFMA_WAVES * WAVE)
assign_mfma_kernel(const float* __restrict__ data, size_t stride, const float* __restrict__ packed, const float* __restrict__ norms,
                   uint32_t* __restrict__ assignment, uint32_t* __restrict__ queue, uint32_t* __restrict__ counters,
                   uint32_t dim, uint32_t k, uint32_t kp, uint32_t n, uint32_t chunk_rows, float kd, float neg_inf, float kd_unmoved)
{
	constexpr uint32_t DP = 2 * DPH;
	constexpr uint32_t RS = DP + ROW_PAD;
	extern __shared__ float lds[];
	/* the frame of the sweep (sweep_frame; the packing kernel moved the centroids): m, |m|^2 and |m| */
	__shared__ __attribute__((aligned(16))) float frame_lds[DP];
	for (uint32_t i = threadIdx.x; i < DP; i += blockDim.x) frame_lds[i] = norms[plain_frame_offset(kp) + i];
	const float frame_m2 = norms[plain_frame_offset(kp) + FRAME_DIMS], frame_norm = norms[plain_frame_offset(kp) + FRAME_DIMS + 1];
	__shared__ uint32_t wave_max[MFMA_WAVES];
	__shared__ uint32_t flag_list[MFMA_WAVES][2 * FLAG_CAP]; /* (point, threshold) pairs */

	const uint32_t lane = threadIdx.x & (WAVE - 1);
	const uint32_t wave = threadIdx.x / WAVE;
	const uint32_t col = lane & 31; /* point within a tile (B column) / centroid row fed to A */
	const uint32_t h = lane >> 5;   /* half-wave: K split and the +4 row group of the result    */

	/* max_j |c_j|^2 (bit pattern maximum: propagates NaN and +inf, which then flag every point) */
	uint32_t cmax = 0;
	for (uint32_t j = threadIdx.x; j < k; j += blockDim.x) cmax = max(cmax, __float_as_uint(norms[norm_at(j)]));
	for (int off = WAVE / 2; off > 0; off >>= 1) cmax = max(cmax, (uint32_t)__shfl_xor((int)cmax, off));
	if (lane == 0) wave_max[wave] = cmax;
	__syncthreads();
	cmax = 0;
	for (uint32_t w = 0; w < MFMA_WAVES; ++w) cmax = max(cmax, wave_max[w]);
	const float c2max = __uint_as_float(cmax);

	float* lds_norms = lds + (size_t)(chunk_rows / TILE) * tile_floats(RS);
	const uint32_t chunks = (kp + chunk_rows - 1) / chunk_rows;

	auto stage = [&](uint32_t row0, uint32_t rows) {
		/* flat 16-byte copies of `rows` packed rows (whole tiles) and of their norms */
		const f32x4* src = (const f32x4*)(packed + packed_row(row0, RS));
		f32x4* dst = (f32x4*)lds;
		const uint32_t vecs = (rows / TILE) * tile_floats(RS) / 4;
		for (uint32_t i = threadIdx.x; i < vecs; i += blockDim.x) dst[i] = src[i];
		const f32x4* nsrc = (const f32x4*)(norms + (size_t)(row0 / TILE) * NORM_TILE);
		f32x4* ndst = (f32x4*)lds_norms;
		const uint32_t nvecs = (rows / TILE) * NORM_TILE / 4;
		for (uint32_t i = threadIdx.x; i < nvecs; i += blockDim.x) ndst[i] = nsrc[i];
	};

	if (!STREAM) {
		stage(0, kp);
		__syncthreads();
	}

	/* flagged points are collected per wavefront in LDS and appended to the queue FLAG_CAP at a time */
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

	/* one sweep unit = P tiles of 32 points per wavefront; the next unit's points are requested
	 * before the sweep over the centroids starts, so the load latency hides behind it */
	const uint32_t unit_points = MFMA_WAVES * P * TILE;
	const uint32_t units = (n + unit_points - 1) / unit_points;

	auto sweep = [&](float (&b)[P][DPH], uint32_t base) {
		float x2[P], along_m[P]; /* |x - m|^2 and (x - m) . m of the points */
		Track st[P];
#pragma unroll
		for (int p = 0; p < P; ++p) {
			float part = 0.0f, along = 0.0f;
#pragma unroll
			for (int s = 0; s < DPH; ++s) {
				const float m = frame_lds[h * DPH + s];
				b[p][s] -= m; /* the rows are swept in the moved frame (rows beyond n, read as zero, become -m: they are not written back) */
				part += b[p][s] * b[p][s];
				along += b[p][s] * m;
			}
			x2[p] = part + __shfl_xor(part, 32);
			along_m[p] = along + __shfl_xor(along, 32);
			st[p].m1 = __builtin_inff();
			st[p].m2 = __builtin_inff();
			st[p].tile = 0;
			st[p].loc = 0;
		}
		f32x16 acc0[P], acc1[P];
		for (uint32_t chunk = 0; chunk < chunks; ++chunk) {
			const uint32_t row0 = chunk * chunk_rows;
			const uint32_t rows = min(chunk_rows, kp - row0);
			if (STREAM) {
				__syncthreads(); /* everyone is done with the previous chunk */
				stage(row0, rows);
				__syncthreads();
			}
			const uint32_t tiles = rows / TILE;
			const uint32_t tile0 = row0 / TILE; /* global number of the chunk's first tile */
			tile_step<DPH, P, false, COARSE>(lds, lds_norms, 0, col, h, b, acc0, acc1, 0, st, neg_inf);
			uint32_t t = 0; /* acc0 holds tile t, not yet tracked */
			while (t + 2 < tiles) {
				tile_step<DPH, P, true, COARSE>(lds, lds_norms, t + 1, col, h, b, acc1, acc0, tile0 + t, st, neg_inf);
				tile_step<DPH, P, true, COARSE>(lds, lds_norms, t + 2, col, h, b, acc0, acc1, tile0 + t + 1, st, neg_inf);
				t += 2;
			}
			if (t + 1 < tiles) {
				tile_step<DPH, P, true, COARSE>(lds, lds_norms, t + 1, col, h, b, acc1, acc0, tile0 + t, st, neg_inf);
#pragma unroll
				for (int p = 0; p < P; ++p) track_tile<COARSE, fine8<DPH>()>(acc1[p], st[p], tile0 + t + 1, neg_inf);
			}
			else {
#pragma unroll
				for (int p = 0; p < P; ++p) track_tile<COARSE, fine8<DPH>()>(acc0[p], st[p], tile0 + t, neg_inf);
			}
		}

#pragma unroll
		for (int p = 0; p < P; ++p) {
			/* the other half-wave's state for the same point */
			const float o1 = __shfl_xor(st[p].m1, 32);
			const float o2 = __shfl_xor(st[p].m2, 32);
			const uint32_t ot = (uint32_t)__shfl_xor((int)st[p].tile, 32);
			const bool win = st[p].m1 < o1 || (st[p].m1 == o1 && h == 0);
			uint32_t idx;
			float first, second;
			if (COARSE) {
				/*
				 * Refinement. The two half-waves hold disjoint 16-row subsets of every tile, tracked whole or (FINE8)
				 * as two groups of 8 rows. The tracked group with the smallest m1 (half wh, tile ts) contains the
				 * winner; everything outside it is bounded below by W = min(the other half's m1, the winning
				 * half's m2). The values of the winning group are
				 * recomputed with plain fused multiply-adds (both half-waves contribute their half of the
				 * dimensions), which yields the winner's row and the runner-up inside the subset. The
				 * recomputed values obey the same rounding-error bound as the MFMA results, so tau covers them.
				 */
				constexpr bool FINE8 = fine8<DPH>();
				constexpr int ROWS = FINE8 ? 8 : 16;
				const uint32_t code = win ? st[p].tile : ot;
				const uint32_t ts = FINE8 ? code >> 1 : code;      /* tile */
				const uint32_t sub = FINE8 ? 2 * (code & 1u) : 0u; /* first group of 4 rows of the tracked group */
				const uint32_t wh = win ? h : 1u - h;
				const float W = win ? fminf(o1, st[p].m2) : fminf(st[p].m1, o2);
				const float* tile_base = STREAM ? packed + (size_t)ts * tile_floats(RS) : lds + (size_t)ts * tile_floats(RS);
				const float* norm_base = STREAM ? norms + ts * NORM_TILE : lds_norms + ts * NORM_TILE;
				float tot[ROWS];
#pragma unroll
				for (int r = 0; r < ROWS; ++r) {
					const float* ar = tile_base + (size_t)(8 * (sub + r / 4) + 4 * wh + (r % 4)) * RS + h * DPH;
					float part = 0.0f;
					if (DPH % 4 == 0) {
#pragma unroll
						for (int s = 0; s < DPH; s += 4) {
							const f32x4 v = *(const f32x4*)(ar + s);
							part = __builtin_fmaf(v.x, b[p][s], part);
							part = __builtin_fmaf(v.y, b[p][s + 1], part);
							part = __builtin_fmaf(v.z, b[p][s + 2], part);
							part = __builtin_fmaf(v.w, b[p][s + 3], part);
						}
					}
					else {
#pragma unroll
						for (int s = 0; s < DPH; s += 2) {
							const f32x2 v = *(const f32x2*)(ar + s);
							part = __builtin_fmaf(v.x, b[p][s], part);
							part = __builtin_fmaf(v.y, b[p][s + 1], part);
						}
					}
					tot[r] = part;
				}
				float v1 = __builtin_inff(), v2 = __builtin_inff();
				uint32_t rbest = 0;
#pragma unroll
				for (int g = 0; g < ROWS / 4; ++g) {
					const f32x4 c2 = *(const f32x4*)(norm_base + 8 * (sub + g) + 4 * wh);
#pragma unroll
					for (int q = 0; q < 4; ++q) {
						const int r = 4 * g + q;
						const float v = (tot[r] + __shfl_xor(tot[r], 32)) + c2[q];
						v2 = __builtin_amdgcn_fmed3f(v1, v2, v);
						const bool lt = v < v1;
						rbest = lt ? (uint32_t)r : rbest;
						v1 = lt ? v : v1;
					}
				}
				idx = ts * TILE + 8 * (sub + rbest / 4) + 4 * wh + (rbest % 4);
				first = v1;
				second = fminf(v2, W);
			}
			else {
				const uint32_t mine_idx = st[p].tile * TILE + st[p].loc + 4 * h;
				const uint32_t oi = (uint32_t)__shfl_xor((int)mine_idx, 32);
				idx = win ? mine_idx : oi;
				first = fminf(st[p].m1, o1);
				second = fminf(fmaxf(st[p].m1, o1), fminf(st[p].m2, o2));
			}
			const float tau = kd * (x2[p] + c2max);
			const uint32_t pt = base + p * TILE + col;
			const bool mine = h == 0 && pt < n;
			const bool decided = (second - first > tau) && (x2[p] + c2max > 1e-30f);
			if (mine) assignment[pt] = idx < k ? idx : 0u;
			const bool flag = mine && !decided;
			const unsigned long long mask = __ballot(flag);
			if (mask) {
				const uint32_t add = (uint32_t)__builtin_popcountll(mask);
				if (flagged + add > FLAG_CAP) flush_flags();
				if (flag) {
					const uint32_t at = 2 * (flagged + __builtin_popcountll(mask & ((1ull << lane) - 1ull)));
					flag_list[wave][at] = pt;
					/* the exact pass evaluates in the frame of the data (certificate.h) */
					flag_list[wave][at + 1] = kd_unmoved > 0.0f
						? screening_threshold(cert_unmoved_threshold(first, tau, x2[p], along_m[p], c2max, frame_m2, frame_norm, kd_unmoved), 0.0f)
						: screening_threshold(first, tau);
				}
				flagged += add;
			}
		}
	};

	if (PREFETCH) {
		float b0[P][DPH], b1[P][DPH];
		uint32_t unit = blockIdx.x;
		if (unit < units) load_points<DPH, P, LD, VEC>(b0, data, stride, (unit * MFMA_WAVES + wave) * P * TILE, col, h, dim, n);
		while (unit < units) {
			uint32_t next = unit + gridDim.x;
			if (next < units) load_points<DPH, P, LD, VEC>(b1, data, stride, (next * MFMA_WAVES + wave) * P * TILE, col, h, dim, n);
			sweep(b0, (unit * MFMA_WAVES + wave) * P * TILE);
			unit = next;
			if (unit >= units) break;
			next = unit + gridDim.x;
			if (next < units) load_points<DPH, P, LD, VEC>(b0, data, stride, (next * MFMA_WAVES + wave) * P * TILE, col, h, dim, n);
			sweep(b1, (unit * MFMA_WAVES + wave) * P * TILE);
			unit = next;
		}
	}
	else {
		/* wide rows: one set of point registers, the (long) sweep dwarfs the load latency */
		float b0[P][DPH];
		for (uint32_t unit = blockIdx.x; unit < units; unit += gridDim.x) {
			load_points<DPH, P, LD, VEC>(b0, data, stride, (unit * MFMA_WAVES + wave) * P * TILE, col, h, dim, n);
			sweep(b0, (unit * MFMA_WAVES + wave) * P * TILE);
		}
	}
	if (flagged) flush_flags();
}

/* points per wavefront and sweep, and whether the next sweep's points are prefetched: bounded by the register file */
template <int DPH> struct SweepShape { static constexpr int P = DPH <= 8 ? 4 : (DPH <= 32 ? 2 : 1); static constexpr bool PREFETCH = DPH <= 64; };

template <int DPH, int LD, bool VEC>
static int launch_mfma_t(const AssignArgs& a, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev, uint32_t kp, float kd)
{
	constexpr uint32_t RS = 2 * DPH + ROW_PAD;
	constexpr int P = SweepShape<DPH>::P;
	constexpr bool PF = SweepShape<DPH>::PREFETCH;
	uint32_t budget = exec->shared_mem_bytes ? std::min(exec->shared_mem_bytes, dev.lds_bytes) : dev.lds_bytes;
	const uint32_t static_bytes = (2 * FLAG_CAP * MFMA_WAVES + 64 + 2 * DPH) * 4; /* static LDS of the kernel */
	const uint32_t tile_bytes = (tile_floats(RS) + NORM_TILE) * 4;
	if (budget < static_bytes + tile_bytes) return fail(KMX_ERR_UNSUPPORTED, "assign (MFMA): LDS budget of %u bytes is too small", budget);
	const uint32_t chunk_rows = std::min<uint32_t>(kp, (budget - static_bytes) / tile_bytes * TILE);
	const bool stream_mode = chunk_rows < kp;
	/* per-tile tracking + refinement pays from about ten tiles on and while a row is short; long rows make the
	 * per-result tracking cheap relative to the MFMAs and the refinement expensive */
	const bool coarse = kp / TILE >= COARSE_MIN_TILES && DPH <= 32;
	const uint32_t lds_bytes = chunk_rows / TILE * tile_bytes;
	const uint32_t unit_points = MFMA_WAVES * P * TILE;
	const uint32_t units = (a.n + unit_points - 1) / unit_points;
	void (*kernel)(const float*, size_t, const float*, const float*, uint32_t*, uint32_t*, uint32_t*,
	               uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, float, float, float) = nullptr;
	if constexpr (DPH <= 32) {
		if (stream_mode) kernel = coarse ? assign_mfma_kernel<DPH, P, LD, VEC, true, true, PF> : assign_mfma_kernel<DPH, P, LD, VEC, true, false, PF>;
		else kernel = coarse ? assign_mfma_kernel<DPH, P, LD, VEC, false, true, PF> : assign_mfma_kernel<DPH, P, LD, VEC, false, false, PF>;
	}
	else {
		/* wide rows: one instantiation (chunked staging also serves a single chunk; per-result tracking) */
		kernel = assign_mfma_kernel<DPH, P, LD, VEC, true, false, PF>;
	}
	KMX_HIP(hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
	/* persistent work-groups: as many as fit a CU at once (small k leaves room for several, which the
	 * HBM-bound shapes need to keep enough loads in flight) */
	int per_cu = 1;
	KMX_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, (const void*)kernel, (int)(MFMA_WAVES * WAVE), lds_bytes));
	per_cu = std::max(1, std::min(per_cu, 4));
	const uint32_t grid = std::min(units, dev.compute_units * (uint32_t)per_cu);
	exec->block_count = grid;
	int rc = profile_begin(0);
	if (rc) return rc;
	KMX_LAUNCH_KERNEL(kernel, dim3(grid), dim3(MFMA_WAVES * WAVE), lds_bytes, stream(),
	                   a.data, a.stride, ws->packed_means, ws->norms, a.assignment, ws->queue, ws->counters,
	                   a.dim, a.k, kp, a.n, chunk_rows, kd, -__builtin_inff(), a.unmoved_thresholds ? cert_kd_unmoved(a.dim) : 0.0f);
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


} // namespace kmx

#endif
