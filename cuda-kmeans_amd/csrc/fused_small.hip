/*
 * One whole iteration in a single pass over the points, for a handful of centroids (k <= 32, rows up to 32
 * floats): the shapes where the iteration is bound by HBM and reading the points twice (assignment, then
 * update) costs the most. Role of the reference's fused kernels (kernels.cu:883-1190).
 *
 * Two kernels, by the width of the rows (launch_fused_t): fused_small_kernel, one lane per point, for rows of 4 and 24
 * floats, and fused_matrix_kernel (described where it stands), which ranks on the matrix cores, for rows of 8, 16 and 32.
 * fused_small_kernel: one lane owns one point, its coordinates in registers.
 *   1. Ranking a[j] = |c_j|^2 - 2 c_j.x with plain fused multiply-adds; the packed centroid rows are read with
 *      wave-uniform addresses (scalar loads, scalar operands). The low bits of a value's
 *      mantissa are replaced by the centroid's number, so the lane tracks its three smallest values with one
 *      minimum and two medians per centroid and reads the two leaders out of the values at the end; the bound
 *      tau pays for the replaced bits (cert_kd_keyed).
 *   2. Exact result without a second kernel: if the runner-up is further than tau from the best, the best is the
 *      serial result (same bound as the other fast variants, see assign_mfma.hip); if only the THIRD is further
 *      than tau, the serial result is one of the two leaders, and the serial arithmetic on those two settles it.
 *      Such points (a few in a hundred) are not settled where they turn up: the wavefront notes them in a list in
 *      LDS and, once half a wavefront of them waits, reads their rows again and settles them together, one per
 *      lane. Only a point with three or more centroids within tau, or with data the bound does not cover (NaN,
 *      overflow), stays unresolved: it goes to the recheck queue and a fix-up kernel adds it to the sums afterwards.
 *   3. Accumulation on the matrix cores: the sums of a wavefront's 64 points are the product of the k x 64 indicator
 *      matrix (1 where the point belongs to the cluster) with the 64 x dim block of coordinates. The wavefront parks
 *      its rows and results in LDS (that transposes them: the MFMA wants one lane per dimension) and issues
 *      v_mfma_f32_16x16x4_f32 with the indicator as A and the coordinates as B; the accumulators stay in registers
 *      for the whole kernel. 1.0 * x is exact, so only the summation order differs from the serial one. Rows of
 *      points that are not settled yet are parked as zeros (0 * NaN would poison every cluster). Counts are integer
 *      LDS atomics. At the end the four wavefronts' accumulators meet in LDS: one global atomic per element and
 *      work-group.
 *
 * Floating-point contraction is off for the whole file (the serial arithmetic must not fuse); the rankings use
 * explicit fused multiply-adds and matrix instructions.
 */
#include <type_traits>
#include "certificate.h"
#include "assign_mfma_impl.h"

#pragma clang fp contract(off)

namespace kmx {

constexpr uint32_t FUSED_WAVES = 4;
constexpr uint32_t UNRESOLVED = 0xFFFFFFFFu;
constexpr uint32_t FUSED_FLAG_CAP = WAVE;      /* per-wavefront list of points on their way to the recheck queue */
constexpr uint32_t FUSED_LATER_CAP = WAVE;     /* per-wavefront list of points waiting for the arithmetic on their two leaders */
constexpr uint32_t FUSED_LATER_DRAIN = WAVE / 2;

typedef float f32x4v __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
constexpr size_t FUSED_MAX_DATA_BYTES = 0xF0000000u; /* what one buffer descriptor spans, less room for a batch past the end */

/* LDS words per wavefront of the matrix-ranking kernel: parked rows (or the sums at the end) and the membership rows */
__host__ __device__ constexpr uint32_t fused_matrix_wave_floats(uint32_t nt, uint32_t mt)
{
	return (WAVE * (nt * 16 + 2) > mt * 16 * nt * 16 ? WAVE * (nt * 16 + 2) : mt * 16 * nt * 16) + WAVE * mt * 16 / 2;
}

__host__ __device__ constexpr uint32_t fused_key_bits(uint32_t mt) { return mt == 1 ? 4u : 5u; } /* 16 centroids per MT */

/* EMIT: the result of every point the kernel settles is also written to `assignment` (the points it leaves to the exact
 * pass are written there by that pass): the iteration then hands out the assignment vector the reference's unfused driver
 * keeps (cuda.hpp:26,72-85), for one more coalesced store of 4 n bytes. */
template <int DP, int LD, int LM, int MT, bool EMIT>
__global__ void __launch_bounds__(FUSED_WAVES * WAVE) __attribute__((amdgpu_waves_per_eu(DP == 16 ? 7 : 1)))
fused_small_kernel(const float* __restrict__ data, size_t stride, const float* __restrict__ packed, const float* __restrict__ norms,
                   const float* __restrict__ means_in, size_t stride_means,
                   float* __restrict__ means_out, uint32_t* __restrict__ sizes,
                   uint32_t* __restrict__ queue, uint32_t* __restrict__ counters,
                   uint32_t dim, uint32_t k, uint32_t n, float kd, uint32_t vec4, float kd_unmoved, uint32_t* __restrict__ assignment, uint32_t data_bytes)
{
	/* the frame of the ranking (sweep_frame; the packing kernel moved the centroids): the same words for every lane, so they
	 * arrive as scalar operands. Only the ranking uses the moved coordinates; the serial arithmetic and the sums take the
	 * points as given. */
	const float* __restrict__ frame = norms + plain_frame_offset(round_up(k, TILE));
	const float frame_m2 = frame[FRAME_DIMS], frame_norm = frame[FRAME_DIMS + 1];
	constexpr uint32_t RS = DP + ROW_PAD;
	constexpr int NT = DP <= 16 ? 1 : 2;        /* tiles of 16 dimensions */
	constexpr uint32_t PARK = NT * 16 + 1;      /* a parked row: coordinates padded with zeros to whole tiles, then the result */
	constexpr uint32_t EX = DP + 1;             /* row stride of the exact centroid copy: odd, so that different rows start in different banks */
	constexpr uint32_t SUM_ROWS = MT * 16, SUM_COLS = NT * 16;
	constexpr uint32_t KEY = (1u << fused_key_bits(MT)) - 1u;
	extern __shared__ float lds[];
	__shared__ uint32_t wave_max[FUSED_WAVES];
	__shared__ uint32_t flag_list[FUSED_WAVES][2 * FUSED_FLAG_CAP];
	__shared__ uint32_t later_list[FUSED_WAVES][2 * FUSED_LATER_CAP];
	__shared__ uint32_t members[32];
	const uint32_t lane = threadIdx.x & (WAVE - 1);
	const uint32_t wave = threadIdx.x / WAVE;
	const unsigned long long lanes_below = (1ull << lane) - 1ull;

	/* LDS: [exact centroids k x EX][per wavefront: 64 parked rows, later its SUM_ROWS x SUM_COLS sums] */
	constexpr uint32_t WAVE_FLOATS = WAVE * PARK > SUM_ROWS * SUM_COLS ? WAVE * PARK : SUM_ROWS * SUM_COLS;
	float* exact = lds;
	float* parked = exact + (size_t)k * EX + (size_t)wave * WAVE_FLOATS;
	for (uint32_t i = threadIdx.x; i < k * EX; i += blockDim.x) {
		const uint32_t j = i / EX, q = i - j * EX;
		exact[i] = q < dim ? means_in[elem<LM>(stride_means, j, q)] : 0.0f;
	}
	for (uint32_t i = lane; i < WAVE * PARK; i += WAVE) parked[i] = 0.0f; /* the padding columns stay zero */
	if (threadIdx.x < 32) members[threadIdx.x] = 0u;

	uint32_t cmax = 0;
	for (uint32_t j = threadIdx.x; j < k; j += blockDim.x) cmax = max(cmax, __float_as_uint(norms[norm_at(j)]));
	for (int off = WAVE / 2; off > 0; off >>= 1) cmax = max(cmax, (uint32_t)__shfl_xor((int)cmax, off));
	if (lane == 0) wave_max[wave] = cmax;
	__syncthreads();
	cmax = 0;
	for (uint32_t w = 0; w < FUSED_WAVES; ++w) cmax = max(cmax, wave_max[w]);
	const float c2max = __uint_as_float(cmax);

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
	/* a point for the recheck queue, with the threshold its exact pass screens by (m1: its best ranking value) */
	auto flag_points = [&](bool flag, uint32_t pt, const float (&x)[DP], float m1, float tau, float x2) {
		const unsigned long long mask = __ballot(flag);
		if (!mask) return;
		const uint32_t add = (uint32_t)__builtin_popcountll(mask);
		if (flagged + add > FUSED_FLAG_CAP) flush_flags();
		if (flag) {
			const uint32_t at = 2 * (flagged + __builtin_popcountll(mask & lanes_below));
			flag_list[wave][at] = pt;
			/* the exact pass evaluates in the frame of the data (certificate.h); (x - m) . m only for these few points */
			float along = 0.0f;
#pragma unroll
			for (int q = 0; q < DP; ++q) along = __builtin_fmaf(x[q] - frame[q], frame[q], along);
			flag_list[wave][at + 1] = screening_threshold(cert_unmoved_threshold(m1, tau, x2, along, c2max, frame_m2, frame_norm, kd_unmoved), 0.0f);
		}
		flagged += add;
	};

	/* accumulators: MT x NT tiles of 16 clusters x 16 dimensions; this lane holds dimension lane % 16 of clusters
	 * 4 * (lane / 16) + 0..3 of every tile */
	f32x4v acc[MT][NT];
#pragma unroll
	for (int mt = 0; mt < MT; ++mt)
#pragma unroll
		for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = f32x4v{ 0.0f, 0.0f, 0.0f, 0.0f };
	const uint32_t col = lane & 15, quad = lane >> 4;

	auto load_point = [&](float (&x)[DP], uint32_t pt, bool valid) {
		if (LD == KMX_AOS && vec4) {
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
	};

	/* 3. park the rows (zeros for a point that is not accumulated here), then indicator x coordinates on the MFMA */
	auto accumulate = [&](const float (&x)[DP], uint32_t result) {
		const bool counted = result != UNRESOLVED;
		float* mine = parked + (size_t)lane * PARK;
#pragma unroll
		for (int q = 0; q < DP; ++q) mine[q] = counted ? x[q] : 0.0f;
		mine[NT * 16] = __uint_as_float(result);
		if (counted) atomicAdd(&members[result], 1u);
		__builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
		__builtin_amdgcn_wave_barrier();
#pragma unroll 4
		for (uint32_t s = 0; s < WAVE / 4; ++s) {
			/* this lane feeds point 4 s + quad: its membership of cluster col (A) and its coordinate col (B) */
			const float* row = parked + (size_t)(4 * s + quad) * PARK;
			const uint32_t t = __float_as_uint(row[NT * 16]);
			float b[NT];
#pragma unroll
			for (int nt = 0; nt < NT; ++nt) b[nt] = row[nt * 16 + col];
#pragma unroll
			for (int mt = 0; mt < MT; ++mt) {
				const float a = t == (uint32_t)(mt * 16) + col ? 1.0f : 0.0f;
#pragma unroll
				for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b[nt], acc[mt][nt], 0, 0, 0);
			}
		}
		__builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
		__builtin_amdgcn_wave_barrier();
	};

	/* 2. the serial arithmetic on the two leaders of the points that wait for it (rows of the exact copy in LDS, one row per
	 * lane; the points' own rows are read again): the last up to 64 entries of the list, one per lane. The sums of squares
	 * are compared first: a sum below the other by more than a 2^-21th has the strictly smaller correctly rounded root (the
	 * roots are then more than one unit in the last place apart, and two reals that far apart do not round to one float),
	 * so the square roots are taken only in between. */
	uint32_t waiting = 0; /* wave-uniform */
	auto settle_waiting = [&]() {
		__builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
		__builtin_amdgcn_wave_barrier();
		const uint32_t take = min(waiting, (uint32_t)WAVE), base = waiting - take;
		const bool have = lane < take;
		const uint32_t pt = have ? later_list[wave][2 * (base + lane)] : 0u;
		const uint32_t leaders = have ? later_list[wave][2 * (base + lane) + 1] : 0u;
		const uint32_t i1 = leaders & 0xFFu, i2 = leaders >> 8;
		float x[DP];
		load_point(x, pt, have);
		const float* c1 = exact + (size_t)i1 * EX;
		const float* c2 = exact + (size_t)i2 * EX;
		float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
		for (int q = 0; q < DP; ++q) {
			float e1 = x[q] - c1[q];
			float e2 = x[q] - c2[q];
			float q1 = e1 * e1;
			float q2 = e2 * e2;
			s1 = s1 + q1;
			s2 = s2 + q2;
		}
		constexpr float BELOW = 1.0f - 0x1p-21f, ABOVE = 1.0f + 0x1p-21f;
		bool second_wins = s2 < s1 * BELOW;
		const bool close = !second_wins && !(s2 > s1 * ABOVE);
		if (close || !(s1 > 1e-30f)) { /* ties, near-ties, sums near the subnormal range, NaN: as the serial scan compares */
			const float d1 = __builtin_sqrtf(s1), d2 = __builtin_sqrtf(s2);
			second_wins = d2 < d1 || (d2 == d1 && i2 < i1);
		}
		const uint32_t result = have ? (second_wins ? i2 : i1) : UNRESOLVED;
		if constexpr (EMIT) {
			if (have) assignment[pt] = result;
		}
		accumulate(x, result);
		waiting = base;
	};

	const uint32_t batch_points = FUSED_WAVES * WAVE;
	const uint32_t batches = (n + batch_points - 1) / batch_points;
	for (uint32_t batch = blockIdx.x; batch < batches; batch += gridDim.x) {
		if (waiting >= FUSED_LATER_DRAIN) settle_waiting(); /* before this batch's registers are live */
		const uint32_t pt = batch * batch_points + threadIdx.x;
		const bool valid = pt < n;
		float x[DP];
		load_point(x, pt, valid);
		/* 1. ranking: the three smallest keyed values; in the moved frame when the packing kernel moved the centroids (the
		 * same for the whole launch), else on the coordinates as they are. k <= 32: one tile of packed rows, RS floats apart. */
		float x2 = 0.0f; /* |x - m|^2 */
		float m1 = __builtin_inff(), m2 = __builtin_inff(), m3 = __builtin_inff();
		auto rank = [&](const float (&p)[DP]) {
#pragma unroll
			for (int q = 0; q < DP; ++q) x2 = __builtin_fmaf(p[q], p[q], x2);
			auto fetch = [&](float (&c)[DP + 1], uint32_t r) { /* uniform addresses: scalar loads */
				const float* row = packed + (size_t)r * RS;
#pragma unroll
				for (int q = 0; q < DP; ++q) c[q] = row[q];
				c[DP] = norms[r];
			};
			auto take = [&](const float (&c)[DP + 1], uint32_t r) {
				float a = c[DP];
#pragma unroll
				for (int q = 0; q < DP; ++q) a = __builtin_fmaf(c[q], p[q], a);
				const float keyed = __uint_as_float((__float_as_uint(a) & ~KEY) | r);
				m3 = __builtin_amdgcn_fmed3f(m2, m3, keyed); /* third smallest of {m1, m2, m3, keyed} as m1 <= m2 <= m3 */
				m2 = __builtin_amdgcn_fmed3f(m1, m2, keyed);
				asm("v_min_f32 %0, %1, %2" : "=v"(m1) : "v"(m1), "v"(keyed)); /* as it stands: fminf() would first canonicalise both */
			};
			for (uint32_t r = 0; r < k; ++r) {
				float c[DP + 1];
				fetch(c, r);
				take(c, r);
			}
		};
		if (frame_norm > 0.0f) {
			float xs[DP];
#pragma unroll
			for (int q = 0; q < DP; ++q) xs[q] = x[q] - frame[q];
			rank(xs);
		}
		else rank(x);
		const uint32_t i1 = __float_as_uint(m1) & KEY, i2 = __float_as_uint(m2) & KEY;

		const float span = x2 + c2max;
		const float tau = kd * span;
		const bool covered = span > 1e-30f;
		const bool decided = valid && (m2 - m1 > tau) && covered;
		const bool two = (m3 - m1 > tau) && covered;
		const uint32_t result = decided ? i1 : UNRESOLVED;
		if constexpr (EMIT) {
			if (decided) assignment[pt] = result;
		}

		/* the points with two candidates wait for the arithmetic on those (what the list cannot take goes the way of the
		 * points with three: the list has room for 32 more whenever a batch starts) */
		bool later = valid && !decided && two;
		const unsigned long long later_mask = __ballot(later);
		if (later_mask) {
			const uint32_t at = waiting + __builtin_popcountll(later_mask & lanes_below);
			later = later && at < FUSED_LATER_CAP;
			if (later) {
				later_list[wave][2 * at] = pt;
				later_list[wave][2 * at + 1] = i1 | (i2 << 8);
			}
			waiting = min(waiting + (uint32_t)__builtin_popcountll(later_mask), FUSED_LATER_CAP);
		}
		flag_points(valid && !decided && !later, pt, x, m1, tau, x2);
		accumulate(x, result);
	}
	while (waiting) settle_waiting();
	if (flagged) flush_flags();

	/* the wavefront's sums to its LDS region (row = cluster, column = dimension), then one atomic per element */
	__builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
	__builtin_amdgcn_wave_barrier();
#pragma unroll
	for (int mt = 0; mt < MT; ++mt)
#pragma unroll
		for (int nt = 0; nt < NT; ++nt)
#pragma unroll
			for (int r = 0; r < 4; ++r) parked[(size_t)(mt * 16 + 4 * quad + r) * SUM_COLS + nt * 16 + col] = acc[mt][nt][r];
	__syncthreads();
	const float* sums = exact + (size_t)k * EX;
	for (uint32_t e = threadIdx.x; e < k * dim; e += blockDim.x) {
		const uint32_t c = e / dim, d = e - c * dim;
		float s = 0.0f;
		for (uint32_t w = 0; w < FUSED_WAVES; ++w) s += sums[(size_t)w * WAVE_FLOATS + (size_t)c * SUM_COLS + d];
		if (s != 0.0f) unsafeAtomicAdd(&means_out[elem<LM>(stride_means, c, d)], s);
	}
	if (threadIdx.x < k && members[threadIdx.x]) atomicAdd(&sizes[threadIdx.x], members[threadIdx.x]);
}

/* the three smallest of the union of two ascending triples; a NaN anywhere reaches a1 */
__device__ __forceinline__ void merge_triples(float& a1, float& a2, float& a3, float b1, float b2, float b3)
{
	const float t = __builtin_elementwise_minimum(a2, b2);
	const float second = __builtin_amdgcn_fmed3f(a1, b1, t);       /* min(a1, b1) <= t: the median is min(max(a1, b1), t) */
	const float u = __builtin_elementwise_maximum(__builtin_elementwise_maximum(a1, b1), t);
	const float w = __builtin_elementwise_minimum(__builtin_elementwise_minimum(__builtin_elementwise_maximum(a2, b2), a3), b3);
	a1 = __builtin_elementwise_minimum(a1, b1);
	a2 = second;
	a3 = __builtin_elementwise_minimum(u, w);
}

/* v_permlane16_swap: rows 1 and 3 (lanes 16-31, 48-63) of a change places with rows 0 and 2 of b;
 * v_permlane32_swap: rows 2 and 3 of a change places with rows 0 and 1 of b */
__device__ __forceinline__ void swap_rows16(float& a, float& b)
{
	const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
	a = __uint_as_float(r[0]); b = __uint_as_float(r[1]);
}
__device__ __forceinline__ void swap_rows32(float& a, float& b)
{
	const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(b), false, false);
	a = __uint_as_float(r[0]); b = __uint_as_float(r[1]);
}

/* The same iteration with the ranking on the matrix cores as well: a[j] for 16 points x 16 centroids is one chain of
 * v_mfma_f32_16x16x4_f32 (centroids as the rows of A, held in registers for the whole kernel; points as the columns of B;
 * the accumulator started from the norms). Lane (col, quad) = (lane % 16, lane / 16) loads the 16-byte piece `quad` of
 * every 64-byte chunk of the rows of points 16 g + col, g = 0..3: one coalesced 128-bit load per group, and exactly the B
 * operand of four instructions (the order of the dimensions inside a chain is free as long as A uses the same). It then
 * holds the values of centroids 4 quad + 0..3 (of every tile of 16) for those four points; the four lanes of a point
 * merge their three smallest keyed values in two exchanges of register rows, laid out so that lane l ends up with point l
 * of the batch: from there on one lane owns one point, as in the decision, the lists and the stores. */
template <int DP, int LD, int LM, int MT, bool EMIT, bool VEC>
__global__ void __launch_bounds__(FUSED_WAVES * WAVE) __attribute__((amdgpu_waves_per_eu(DP == 16 && MT == 1 ? 4 : 1)))
fused_matrix_kernel(const float* __restrict__ data, size_t stride, const float* __restrict__ packed, const float* __restrict__ norms,
                    const float* __restrict__ means_in, size_t stride_means,
                    float* __restrict__ means_out, uint32_t* __restrict__ sizes,
                    uint32_t* __restrict__ queue, uint32_t* __restrict__ counters,
                    uint32_t dim, uint32_t k, uint32_t n, float kd, uint32_t vec4, float kd_unmoved, uint32_t* __restrict__ assignment, uint32_t data_bytes)
{
	const float* __restrict__ frame = norms + plain_frame_offset(round_up(k, TILE));
	const float frame_m2 = frame[FRAME_DIMS], frame_norm = frame[FRAME_DIMS + 1];
	constexpr uint32_t RS = DP + ROW_PAD;
	constexpr int CH = (DP + 15) / 16;          /* chunks of 16 dimensions: one 16-byte piece per quad */
	constexpr bool DEEP = CH == 1;              /* two batches of rows requested ahead (their pieces wait in registers) */
	constexpr uint32_t AHEAD = DEEP ? 2 : 1;
	constexpr int NT = CH;                      /* tiles of 16 dimensions of the sums */
	constexpr uint32_t PARK = NT * 16 + 2;      /* a parked row: coordinates padded with zeros to whole tiles; rows 8 apart start 16 banks apart */
	constexpr uint32_t EX = DP + 1;             /* row stride of the exact centroid copy: odd, so that different rows start in different banks */
	constexpr uint32_t SUM_ROWS = MT * 16, SUM_COLS = NT * 16;
	constexpr uint32_t KEY = (1u << fused_key_bits(MT)) - 1u;
	extern __shared__ float lds[];
	__shared__ uint32_t wave_max[FUSED_WAVES];
	__shared__ uint32_t flag_list[FUSED_WAVES][2 * FUSED_FLAG_CAP];
	__shared__ uint32_t later_list[FUSED_WAVES][2 * FUSED_LATER_CAP];
	__shared__ uint32_t members[32];
	__shared__ __attribute__((aligned(16))) float start_norms[32]; /* what the ranking chains start from */
	const uint32_t lane = threadIdx.x & (WAVE - 1);
	const uint32_t wave = threadIdx.x / WAVE;
	const uint32_t col = lane & 15, quad = lane >> 4;
	/* how many of the lanes below this one are set in a mask */
	auto below = [](unsigned long long mask) -> uint32_t {
		return __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
	};

	/* LDS: [exact centroids k x EX][per wavefront: 64 parked rows, later its SUM_ROWS x SUM_COLS sums; SUM_ROWS rows of 64
	 * membership halfwords: bf16 1.0 at a point's place in its cluster's row while its batch is summed, zeros otherwise] */
	constexpr uint32_t WAVE_FLOATS = fused_matrix_wave_floats(NT, MT);
	float* exact = lds;
	float* parked = exact + (size_t)k * EX + (size_t)wave * WAVE_FLOATS;
	unsigned short* member_of = (unsigned short*)(parked + (WAVE * PARK > SUM_ROWS * SUM_COLS ? WAVE * PARK : SUM_ROWS * SUM_COLS));
	for (uint32_t i = threadIdx.x; i < k * EX; i += blockDim.x) {
		const uint32_t j = i / EX, q = i - j * EX;
		exact[i] = q < dim ? means_in[elem<LM>(stride_means, j, q)] : 0.0f;
	}
	for (uint32_t i = lane; i < WAVE_FLOATS; i += WAVE) parked[i] = 0.0f; /* the padding columns and the membership words stay zero */
	if (threadIdx.x < 32) {
		members[threadIdx.x] = 0u;
		/* rows past k never win: a large finite norm (an infinity would turn into a NaN under the key) */
		start_norms[threadIdx.x] = threadIdx.x < k ? norms[threadIdx.x] : 3.0e38f;
	}

	uint32_t cmax = 0;
	for (uint32_t j = threadIdx.x; j < k; j += blockDim.x) cmax = max(cmax, __float_as_uint(norms[norm_at(j)]));
	for (int off = WAVE / 2; off > 0; off >>= 1) cmax = max(cmax, (uint32_t)__shfl_xor((int)cmax, off));
	if (lane == 0) wave_max[wave] = cmax;
	__syncthreads();
	cmax = 0;
	for (uint32_t w = 0; w < FUSED_WAVES; ++w) cmax = max(cmax, wave_max[w]);
	const float c2max = __uint_as_float(cmax);

	/* the operands that stay: this lane's pieces of centroid rows mt * 16 + col (A) and of the frame, and the numbers of
	 * centroids mt * 16 + 4 quad + 0..3 (the rows of D this lane holds; their norms are read from LDS where a chain
	 * starts). k <= 32: one tile of packed rows, RS floats apart. */
	float ca[MT][CH][4], fr[CH][4];
	uint32_t key[MT][4];
#pragma unroll
	for (int j = 0; j < CH; ++j)
#pragma unroll
		for (int e = 0; e < 4; ++e) {
			const uint32_t q = 16 * j + 4 * quad + e;
			fr[j][e] = (q < (uint32_t)DP && frame_norm > 0.0f) ? frame[q] : 0.0f;
#pragma unroll
			for (int mt = 0; mt < MT; ++mt) {
				const uint32_t r = mt * 16 + col;
				ca[mt][j][e] = (q < (uint32_t)DP && r < k) ? packed[(size_t)r * RS + q] : 0.0f;
			}
		}
#pragma unroll
	for (int mt = 0; mt < MT; ++mt)
#pragma unroll
		for (int i = 0; i < 4; ++i) {
			key[mt][i] = mt * 16 + 4 * quad + i;
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

	/* sums: MT x NT tiles of 16 clusters x 16 dimensions; this lane holds dimension col of clusters 4 quad + 0..3 of every tile */
	f32x4v acc[MT][NT];
#pragma unroll
	for (int mt = 0; mt < MT; ++mt)
#pragma unroll
		for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = f32x4v{ 0.0f, 0.0f, 0.0f, 0.0f };

	/* one lane per point: the whole row (the points that are settled later, the points for the recheck queue) */
	auto load_row = [&](float (&x)[DP], uint32_t pt, bool valid) {
		if (LD == KMX_AOS && vec4) {
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
	};

	/* 3. the parked rows (row l: point l of the batch, zeros unless it is accumulated here): membership x coordinates on the
	 * bf16 matrix instruction (v_mfma_f32_16x16x32_bf16: 32 points per instruction, sixteen times the rate of the fp32 one,
	 * and it runs beside the vector ALU, which the fp32 one does not). A coordinate is the exact sum of three bf16 values --
	 * its upper 16 bits, the upper 16 bits of what that leaves, and the rest, at most 8 significant bits each -- and
	 * 1.0 * part is exact, so the three products add up to the coordinate in the fp32 accumulator as 1.0 * x did; only the
	 * order of the additions differs from the serial one (parts below 2^-126 are flushed by the instruction: far below
	 * the tolerance of any sum). This lane feeds dimension col of points 32 blk + 8 quad + 0..7 (B) and their membership
	 * of cluster col (A). */
	auto add_parked = [&](uint32_t result) {
		const bool counted = result != UNRESOLVED;
		unsigned short* mine = member_of + (size_t)(counted ? result : 0u) * WAVE + lane;
		if (counted) {
			*mine = 0x3F80u; /* bf16 1.0 */
			atomicAdd(&members[result], 1u);
		}
		__builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
		__builtin_amdgcn_wave_barrier();
#pragma unroll
		for (uint32_t blk = 0; blk < 2; ++blk) {
			bf16x8 hi[NT], mid[NT], lo[NT];
#pragma unroll
			for (int nt = 0; nt < NT; ++nt) {
				uint32_t ph[8], pm[8], pl[8];
#pragma unroll
				for (int i = 0; i < 8; ++i) {
					const float v = parked[(size_t)(32 * blk + 8 * quad + i) * PARK + nt * 16 + col];
					ph[i] = __float_as_uint(v) & 0xFFFF0000u;
					const float r = v - __uint_as_float(ph[i]);
					pm[i] = __float_as_uint(r) & 0xFFFF0000u;
					pl[i] = __float_as_uint(r - __uint_as_float(pm[i]));
				}
				u32x4 wh, wm, wl; /* the upper halves of two words side by side: __builtin_amdgcn_perm(hi word, lo word, selector) */
#pragma unroll
				for (int i = 0; i < 4; ++i) {
					wh[i] = __builtin_amdgcn_perm(ph[2 * i + 1], ph[2 * i], 0x07060302u);
					wm[i] = __builtin_amdgcn_perm(pm[2 * i + 1], pm[2 * i], 0x07060302u);
					wl[i] = __builtin_amdgcn_perm(pl[2 * i + 1], pl[2 * i], 0x07060302u);
				}
				hi[nt] = __builtin_bit_cast(bf16x8, wh);
				mid[nt] = __builtin_bit_cast(bf16x8, wm);
				lo[nt] = __builtin_bit_cast(bf16x8, wl);
			}
#pragma unroll
			for (int mt = 0; mt < MT; ++mt) {
				const bf16x8 in = *(const bf16x8*)(member_of + (size_t)(mt * 16 + col) * WAVE + 32 * blk + 8 * quad);
#pragma unroll
				for (int nt = 0; nt < NT; ++nt) {
					acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(in, hi[nt], acc[mt][nt], 0, 0, 0);
					acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(in, mid[nt], acc[mt][nt], 0, 0, 0);
					acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(in, lo[nt], acc[mt][nt], 0, 0, 0);
				}
			}
		}
		__builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
		__builtin_amdgcn_wave_barrier();
		if (counted) *mine = 0u;
	};

	/* 2. the serial arithmetic on the two leaders of the points that wait for it (rows of the exact copy in LDS, one row per
	 * lane; the points' own rows are read again): the last up to 64 entries of the list, one per lane. The sums of squares
	 * are compared first: a sum below the other by more than a 2^-21th has the strictly smaller correctly rounded root (the
	 * roots are then more than one unit in the last place apart, and two reals that far apart do not round to one float),
	 * so the square roots are taken only in between. */
	uint32_t waiting = 0; /* wave-uniform */
	auto settle_waiting = [&]() {
		__builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
		__builtin_amdgcn_wave_barrier();
		const uint32_t take = min(waiting, (uint32_t)WAVE), base = waiting - take;
		const bool have = lane < take;
		const uint32_t pt = have ? later_list[wave][2 * (base + lane)] : 0u;
		const uint32_t leaders = have ? later_list[wave][2 * (base + lane) + 1] : 0u;
		const uint32_t i1 = leaders & 0xFFu, i2 = leaders >> 8;
		float x[DP];
		load_row(x, pt, have);
		const float* c1 = exact + (size_t)i1 * EX;
		const float* c2 = exact + (size_t)i2 * EX;
		float s1 = 0.0f, s2 = 0.0f;
#pragma unroll
		for (int q = 0; q < DP; ++q) {
			float e1 = x[q] - c1[q];
			float e2 = x[q] - c2[q];
			float q1 = e1 * e1;
			float q2 = e2 * e2;
			s1 = s1 + q1;
			s2 = s2 + q2;
		}
		constexpr float BELOW = 1.0f - 0x1p-21f, ABOVE = 1.0f + 0x1p-21f;
		bool second_wins = s2 < s1 * BELOW;
		const bool close = !second_wins && !(s2 > s1 * ABOVE);
		if (close || !(s1 > 1e-30f)) { /* ties, near-ties, sums near the subnormal range, NaN: as the serial scan compares */
			const float d1 = __builtin_sqrtf(s1), d2 = __builtin_sqrtf(s2);
			second_wins = d2 < d1 || (d2 == d1 && i2 < i1);
		}
		const uint32_t result = have ? (second_wins ? i2 : i1) : UNRESOLVED;
		if constexpr (EMIT) {
			if (have) assignment[pt] = result;
		}
		float* mine = parked + (size_t)lane * PARK;
#pragma unroll
		for (int q = 0; q < DP; ++q) mine[q] = have ? x[q] : 0.0f;
		add_parked(result);
		waiting = base;
	};

	const uint32_t batch_points = FUSED_WAVES * WAVE;
	const uint32_t batches = (n + batch_points - 1) / batch_points;
	/* the pieces of the rows of points first + 16 g + col of a batch, requested through a buffer descriptor of the whole
	 * array: a read past its end returns zeros, so the requests need no branches and stay in flight across the work on
	 * the batch before. AoS rows past n lie past the end; SoA points past n get an offset that does; a `dead` batch (past
	 * the last) reads through a descriptor of no bytes. */
	const uint32_t stride32 = (uint32_t)stride;
	auto load_pieces = [&](uint32_t (&x)[4][CH][4], uint32_t batch, bool dead) {
		const uint32_t first = batch * batch_points + wave * WAVE; /* n <= 2^31: no overflow */
		const __amdgpu_buffer_rsrc_t rows = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(data), 0, dead ? 0u : data_bytes, 0x00020000);
		if constexpr (VEC) { /* AoS rows, 16-byte pieces */
#pragma unroll
			for (int g = 0; g < 4; ++g)
#pragma unroll
				for (int j = 0; j < CH; ++j) {
					const uint32_t at = ((first + 16 * g + col) * stride32 + 16 * j + 4 * quad) * 4u;
					const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rows, at, 0, 0);
					x[g][j][0] = v.x; x[g][j][1] = v.y; x[g][j][2] = v.z; x[g][j][3] = v.w;
				}
		}
		else {
#pragma unroll
			for (int g = 0; g < 4; ++g) {
				const uint32_t p = first + 16 * g + col;
				const bool none = LD == KMX_SOA && p >= n;
#pragma unroll
				for (int j = 0; j < CH; ++j)
#pragma unroll
					for (int e = 0; e < 4; ++e) {
						const uint32_t q = 16 * j + 4 * quad + e;
						const uint32_t at = none ? 0xFFFFFFF0u : (LD == KMX_AOS ? p * stride32 + q : q * stride32 + p) * 4u;
						x[g][j][e] = __builtin_amdgcn_raw_buffer_load_b32(rows, at, 0, 0);
					}
			}
		}
	};
	const bool padded = dim < (uint32_t)DP; /* then the pieces hold words of other rows past `dim` */
	/* one batch whose pieces have been requested into `ahead`; the same registers then take the batch two further on */
	auto batch_step = [&](uint32_t (&ahead)[4][CH][4], uint32_t batch) {
		if (waiting >= FUSED_LATER_DRAIN) settle_waiting(); /* before this batch's registers are live */
		const uint32_t first = batch * batch_points + wave * WAVE;
		float x[4][CH][4];
#pragma unroll
		for (int g = 0; g < 4; ++g)
#pragma unroll
			for (int j = 0; j < CH; ++j)
#pragma unroll
				for (int e = 0; e < 4; ++e) x[g][j][e] = __uint_as_float(ahead[g][j][e]);
		if (padded) {
#pragma unroll
			for (int g = 0; g < 4; ++g)
#pragma unroll
				for (int j = 0; j < CH; ++j)
#pragma unroll
					for (int e = 0; e < 4; ++e)
						if (16 * j + 4 * quad + e >= dim) x[g][j][e] = 0.0f;
		}
		/* park the pieces as they are; the rows of the points that are not accumulated here are cleared below */
#pragma unroll
		for (int g = 0; g < 4; ++g)
#pragma unroll
			for (int j = 0; j < CH; ++j)
#pragma unroll
				for (int e = 0; e < 4; ++e)
					if (16 * j + 4 * quad + e < (uint32_t)DP) parked[(size_t)(16 * g + col) * PARK + 16 * j + 4 * quad + e] = x[g][j][e];
		/* 1. ranking in the frame of the sweep; per group the lane's three smallest keyed values and its share of |x - m|^2.
		 * The four lanes of a point then meet: rows of registers change places so that every merge has one lane's values on
		 * either side; after the second exchange quad q holds group q, that is lane l holds point first + l. */
		float m1[4], m2[4], m3[4], x2[4];
		auto rank_pair = [&](auto in_frame, int g0) {
#pragma unroll
			for (int g = g0; g < g0 + 2; ++g) {
				f32x4v d[MT];
#pragma unroll
				for (int mt = 0; mt < MT; ++mt) d[mt] = *(const f32x4v*)(start_norms + mt * 16 + 4 * quad);
				float sq = 0.0f;
#pragma unroll
				for (int j = 0; j < CH; ++j)
#pragma unroll
					for (int e = 0; e < 4; ++e) {
						const float xs = decltype(in_frame)::value ? x[g][j][e] - fr[j][e] : x[g][j][e];
						sq = __builtin_fmaf(xs, xs, sq);
#pragma unroll
						for (int mt = 0; mt < MT; ++mt) d[mt] = __builtin_amdgcn_mfma_f32_16x16x4f32(ca[mt][j][e], xs, d[mt], 0, 0, 0);
					}
				x2[g] = sq;
				float v[MT * 4];
#pragma unroll
				for (int mt = 0; mt < MT; ++mt)
#pragma unroll
					for (int i = 0; i < 4; ++i) v[mt * 4 + i] = __uint_as_float((__float_as_uint(d[mt][i]) & ~KEY) | key[mt][i]);
				float lo = __builtin_elementwise_minimum(__builtin_elementwise_minimum(v[0], v[1]), v[2]);
				float mid = __builtin_amdgcn_fmed3f(v[0], v[1], v[2]);
				float hi = __builtin_elementwise_maximum(__builtin_elementwise_maximum(v[0], v[1]), v[2]);
#pragma unroll
				for (int i = 3; i < MT * 4; ++i) { /* lo <= mid <= hi and one more value */
					hi = __builtin_amdgcn_fmed3f(mid, hi, v[i]);
					mid = __builtin_amdgcn_fmed3f(lo, mid, v[i]);
					lo = __builtin_elementwise_minimum(lo, v[i]);
				}
				m1[g] = lo; m2[g] = mid; m3[g] = hi;
			}
			swap_rows16(m1[g0], m1[g0 + 1]); swap_rows16(m2[g0], m2[g0 + 1]); swap_rows16(m3[g0], m3[g0 + 1]); swap_rows16(x2[g0], x2[g0 + 1]);
			merge_triples(m1[g0], m2[g0], m3[g0], m1[g0 + 1], m2[g0 + 1], m3[g0 + 1]);
			x2[g0] += x2[g0 + 1];
		};
		if (frame_norm > 0.0f) { rank_pair(std::true_type{}, 0); rank_pair(std::true_type{}, 2); }
		else { rank_pair(std::false_type{}, 0); rank_pair(std::false_type{}, 2); }
		swap_rows32(m1[0], m1[2]); swap_rows32(m2[0], m2[2]); swap_rows32(m3[0], m3[2]); swap_rows32(x2[0], x2[2]);
		merge_triples(m1[0], m2[0], m3[0], m1[2], m2[2], m3[2]);
		const float best = m1[0], second = m2[0], third = m3[0];
		const float xx = x2[0] + x2[2];

		const uint32_t pt = first + lane;
		const bool valid = pt < n;
		const uint32_t i1 = __float_as_uint(best) & KEY, i2 = __float_as_uint(second) & KEY;
		const float span = xx + c2max;
		const float tau = kd * span;
		const bool covered = span > 1e-30f;
		const bool decided = valid && (second - best > tau) && covered;
		const bool two = (third - best > tau) && covered;
		const uint32_t result = decided ? i1 : UNRESOLVED;
		if constexpr (EMIT) {
			/* whole lines: the lanes without a result store UNRESOLVED, which the wavefront (settle_waiting) or the exact pass
			 * overwrites later. Through a descriptor of the n results: the lanes past n aim past its end, where stores are
			 * dropped. (What the output costs is the stores themselves, not the code around them: N = 16.7M, d = 16, one
			 * GPU, the kernel compiled with the output and the stores replaced by statements that only keep their operands
			 * alive: 0.249 ms as without the output; these stores alone 0.276 ms; those of settle_waiting alone 0.272 ms;
			 * both 0.285 ms. 64 MB written next to 1.07 GB read cost as much as 110 MB of reads -- a copy runs at three
			 * quarters of the bandwidth of a read on this memory as well -- and the results of the points settled later,
			 * 5 % of all, as much again when they stand alone: a word stored into a line that has left the caches makes the
			 * memory read and write the line. Holding the lines back in LDS until their last point is settled takes those
			 * away (0.278 ms) but costs 3 to 10 % on data with few or very many such points, and was dropped.) */
			const __amdgpu_buffer_rsrc_t results = __builtin_amdgcn_make_buffer_rsrc(assignment, 0, n * 4u, 0x00020000);
			__builtin_amdgcn_raw_buffer_store_b32(result, results, pt * 4u, 0, 0);
		}
		/* the next requests into the registers of this batch (x is not read past this line) */
		load_pieces(ahead, batch + AHEAD * gridDim.x, batch + AHEAD * gridDim.x >= batches);

		/* the points with two candidates wait for the arithmetic on those (what the list cannot take goes the way of the
		 * points with three: the list has room for 32 more whenever a batch starts) */
		bool later = valid && !decided && two;
		const unsigned long long later_mask = __ballot(later);
		if (later_mask) {
			const uint32_t at = waiting + below(later_mask);
			later = later && at < FUSED_LATER_CAP;
			if (later) {
				later_list[wave][2 * at] = pt;
				later_list[wave][2 * at + 1] = i1 | (i2 << 8);
			}
			waiting = min(waiting + (uint32_t)__builtin_popcountll(later_mask), FUSED_LATER_CAP);
		}
		const bool flag = valid && !decided && !later;
		const unsigned long long flag_mask = __ballot(flag);
		if (flag_mask) {
			const uint32_t add = (uint32_t)__builtin_popcountll(flag_mask);
			if (flagged + add > FUSED_FLAG_CAP) flush_flags();
			if (flag) {
				const uint32_t at = 2 * (flagged + below(flag_mask));
				flag_list[wave][at] = pt;
				/* the exact pass evaluates in the frame of the data (certificate.h); (x - m) . m only for these few points,
				 * from their rows in memory */
				float along = 0.0f;
				for (uint32_t q = 0; q < dim; ++q) along = __builtin_fmaf(data[elem<LD>(stride, pt, q)] - frame[q], frame[q], along);
				flag_list[wave][at + 1] = screening_threshold(cert_unmoved_threshold(best, tau, xx, along, c2max, frame_m2, frame_norm, kd_unmoved), 0.0f);
			}
			flagged += add;
		}
		if (__ballot(!decided)) {
			if (!decided) {
				float* mine = parked + (size_t)lane * PARK;
#pragma unroll
				for (int q = 0; q < DP; ++q) mine[q] = 0.0f;
			}
		}
		add_parked(result);
	};
	/* one batch, or with rows of up to 16 floats two, on their way while another is worked on: what a compute unit keeps in
	 * flight, not its arithmetic, decides how much of the memory's bandwidth it sees */
	if constexpr (DEEP) {
		uint32_t even[4][CH][4], odd[4][CH][4];
		load_pieces(even, blockIdx.x, blockIdx.x >= batches);
		load_pieces(odd, blockIdx.x + gridDim.x, blockIdx.x + gridDim.x >= batches);
		for (uint32_t batch = blockIdx.x; batch < batches; batch += 2 * gridDim.x) {
			batch_step(even, batch);
			if (batch + gridDim.x < batches) batch_step(odd, batch + gridDim.x);
		}
	}
	else {
		uint32_t ahead[4][CH][4];
		load_pieces(ahead, blockIdx.x, blockIdx.x >= batches);
		for (uint32_t batch = blockIdx.x; batch < batches; batch += gridDim.x) batch_step(ahead, batch);
	}
	while (waiting) settle_waiting();
	if (flagged) flush_flags();

	/* the wavefront's sums to its LDS region (row = cluster, column = dimension), then one atomic per element */
	__builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
	__builtin_amdgcn_wave_barrier();
#pragma unroll
	for (int mt = 0; mt < MT; ++mt)
#pragma unroll
		for (int nt = 0; nt < NT; ++nt)
#pragma unroll
			for (int r = 0; r < 4; ++r) parked[(size_t)(mt * 16 + 4 * quad + r) * SUM_COLS + nt * 16 + col] = acc[mt][nt][r];
	__syncthreads();
	const float* sums = exact + (size_t)k * EX;
	for (uint32_t e = threadIdx.x; e < k * dim; e += blockDim.x) {
		const uint32_t c = e / dim, d = e - c * dim;
		float s = 0.0f;
		for (uint32_t w = 0; w < FUSED_WAVES; ++w) s += sums[(size_t)w * WAVE_FLOATS + (size_t)c * SUM_COLS + d];
		if (s != 0.0f) unsafeAtomicAdd(&means_out[elem<LM>(stride_means, c, d)], s);
	}
	if (threadIdx.x < k && members[threadIdx.x]) atomicAdd(&sizes[threadIdx.x], members[threadIdx.x]);
}

/* adds the points the exact pass has just resolved (the queue of the fused kernel) to the sums and counts: every
 * work-group gathers its share in LDS first, so the few hundred result words see one global atomic per work-group */
template <int LD, int LM>
__global__ void __launch_bounds__(256)
fused_fixup_kernel(const float* __restrict__ data, size_t stride, const uint32_t* __restrict__ assignment,
                   float* __restrict__ means_out, size_t stride_means, uint32_t* __restrict__ sizes,
                   const uint32_t* __restrict__ queue, const uint32_t* __restrict__ counters, uint32_t dim, uint32_t k)
{
	__shared__ float sums[32 * 32];
	__shared__ uint32_t members[32];
	const uint32_t count = counters[0];
	if ((uint64_t)blockIdx.x * blockDim.x >= (uint64_t)count * dim) return; /* nothing for this work-group */
	for (uint32_t i = threadIdx.x; i < k * dim; i += blockDim.x) sums[i] = 0.0f;
	if (threadIdx.x < 32) members[threadIdx.x] = 0u;
	__syncthreads();
	const uint64_t total = (uint64_t)count * dim;
	for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (uint64_t)gridDim.x * blockDim.x) {
		const uint32_t entry = (uint32_t)(i / dim), d = (uint32_t)(i - (uint64_t)entry * dim);
		const uint32_t pt = queue[2 * (size_t)entry];
		const uint32_t t = assignment[pt];
		unsafeAtomicAdd(&sums[t * dim + d], data[elem<LD>(stride, pt, d)]);
		if (d == 0) atomicAdd(&members[t], 1u);
	}
	__syncthreads();
	for (uint32_t e = threadIdx.x; e < k * dim; e += blockDim.x) {
		const uint32_t c = e / dim, d = e - c * dim;
		if (sums[e] != 0.0f) unsafeAtomicAdd(&means_out[elem<LM>(stride_means, c, d)], sums[e]);
	}
	if (threadIdx.x < k && members[threadIdx.x]) atomicAdd(&sizes[threadIdx.x], members[threadIdx.x]);
}

/* the padded row widths whose ranking runs on the matrix cores (fused_matrix_kernel): measured against the lane-per-point
 * kernel on one MI355X, rows of 16 and 32 floats gain a quarter, rows of 8 are level, rows of 4 lose (the chains of four
 * dimensions per instruction run three quarters empty) and rows of 24 lose a few per cent */
constexpr bool fused_matrix_rows(uint32_t dp) { return dp == 8 || dp == 16 || dp == 32; }

static uint32_t fused_dp(uint32_t dim)
{
	for (uint32_t o : { 4u, 8u, 16u, 24u, 32u })
		if (dim <= o) return o;
	return 0;
}

bool fused_small_supports(uint32_t dim, uint32_t k, int layout, size_t stride, uint32_t n)
{
	const size_t data_bytes = (layout == KMX_AOS ? (size_t)n * stride : (size_t)dim * stride) * sizeof(float);
	return k <= 32 && fused_dp(dim) != 0 && data_bytes <= FUSED_MAX_DATA_BYTES;
}

template <int DP, int LD, int LM>
static int launch_fused_t(const AssignArgs& a, float* means_out, uint32_t* sizes, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev, float kd)
{
	constexpr uint32_t NT = DP <= 16 ? 1 : 2;
	const uint32_t mt = a.k <= 16 ? 1 : 2;
	const uint32_t wave_floats = std::max<uint32_t>(WAVE * (NT * 16 + 1), mt * 16 * NT * 16);
	const uint32_t lds_bytes = (a.k * (DP + 1) + FUSED_WAVES * (fused_matrix_rows(DP) ? fused_matrix_wave_floats(NT, mt) : wave_floats)) * 4;
	const uint32_t static_bytes = (2 * (FUSED_FLAG_CAP + FUSED_LATER_CAP) * FUSED_WAVES + 128 + 32) * 4;
	if (lds_bytes + static_bytes > dev.lds_bytes) return fail(KMX_ERR_UNSUPPORTED, "fused iteration: %u bytes of LDS needed", lds_bytes + static_bytes);
	void (*kernel)(const float*, size_t, const float*, const float*, const float*, size_t, float*, uint32_t*, uint32_t*, uint32_t*,
	               uint32_t, uint32_t, uint32_t, float, uint32_t, float, uint32_t*, uint32_t) = nullptr;
	const uint32_t vec4 = (a.layout == KMX_AOS && a.dim % 4 == 0 && a.stride % 4 == 0 && ((uintptr_t)a.data % 16) == 0) ? 1u : 0u;
	if constexpr (fused_matrix_rows(DP)) {
		if (LD == KMX_AOS && vec4)
			kernel = a.emit_assignment ? (mt == 1 ? fused_matrix_kernel<DP, KMX_AOS, LM, 1, true, true> : fused_matrix_kernel<DP, KMX_AOS, LM, 2, true, true>)
			                           : (mt == 1 ? fused_matrix_kernel<DP, KMX_AOS, LM, 1, false, true> : fused_matrix_kernel<DP, KMX_AOS, LM, 2, false, true>);
		else
			kernel = a.emit_assignment ? (mt == 1 ? fused_matrix_kernel<DP, LD, LM, 1, true, false> : fused_matrix_kernel<DP, LD, LM, 2, true, false>)
			                           : (mt == 1 ? fused_matrix_kernel<DP, LD, LM, 1, false, false> : fused_matrix_kernel<DP, LD, LM, 2, false, false>);
	}
	else {
		kernel = a.emit_assignment ? (mt == 1 ? fused_small_kernel<DP, LD, LM, 1, true> : fused_small_kernel<DP, LD, LM, 2, true>)
		                           : (mt == 1 ? fused_small_kernel<DP, LD, LM, 1, false> : fused_small_kernel<DP, LD, LM, 2, false>);
	}
	const uint32_t batches = (a.n + FUSED_WAVES * WAVE - 1) / (FUSED_WAVES * WAVE);
	const size_t data_bytes = (a.layout == KMX_AOS ? (size_t)a.n * a.stride : (size_t)a.dim * a.stride) * sizeof(float);
	if (data_bytes > FUSED_MAX_DATA_BYTES) return fail(KMX_ERR_UNSUPPORTED, "fused iteration: the single-pass kernel takes up to %zu bytes of points", (size_t)FUSED_MAX_DATA_BYTES);
	/* as many work-groups as the device holds at once (registers and LDS decide): every one of them takes its share of the batches */
	int resident = 0;
	if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&resident, reinterpret_cast<const void*>(kernel), FUSED_WAVES * WAVE, lds_bytes) != hipSuccess || resident < 1) {
		(void)hipGetLastError();
		resident = 1;
	}
	const uint32_t grid = std::min(batches, dev.compute_units * (uint32_t)resident);
	exec->block_count = grid;
	int rc = profile_begin(0);
	if (rc) return rc;
	KMX_LAUNCH_KERNEL(kernel, dim3(grid), dim3(FUSED_WAVES * WAVE), lds_bytes, stream(),
	                   a.data, a.stride, ws->packed_means, ws->norms, a.means, a.stride_means, means_out, sizes,
	                   ws->queue, ws->counters, a.dim, a.k, a.n, kd, vec4, cert_kd_unmoved(a.dim), a.assignment, (uint32_t)data_bytes);
	KMX_LAUNCH_CHECK("fused_small_kernel");
	return profile_end(0);
}

template <int LD, int LM>
static int launch_fused_layouts(const AssignArgs& a, float* means_out, uint32_t* sizes, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev)
{
	const uint32_t dp = fused_dp(a.dim);
	const uint32_t kp = round_up(a.k, TILE);
	/* the ranking works in a frame moved to the middle of the centroids when they lie far from the origin */
	int rc = launch_pack_means(a, ws, dp, kp, FRAME_MOVED_IF_FAR);
	if (rc) return rc;
	/* the bound of a ranking by chains of fused multiply-adds, or by the fp32 matrix instruction, see certificate.h;
	 * 8 * 2^-23 for the roundings of x - m, c - m; the low bits of the values carry the centroid's number */
	const float kd = (fused_matrix_rows(dp) ? cert_kd_fp32(a.dim) : cert_kd_fma(a.dim)) + 8.0f * CERT_UNIT + cert_kd_keyed(fused_key_bits(a.k <= 16 ? 1 : 2));
	switch (dp) {
	case 4: rc = launch_fused_t<4, LD, LM>(a, means_out, sizes, exec, ws, dev, kd); break;
	case 8: rc = launch_fused_t<8, LD, LM>(a, means_out, sizes, exec, ws, dev, kd); break;
	case 16: rc = launch_fused_t<16, LD, LM>(a, means_out, sizes, exec, ws, dev, kd); break;
	case 24: rc = launch_fused_t<24, LD, LM>(a, means_out, sizes, exec, ws, dev, kd); break;
	case 32: rc = launch_fused_t<32, LD, LM>(a, means_out, sizes, exec, ws, dev, kd); break;
	default: return fail(KMX_ERR_UNSUPPORTED, "fused iteration: dim %u is not supported by the single-pass kernel", a.dim);
	}
	if (rc) return rc;
	/* the unresolved points: exact pass into the work-space assignment vector, then their share of the sums */
	ws->exact_norms = ws->norms + plain_exact_norms_offset(kp);
	rc = launch_recheck(a, ws, kp);
	ws->exact_norms = nullptr;
	if (rc) return rc;
	KMX_LAUNCH_KERNEL((fused_fixup_kernel<LD, LM>), dim3(64), dim3(256), 0, stream(),
	                   a.data, a.stride, a.assignment, means_out, a.stride_means, sizes, ws->queue, ws->counters, a.dim, a.k);
	KMX_LAUNCH_CHECK("fused_fixup_kernel");
	return KMX_OK;
}

/* a.assignment: a vector of n entries -- the work-space vector (only the entries of the points left to the exact pass are
 * written), or with a.emit_assignment the caller's, which then receives every point's result; means_out and sizes are zero
 * on entry; the caller divides */
int launch_fused_small(const AssignArgs& a, float* means_out, uint32_t* sizes, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev)
{
	if (a.layout == KMX_AOS && a.layout_means == KMX_AOS) return launch_fused_layouts<KMX_AOS, KMX_AOS>(a, means_out, sizes, exec, ws, dev);
	if (a.layout == KMX_AOS && a.layout_means == KMX_SOA) return launch_fused_layouts<KMX_AOS, KMX_SOA>(a, means_out, sizes, exec, ws, dev);
	if (a.layout == KMX_SOA && a.layout_means == KMX_AOS) return launch_fused_layouts<KMX_SOA, KMX_AOS>(a, means_out, sizes, exec, ws, dev);
	return launch_fused_layouts<KMX_SOA, KMX_SOA>(a, means_out, sizes, exec, ws, dev);
}

} // namespace kmx
