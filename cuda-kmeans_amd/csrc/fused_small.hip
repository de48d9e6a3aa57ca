/*
 * One whole iteration in a single pass over the points, for a handful of centroids (k <= 32, rows up to 32
 * floats): the shapes where the iteration is bound by HBM and reading the points twice (assignment, then
 * update) costs the most. Role of the reference's fused kernels (kernels.cu:883-1190).
 *
 * One lane owns one point, its coordinates in registers.
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
 * Floating-point contraction is off for the whole file (the serial arithmetic must not fuse); the ranking uses
 * explicit fused multiply-adds.
 */
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
                   uint32_t dim, uint32_t k, uint32_t n, float kd, uint32_t vec4, float kd_unmoved, uint32_t* __restrict__ assignment)
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

static uint32_t fused_dp(uint32_t dim)
{
	for (uint32_t o : { 4u, 8u, 16u, 24u, 32u })
		if (dim <= o) return o;
	return 0;
}

bool fused_small_supports(uint32_t dim, uint32_t k)
{
	return k <= 32 && fused_dp(dim) != 0;
}

template <int DP, int LD, int LM>
static int launch_fused_t(const AssignArgs& a, float* means_out, uint32_t* sizes, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev, float kd)
{
	constexpr uint32_t NT = DP <= 16 ? 1 : 2;
	const uint32_t mt = a.k <= 16 ? 1 : 2;
	const uint32_t wave_floats = std::max<uint32_t>(WAVE * (NT * 16 + 1), mt * 16 * NT * 16);
	const uint32_t lds_bytes = (a.k * (DP + 1) + FUSED_WAVES * wave_floats) * 4;
	const uint32_t static_bytes = (2 * (FUSED_FLAG_CAP + FUSED_LATER_CAP) * FUSED_WAVES + 128) * 4;
	if (lds_bytes + static_bytes > dev.lds_bytes) return fail(KMX_ERR_UNSUPPORTED, "fused iteration: %u bytes of LDS needed", lds_bytes + static_bytes);
	void (*kernel)(const float*, size_t, const float*, const float*, const float*, size_t, float*, uint32_t*, uint32_t*, uint32_t*,
	               uint32_t, uint32_t, uint32_t, float, uint32_t, float, uint32_t*) =
		a.emit_assignment ? (mt == 1 ? fused_small_kernel<DP, LD, LM, 1, true> : fused_small_kernel<DP, LD, LM, 2, true>)
		                  : (mt == 1 ? fused_small_kernel<DP, LD, LM, 1, false> : fused_small_kernel<DP, LD, LM, 2, false>);
	const uint32_t batches = (a.n + FUSED_WAVES * WAVE - 1) / (FUSED_WAVES * WAVE);
	const uint32_t per_cu = std::max<uint32_t>(1, std::min<uint32_t>(8, dev.lds_bytes / (lds_bytes + static_bytes)));
	const uint32_t grid = std::min(batches, dev.compute_units * per_cu);
	exec->block_count = grid;
	const uint32_t vec4 = (a.layout == KMX_AOS && a.dim % 4 == 0 && a.stride % 4 == 0 && ((uintptr_t)a.data % 16) == 0) ? 1u : 0u;
	int rc = profile_begin(0);
	if (rc) return rc;
	KMX_LAUNCH_KERNEL(kernel, dim3(grid), dim3(FUSED_WAVES * WAVE), lds_bytes, stream(),
	                   a.data, a.stride, ws->packed_means, ws->norms, a.means, a.stride_means, means_out, sizes,
	                   ws->queue, ws->counters, a.dim, a.k, a.n, kd, vec4, cert_kd_unmoved(a.dim), a.assignment);
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
	/* the bound of a ranking by chains of fused multiply-adds, see certificate.h; 8 * 2^-23 for the roundings of x - m, c - m;
	 * the low bits of the values carry the centroid's number */
	const float kd = cert_kd_fma(a.dim) + 8.0f * CERT_UNIT + cert_kd_keyed(fused_key_bits(a.k <= 16 ? 1 : 2));
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
