/*
 * Device code of the split-bf16 MFMA assignment (see assign_bf16.hip for the design notes and the error bound).
 * Instantiated per row width in separate translation units (assign_bf16_inst.hip, one object per KMX_KB value).
 * Tile geometry, padding, tracking and the recheck hand-over are those of the fp32 MFMA kernel.
 */
#ifndef KMX_ASSIGN_BF16_IMPL_H
#define KMX_ASSIGN_BF16_IMPL_H

#include "assign_mfma_impl.h"
#include "certificate.h"

#include <type_traits>

namespace kmx {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr uint32_t KBLOCK = 16; /* dimensions per v_mfma_f32_32x32x16_bf16 */
constexpr uint32_t SLICED_MIN_POINTS = 1u << 16; /* fewer points: the streamed kernel, one launch */
constexpr uint32_t SLICED_MAX_SLICES = 8;
/* rows of 49 to 64 dimensions: their streamed step catches up with more centroids (N = 1M, d = 64, k = 1024: 0.398 ms in
 * two slices, 0.422 ms streamed; k = 2048: the same; k = 4096: 1.50 against 1.45 ms), and SoA points cost more to read
 * twice than the slices save (d = 56, k = 1024: 0.434 against 0.380 ms) */
constexpr uint32_t SLICED_MAX_SLICES_WIDE = 2;
/* The two-level sweep (LevelOne / ListedPoints below) pays when the first level settles most points and the sweep, not
 * the launches, is what the call costs. */
#ifndef KMX_TWO_LEVEL_MIN_POINTS
#define KMX_TWO_LEVEL_MIN_POINTS (1u << 18)
#endif
constexpr uint32_t TWO_LEVEL_MIN_TILES = 4; /* centroid tiles (from 97 centroids on) */
constexpr int STAGE_VECS = 9;   /* 16-byte pieces of a streamed chunk per lane: a chunk holds at most 9 * 512 * 16 bytes of tiles */

/* Floats per packed centroid row. The PACKED form (rows of at most 4 dimensions) has 16 slots = 8 floats per row and no
 * padding: inside a tile the slots 0..7 of the 32 rows come first, then their slots 8..15, so that the lanes of a
 * half-wave read consecutive 16-byte pieces (no bank conflicts without padding, and 4096 centroids fit the LDS). */
template <int KB, bool PACKED> constexpr uint32_t row_floats() { return PACKED ? 8 : KBLOCK * KB + ROW_PAD; }
/* PACKED: where the 8 slots of half-wave h of row r (0..31) of a tile begin */
__host__ __device__ constexpr uint32_t packed_half(uint32_t r, uint32_t h) { return h * (TILE * 4) + r * 4; }

/* rows of at most 4 dimensions: the four products of all dimensions in one block of MFMA slots (load_packed_points) */
inline bool packed_rows(uint32_t dim) { return dim <= 4; }

/* value = hi + mid + rest, both parts bf16 (round to nearest even), |mid| <= 2^-8 |value|, |rest| <= 2^-8 |mid|; returns
 * rest (both subtractions are exact in fp32) */
__device__ __forceinline__ float split_bf16(float v, __bf16& hi, __bf16& mid)
{
	hi = (__bf16)v;
	const float r = v - (float)hi;
	mid = (__bf16)r;
	return r - (float)mid;
}

/* The norms array of the split-bf16 kernels: the tiles of |c|^2 (NORM_TILE floats per tile), then per padded row
 * sum_i c'mid_i^2 and, kp floats on, sum_i c'rest_i^2 (c' = -2c; what the certificate needs, see certificate.h). */
__host__ __device__ __forceinline__ size_t split_norms_offset(uint32_t kp) { return (size_t)(kp / TILE) * NORM_TILE; }
/* ... and behind those the frame the rows are swept in (FRAME_FLOATS floats, see sweep_frame) */
__host__ __device__ __forceinline__ size_t frame_offset(uint32_t kp) { return split_norms_offset(kp) + 2 * (size_t)kp; }
/* ... and behind the frame |c|^2 of the centroids as given, in the layout of the first block (for the exact pass) */
__host__ __device__ __forceinline__ size_t exact_norms_offset(uint32_t kp) { return frame_offset(kp) + FRAME_FLOATS; }
__host__ __device__ __forceinline__ size_t split_norms_floats(uint32_t kp) { return exact_norms_offset(kp) + split_norms_offset(kp); }
struct Frame { float m[4]; };

/* One tile of 32 points as B operands: per block of 16 dimensions the lane holds the 8 dimensions of its
 * half-wave (lanes 0-31: the first 8, lanes 32-63: the second 8) of ONE point, as hi and mid parts. */
template <int KB> struct SplitPoints {
	bf16x8 hi[KB], mid[KB];
};

/* points of one sweep unit -> split B operands; xx = this lane's share of |x|^2; rows beyond n read as zero */
/*
 * Rows of at most 4 dimensions, PACKED form: the four hi/mid products of all dimensions share ONE block of 16 MFMA slots,
 *      slot      0..3       4..7       8..11     12..15
 *      centroid  c'hi       c'mid      c'hi      c'mid
 *      point     x_mid      x_hi       x_hi      x_mid
 * so a tile costs one MFMA instead of three and the mid * mid product is kept (bound at the top of assign_bf16.hip).
 * The lane holds the 8 slots of its half-wave in b.hi[0]; b.mid stays unused.
 */
/* The coordinates a lane holds of P tiles of 32 points as they come from memory (rows beyond n read as zero): requested
 * before a sweep and converted after it, so that the sweep hides the latency of the loads. */
template <int KB, bool PACKED> struct RawPoints {
	float v[PACKED ? 4 : KB * 8];
};

template <int P, int LD, bool VEC>
__device__ __forceinline__ void request_packed_points(RawPoints<1, true> (&raw)[P], const float* __restrict__ data, size_t stride,
                                                      uint32_t base, uint32_t col, uint32_t dim, uint32_t n)
{
#pragma unroll
	for (int p = 0; p < P; ++p) {
		const uint32_t pt = base + p * TILE + col;
		const bool valid = pt < n;
		if (LD == KMX_AOS && VEC) { /* dim == 4, aligned rows */
			f32x4 t = { 0.0f, 0.0f, 0.0f, 0.0f };
			if (valid) t = *(const f32x4*)(data + (size_t)pt * stride);
			raw[p].v[0] = t.x; raw[p].v[1] = t.y; raw[p].v[2] = t.z; raw[p].v[3] = t.w;
		}
		else {
#pragma unroll
			for (int j = 0; j < 4; ++j) raw[p].v[j] = (valid && (uint32_t)j < dim) ? data[elem<LD>(stride, pt, j)] : 0.0f;
		}
	}
}

template <int P>
__device__ __forceinline__ void convert_packed_points(SplitPoints<1> (&b)[P], float (&xx)[P], const RawPoints<1, true> (&raw)[P], uint32_t h, const Frame& frame)
{
#pragma unroll
	for (int p = 0; p < P; ++p) {
		float part = 0.0f, rest2 = 0.0f;
#pragma unroll
		for (int j = 0; j < 4; ++j) {
			const float v = raw[p].v[j] - frame.m[j];
			part += v * v;
			__bf16 hi, mid;
			const float rest = split_bf16(v, hi, mid);
			rest2 += rest * rest;
			b[p].hi[0][j] = h == 0 ? mid : hi;      /* slots 0..3: x_mid,  slots 8..11: x_hi   */
			b[p].hi[0][4 + j] = h == 0 ? hi : mid;  /* slots 4..7: x_hi,   slots 12..15: x_mid */
			b[p].mid[0][j] = (__bf16)0.0f;
			b[p].mid[0][4 + j] = (__bf16)0.0f;
		}
		xx[p] = h == 0 ? part : rest2; /* the two half-waves hold the same point: |x|^2 in the first, sum_i xrest_i^2 in the second */
	}
}

template <int P, int LD, bool VEC>
__device__ __forceinline__ void load_packed_points(SplitPoints<1> (&b)[P], float (&xx)[P], const float* __restrict__ data, size_t stride,
                                                   uint32_t base, uint32_t col, uint32_t h, uint32_t dim, uint32_t n, const Frame& frame)
{
	RawPoints<1, true> raw[P];
	request_packed_points<P, LD, VEC>(raw, data, stride, base, col, dim, n);
	convert_packed_points<P>(b, xx, raw, h, frame);
}

/* LISTED: the sweep covers the points of a list (entries of two words, the first one the point number); position
 * base + p TILE + col of the list stands where the point number itself stands otherwise, n is the length of the list */
template <int KB, int P, int LD, bool VEC, bool LISTED = false>
__device__ __forceinline__ void request_split_points(RawPoints<KB, false> (&raw)[P], const float* __restrict__ data, size_t stride,
                                                     uint32_t base, uint32_t col, uint32_t h, uint32_t dim, uint32_t n,
                                                     const uint32_t* __restrict__ list = nullptr)
{
#pragma unroll
	for (int p = 0; p < P; ++p) {
		const uint32_t slot = base + p * TILE + col;
		const bool valid = slot < n;
		const uint32_t pt = LISTED ? (valid ? list[2 * (size_t)slot] : 0u) : slot;
#pragma unroll
		for (int kb = 0; kb < KB; ++kb) {
			const uint32_t d0 = kb * KBLOCK + h * 8;
			float* v = raw[p].v + 8 * kb;
			if (LD == KMX_AOS && VEC) {
				const float* src = data + (size_t)pt * stride + d0;
				f32x4 lo = { 0.0f, 0.0f, 0.0f, 0.0f }, up = { 0.0f, 0.0f, 0.0f, 0.0f };
				if (valid && d0 < dim) lo = *(const f32x4*)src;
				if (valid && d0 + 4 < dim) up = *(const f32x4*)(src + 4);
				v[0] = lo.x; v[1] = lo.y; v[2] = lo.z; v[3] = lo.w;
				v[4] = up.x; v[5] = up.y; v[6] = up.z; v[7] = up.w;
			}
			else if (LD == KMX_SOA) {
				/* the address advances from load to load; long rows are loaded 16 coordinates at a time, so that only a few
				 * of their 64-bit addresses are alive at once */
				const float* src = data + (size_t)d0 * stride + pt;
#pragma unroll
				for (int j = 0; j < 8; ++j) {
					v[j] = (valid && d0 + j < dim) ? *src : 0.0f;
					src += stride;
				}
				if (KB > 4 && kb % 2 == 1) __builtin_amdgcn_sched_barrier(0);
			}
			else {
#pragma unroll
				for (int j = 0; j < 8; ++j) v[j] = (valid && d0 + j < dim) ? data[elem<LD>(stride, pt, d0 + j)] : 0.0f;
			}
		}
	}
}

/* The rows are swept as x - m (`frame`: the FRAME_DIMS coordinates of m, zero beyond the row; the packing kernel moved the
 * centroids alike). xx = the lane's share of |x - m|^2, xm = its share of (x - m) . m (which takes a threshold back to the
 * frame of the data, see unmoved_threshold). */
/* LEVEL1 (the first level of the two-level sweep, which multiplies the hi parts only): xl = the lane's share of
 * sum_i (v_i - hi_i)^2, what its certificate needs of the point (the subtraction is exact); the mid parts go unused. */
template <int KB, int P, bool LEVEL1 = false>
__device__ __forceinline__ void convert_split_points(SplitPoints<KB> (&b)[P], float (&xx)[P], float (&xm)[P], const RawPoints<KB, false> (&raw)[P],
                                                     const float* frame, uint32_t h, float* xl = nullptr)
{
#pragma unroll
	for (int p = 0; p < P; ++p) {
		float part = 0.0f, along = 0.0f, low = 0.0f;
#pragma unroll
		for (int kb = 0; kb < KB; ++kb) {
			const f32x4 m0 = *(const f32x4*)(frame + kb * KBLOCK + h * 8), m1 = *(const f32x4*)(frame + kb * KBLOCK + h * 8 + 4);
			const float m[8] = { m0.x, m0.y, m0.z, m0.w, m1.x, m1.y, m1.z, m1.w };
#pragma unroll
			for (int j = 0; j < 8; ++j) {
				const float v = raw[p].v[8 * kb + j] - m[j];
				part += v * v;
				along += v * m[j];
				__bf16 hi, mid;
				split_bf16(v, hi, mid);
				b[p].hi[kb][j] = hi;
				b[p].mid[kb][j] = mid;
				if constexpr (LEVEL1) {
					const float r = v - (float)hi;
					low += r * r;
				}
			}
		}
		xx[p] = part;
		xm[p] = along;
		if constexpr (LEVEL1) xl[p] = low;
	}
}

/* Request and conversion of the rows of P tiles. FENCED (the sweeps of rows of more than 64 dimensions, which fill the
 * registers): all coordinates of a point are requested first, then the blocks of 16 dimensions are converted one at a time
 * behind a fence each, so that the coordinates of the frame are not requested ahead and held as well. Otherwise the
 * scheduler is left to interleave the blocks. */
template <int KB, int P, int LD, bool VEC, bool FENCED = false, bool LISTED = false, bool LEVEL1 = false>
__device__ __forceinline__ void load_split_points(SplitPoints<KB> (&b)[P], float (&xx)[P], float (&xm)[P], const float* __restrict__ data, size_t stride,
                                                  uint32_t base, uint32_t col, uint32_t h, uint32_t dim, uint32_t n, const float* frame,
                                                  const uint32_t* __restrict__ list = nullptr, float* xl = nullptr)
{
#pragma unroll
	for (int p = 0; p < P; ++p) {
		const uint32_t slot = base + p * TILE + col;
		const bool valid = slot < n;
		const uint32_t pt = LISTED ? (valid ? list[2 * (size_t)slot] : 0u) : slot; /* (see request_split_points) */
		float v[KB][8];
		auto request = [&](int kb) {
			const uint32_t d0 = kb * KBLOCK + h * 8;
			if (LD == KMX_AOS && VEC) {
				const float* src = data + (size_t)pt * stride + d0;
				f32x4 lo = { 0.0f, 0.0f, 0.0f, 0.0f }, up = { 0.0f, 0.0f, 0.0f, 0.0f };
				if (valid && d0 < dim) lo = *(const f32x4*)src;
				if (valid && d0 + 4 < dim) up = *(const f32x4*)(src + 4);
				v[kb][0] = lo.x; v[kb][1] = lo.y; v[kb][2] = lo.z; v[kb][3] = lo.w;
				v[kb][4] = up.x; v[kb][5] = up.y; v[kb][6] = up.z; v[kb][7] = up.w;
			}
			else if (LD == KMX_SOA) {
				/* the address advances from load to load; long rows are loaded 16 coordinates at a time, so that only a few
				 * of their 64-bit addresses are alive at once */
				const float* src = data + (size_t)d0 * stride + pt;
#pragma unroll
				for (int j = 0; j < 8; ++j) {
					v[kb][j] = (valid && d0 + j < dim) ? *src : 0.0f;
					src += stride;
				}
				if (KB > 4 && kb % 2 == 1) __builtin_amdgcn_sched_barrier(0);
			}
			else {
#pragma unroll
				for (int j = 0; j < 8; ++j) v[kb][j] = (valid && d0 + j < dim) ? data[elem<LD>(stride, pt, d0 + j)] : 0.0f;
			}
		};
		float part = 0.0f, along = 0.0f, low = 0.0f;
		auto convert = [&](int kb) {
			const uint32_t d0 = kb * KBLOCK + h * 8;
			const f32x4 m0 = *(const f32x4*)(frame + d0), m1 = *(const f32x4*)(frame + d0 + 4);
			const float m[8] = { m0.x, m0.y, m0.z, m0.w, m1.x, m1.y, m1.z, m1.w };
#pragma unroll
			for (int j = 0; j < 8; ++j) {
				const float w = v[kb][j] - m[j];
				part += w * w;
				along += w * m[j];
				if constexpr (LEVEL1) { /* the first level multiplies the hi parts only (convert_split_points): no mid part, |w - hi|^2 instead */
					const __bf16 hi = (__bf16)w;
					/* hi as a float: its 16 bits in the upper half of the word */
					const float r = w - __uint_as_float((uint32_t)__builtin_bit_cast(unsigned short, hi) << 16);
					low = __builtin_fmaf(r, r, low);
					b[p].hi[kb][j] = hi;
				}
				else {
					__bf16 hi, mid;
					split_bf16(w, hi, mid);
					b[p].hi[kb][j] = hi;
					b[p].mid[kb][j] = mid;
				}
			}
		};
		if (FENCED) {
#pragma unroll
			for (int kb = 0; kb < KB; ++kb) request(kb);
#pragma unroll
			for (int kb = 0; kb < KB; ++kb) {
				__builtin_amdgcn_sched_barrier(0);
				convert(kb);
			}
		}
		else {
#pragma unroll
			for (int kb = 0; kb < KB; ++kb) {
				request(kb);
				convert(kb);
			}
		}
		xx[p] = part;
		xm[p] = along;
		if constexpr (LEVEL1) {
			/* the sum exists here, in a register: left alone the compiler moves the additions behind the sweep, where the
			 * sum is used, and keeps all coordinates alive until then (150 to 900 spilled registers at 256 dimensions) */
			asm volatile("" : "+v"(low));
			xl[p] = low;
		}
	}
}

/* the 16 bytes (8 bf16) at 16-byte unit `unit` of a packed row */
__device__ __forceinline__ bf16x8 row_unit(const float* row, uint32_t unit) { return *(const bf16x8*)(row + 4 * unit); }

/*
 * One step of the software pipeline: the MFMAs of tile `tile_new` into acc_new (three products per block of 16
 * dimensions: hi*mid, mid*hi, hi*hi -- small terms first) and the tracking of the previous tile's results.
 * Packed row layout, in 16-byte units: block kb, half-wave h -> unit 4 kb + 2 h holds the hi parts of the
 * 8 dimensions, unit 4 kb + 2 h + 1 the mid parts.
 */
/* rows of at least 32 dimensions: the refinement is worth halving (see track_tile) */
template <int KB> constexpr bool fine8_bf16() { return KB >= 2; }

template <int KB, int P, bool TRACK, bool COARSE, bool PACKED = false>
__device__ __forceinline__ void tile_step_bf16(const float* __restrict__ lds, const float* __restrict__ lds_norms, uint32_t tile_new,
                                               uint32_t col, uint32_t h, const SplitPoints<KB> (&b)[P],
                                               f32x16 (&acc_new)[P], const f32x16 (&acc_old)[P], uint32_t tile_old,
                                               Track (&st)[P], float neg_inf)
{
	constexpr uint32_t RS = row_floats<KB, PACKED>();
	const float* arow = lds + (size_t)tile_new * tile_floats(RS) + (PACKED ? packed_half(col, h) : col * RS);
	bf16x8 chi[KB], cmid[KB];
#pragma unroll
	for (int kb = 0; kb < KB; ++kb) {
		chi[kb] = PACKED ? *(const bf16x8*)arow : row_unit(arow, 4 * kb + 2 * h);
		if (!PACKED) cmid[kb] = row_unit(arow, 4 * kb + 2 * h + 1);
	}
	/* C operand: |c|^2 of the 16 rows this lane receives: rows 8g + 4h + (0..3), g = 0..3 */
	f32x16 cinit;
#pragma unroll
	for (int g = 0; g < 4; ++g) {
		f32x4 v = *(const f32x4*)(lds_norms + tile_new * NORM_TILE + 8 * g + 4 * h);
		cinit[4 * g] = v.x; cinit[4 * g + 1] = v.y; cinit[4 * g + 2] = v.z; cinit[4 * g + 3] = v.w;
	}
	if constexpr (PACKED) {
		/* one MFMA per tile: chi[0] holds the half-wave's 8 slots of the row, b.hi[0] the point's */
#pragma unroll
		for (int p = 0; p < P; ++p) acc_new[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(chi[0], b[p].hi[0], cinit, 0, 0, 0);
		if (TRACK) {
#pragma unroll
			for (int p = 0; p < P; ++p) track_tile<COARSE, false>(acc_old[p], st[p], tile_old, neg_inf);
			__builtin_amdgcn_sched_group_barrier(0x008, P, 0);
			__builtin_amdgcn_sched_group_barrier(0x002, (COARSE ? 12 : 67) * P, 0);
		}
		return;
	}
#pragma unroll
	for (int p = 0; p < P; ++p) acc_new[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(chi[0], b[p].mid[0], cinit, 0, 0, 0);
#pragma unroll
	for (int kb = 0; kb < KB; ++kb) {
		if (kb > 0) {
#pragma unroll
			for (int p = 0; p < P; ++p) acc_new[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(chi[kb], b[p].mid[kb], acc_new[p], 0, 0, 0);
		}
#pragma unroll
		for (int p = 0; p < P; ++p) acc_new[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(cmid[kb], b[p].hi[kb], acc_new[p], 0, 0, 0);
#pragma unroll
		for (int p = 0; p < P; ++p) acc_new[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(chi[kb], b[p].hi[kb], acc_new[p], 0, 0, 0);
	}
	if (TRACK) {
#pragma unroll
		for (int p = 0; p < P; ++p) track_tile<COARSE, fine8_bf16<KB>()>(acc_old[p], st[p], tile_old, neg_inf);
		constexpr int MFMAS = 3 * KB * P;
		constexpr int VALU = (COARSE ? (fine8_bf16<KB>() ? 16 : 12) : 67) * P;
		if (KB <= 4) {
			__builtin_amdgcn_sched_group_barrier(0x008, MFMAS, 0);
			__builtin_amdgcn_sched_group_barrier(0x002, VALU, 0);
		}
	}
}

/* acc + a[2i] b[2i] + a[2i+1] b[2i+1] as one v_dot2c_f32_bf16 (pairs taken with constant shuffles: extracting a
 * dword of the bit-cast vector by a loop index made the compiler read element 0 every time) */
#define KMX_DOT2_PAIR(acc, a, b, i) \
	__builtin_amdgcn_fdot2_f32_bf16(__builtin_shufflevector(a, a, 2 * (i), 2 * (i) + 1), __builtin_shufflevector(b, b, 2 * (i), 2 * (i) + 1), acc, false)

/* this half-wave's share of the three-product dot of one packed row with one point (the same terms the MFMAs add) */
template <int KB, bool PACKED = false>
__device__ __forceinline__ float row_dot_bf16(const float* row, uint32_t h, const SplitPoints<KB>& x)
{
	float part = 0.0f;
	if constexpr (PACKED) { /* the half-wave's 8 slots of the packed row (row points at them) against the point's */
		const bf16x8 ch = *(const bf16x8*)row;
		const bf16x8 xh = x.hi[0];
		part = KMX_DOT2_PAIR(part, ch, xh, 0); part = KMX_DOT2_PAIR(part, ch, xh, 1);
		part = KMX_DOT2_PAIR(part, ch, xh, 2); part = KMX_DOT2_PAIR(part, ch, xh, 3);
		return part;
	}
#pragma unroll
	for (int kb = 0; kb < KB; ++kb) {
		const bf16x8 ch = row_unit(row, 4 * kb + 2 * h);
		const bf16x8 cm = row_unit(row, 4 * kb + 2 * h + 1);
		const bf16x8 xh = x.hi[kb];
		const bf16x8 xm = x.mid[kb];
		part = KMX_DOT2_PAIR(part, ch, xm, 0); part = KMX_DOT2_PAIR(part, cm, xh, 0); part = KMX_DOT2_PAIR(part, ch, xh, 0);
		part = KMX_DOT2_PAIR(part, ch, xm, 1); part = KMX_DOT2_PAIR(part, cm, xh, 1); part = KMX_DOT2_PAIR(part, ch, xh, 1);
		part = KMX_DOT2_PAIR(part, ch, xm, 2); part = KMX_DOT2_PAIR(part, cm, xh, 2); part = KMX_DOT2_PAIR(part, ch, xh, 2);
		part = KMX_DOT2_PAIR(part, ch, xm, 3); part = KMX_DOT2_PAIR(part, cm, xh, 3); part = KMX_DOT2_PAIR(part, ch, xh, 3);
	}
	return part;
}

/* the same share of the dot product from the row's 16-byte pieces already in registers: piece 2 kb = hi parts, 2 kb + 1 = mid parts of block kb */
template <int KB, bool PACKED = false>
__device__ __forceinline__ float pieces_dot_bf16(const bf16x8 (&piece)[PACKED ? 1 : 2 * KB], const SplitPoints<KB>& x)
{
	float part = 0.0f;
	if constexpr (PACKED) {
		const bf16x8 ch = piece[0];
		const bf16x8 xh = x.hi[0];
		part = KMX_DOT2_PAIR(part, ch, xh, 0); part = KMX_DOT2_PAIR(part, ch, xh, 1);
		part = KMX_DOT2_PAIR(part, ch, xh, 2); part = KMX_DOT2_PAIR(part, ch, xh, 3);
		return part;
	}
	else {
#pragma unroll
		for (int kb = 0; kb < KB; ++kb) {
			const bf16x8 ch = piece[2 * kb];
			const bf16x8 cm = piece[2 * kb + 1];
			const bf16x8 xh = x.hi[kb];
			const bf16x8 xm = x.mid[kb];
			part = KMX_DOT2_PAIR(part, ch, xm, 0); part = KMX_DOT2_PAIR(part, cm, xh, 0); part = KMX_DOT2_PAIR(part, ch, xh, 0);
			part = KMX_DOT2_PAIR(part, ch, xm, 1); part = KMX_DOT2_PAIR(part, cm, xh, 1); part = KMX_DOT2_PAIR(part, ch, xh, 1);
			part = KMX_DOT2_PAIR(part, ch, xm, 2); part = KMX_DOT2_PAIR(part, cm, xh, 2); part = KMX_DOT2_PAIR(part, ch, xh, 2);
			part = KMX_DOT2_PAIR(part, ch, xm, 3); part = KMX_DOT2_PAIR(part, cm, xh, 3); part = KMX_DOT2_PAIR(part, ch, xh, 3);
		}
		return part;
	}
}

/*
 * The sweep with a SNAPSHOT of the leading group (rows of 17 to 64 dimensions, ten centroid tiles or more).
 *
 * What the counters and a few cut-down kernels showed at N = 2M, d = 32, k = 1024: VALU work next to
 * v_mfma_f32_32x32x16_bf16 is free (a wavefront, or its partner on the SIMD, issues it while the matrix pipe works:
 * 18 MFMAs + 48 VALU operations take the time of the 18 MFMAs); what is not free is the local data share. Recomputing the
 * winning group of rows at the end of a sweep (the refinement of the other kernels) reads eight rows per point from
 * per-lane addresses -- 32 conflicted 16-byte reads per point tile -- and cost 0.11 ms of a 0.36 ms sweep; and the
 * operands of a tile, requested right before its MFMAs, cost another 0.08 ms of waiting. Hence
 *   - tracking keeps, per lane and point tile, the 8 results of the group of rows that holds the smallest value so far
 *     (8 conditional moves per group on top of the 8 operations of the minimum tracking): at the end of the sweep the
 *     winner's row and the runner-up inside its group come from registers, nothing is read again;
 *   - the centroid parts of tile t + 1 are requested before the MFMAs of tile t are issued (two register sets), and its
 *     norms, which start the accumulators, as soon as the accumulators they go to have been tracked, a third of a step
 *     before they are needed: no MFMA waits for the local data share;
 *   - the tracking operations are spread between the MFMAs, a few after each.
 */
template <int KB> struct StepOperands {
	bf16x8 chi[KB], cmid[KB];
};

/* HI_ONLY: the first level of the two-level sweep multiplies the hi parts only and leaves the mid parts in LDS */
template <int KB, bool HI_ONLY = false>
__device__ __forceinline__ void fetch_operands(StepOperands<KB>& o, const float* __restrict__ lds_tiles, uint32_t tile, uint32_t col, uint32_t h)
{
	constexpr uint32_t RS = row_floats<KB, false>();
	const float* arow = lds_tiles + (size_t)tile * tile_floats(RS) + col * RS;
#pragma unroll
	for (int kb = 0; kb < KB; ++kb) {
		o.chi[kb] = row_unit(arow, 4 * kb + 2 * h);
		if constexpr (!HI_ONLY) o.cmid[kb] = row_unit(arow, 4 * kb + 2 * h + 1);
	}
}

/* |c|^2 of the 16 rows of `tile` this lane receives (rows 8g + 4h + 0..3): the C operand of the tile's first MFMAs */
__device__ __forceinline__ void fetch_norms(f32x16& c, const float* __restrict__ lds_norms, uint32_t tile, uint32_t h)
{
#pragma unroll
	for (int g = 0; g < 4; ++g) {
		const f32x4 v = *(const f32x4*)(lds_norms + tile * NORM_TILE + 8 * g + 4 * h);
		c[4 * g] = v.x; c[4 * g + 1] = v.y; c[4 * g + 2] = v.z; c[4 * g + 3] = v.w;
	}
}

/* The MFMAs of one centroid tile for P point tiles: per block of 16 dimensions hi*mid, mid*hi, hi*hi (small terms
 * first). On entry acc[0] holds the tile's norms: they start every accumulator (acc[0] itself last). */
template <int KB, int P, bool HI_ONLY = false>
__device__ __forceinline__ void mfma_tile(f32x16 (&acc)[P], const StepOperands<KB>& o, const SplitPoints<KB> (&b)[P])
{
	if constexpr (HI_ONLY) { /* one product per dimension */
#pragma unroll
		for (int kb = 0; kb < KB; ++kb) {
#pragma unroll
			for (int p = P - 1; p >= 0; --p) acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(o.chi[kb], b[p].hi[kb], kb == 0 ? acc[0] : acc[p], 0, 0, 0);
		}
		return;
	}
#pragma unroll
	for (int p = P - 1; p >= 0; --p) acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(o.chi[0], b[p].mid[0], acc[0], 0, 0, 0);
#pragma unroll
	for (int kb = 0; kb < KB; ++kb) {
		if (kb > 0) {
#pragma unroll
			for (int p = P - 1; p >= 0; --p) acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(o.chi[kb], b[p].mid[kb], acc[p], 0, 0, 0);
		}
#pragma unroll
		for (int p = P - 1; p >= 0; --p) acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(o.cmid[kb], b[p].hi[kb], acc[p], 0, 0, 0);
#pragma unroll
		for (int p = P - 1; p >= 0; --p) acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(o.chi[kb], b[p].hi[kb], acc[p], 0, 0, 0);
	}
}

/* A lane mask that a vector compare has just written to scalar registers, for use by the masked copies below: on gfx940 and later a
 * vector instruction may read a scalar register that a vector instruction wrote only two wait states later. The compiler
 * keeps that distance for its own instructions but does not look inside inline assembly, so the wait is written out here;
 * the copies take the mask from this function's result and are thereby ordered behind it. */
__device__ __forceinline__ uint64_t settled_mask(uint64_t mask)
{
	asm volatile("s_nop 1" : "+s"(mask));
	return mask;
}

/* The snapshot: the 16 results of the tile that holds a lane's smallest ranking value so far. */
constexpr int SNAP_ROWS = 16;

/* Copies in the lanes of `mask` only (a mask from settled_mask), for the lanes whose tile took the lead. The execution mask
 * is narrowed to those lanes and restored inside one assembly statement, so nothing the compiler emits runs under the
 * narrowed mask; in between, plain moves do what would otherwise be one v_cndmask per register, and v_mov_b64 moves two
 * registers at the rate of one: the 16 results of a tile cost 8 instructions. The results are consecutive registers of the
 * MFMA's accumulator, so their pairs cost no copies; the snapshot's pairs are formed here and stay pairs, as nothing else
 * writes them. Fewer, longer statements are better than one per MFMA slot: every switch of the mask costs two scalar
 * instructions and a wait for them. */
#define KMX_SNAPSHOT_PAIRS(r)                                                                                                                \
	f32x2 d0 = {snap[r], snap[r + 1]}, d1 = {snap[r + 2], snap[r + 3]}, d2 = {snap[r + 4], snap[r + 5]}, d3 = {snap[r + 6], snap[r + 7]}; \
	const f32x2 s0 = {a[r], a[r + 1]}, s1 = {a[r + 2], a[r + 3]}, s2 = {a[r + 4], a[r + 5]}, s3 = {a[r + 6], a[r + 7]}
#define KMX_SNAPSHOT_UNPAIR(r)                                                                                    \
	snap[r] = d0.x, snap[r + 1] = d0.y, snap[r + 2] = d1.x, snap[r + 3] = d1.y, snap[r + 4] = d2.x, snap[r + 5] = d2.y, \
	snap[r + 6] = d3.x, snap[r + 7] = d3.y

/* in the lanes of `mask`: the smallest value so far becomes `lowest`, its tile `tile` (the same in every lane: a scalar
 * operand), and results 0..7 of the tile replace the first half of the snapshot */
__device__ __forceinline__ void take_lead_where(uint64_t mask, float& m1, uint32_t& leader_tile, float lowest, uint32_t tile,
                                                float (&snap)[SNAP_ROWS], const f32x16& a)
{
	uint64_t saved;
	KMX_SNAPSHOT_PAIRS(0);
	asm volatile("s_and_saveexec_b64 %[saved], %[mask]\n\tv_mov_b32 %[m1], %[lowest]\n\tv_mov_b32 %[leader], %[tile]\n\t"
	             "v_mov_b64 %[d0], %[s0]\n\tv_mov_b64 %[d1], %[s1]\n\tv_mov_b64 %[d2], %[s2]\n\tv_mov_b64 %[d3], %[s3]\n\ts_mov_b64 exec, %[saved]"
	             : [m1] "+v"(m1), [leader] "+v"(leader_tile), [d0] "+v"(d0), [d1] "+v"(d1), [d2] "+v"(d2), [d3] "+v"(d3), [saved] "=&s"(saved)
	             : [lowest] "v"(lowest), [tile] "s"(tile), [s0] "v"(s0), [s1] "v"(s1), [s2] "v"(s2), [s3] "v"(s3), [mask] "s"(mask)
	             : "scc");
	KMX_SNAPSHOT_UNPAIR(0);
}

/* in the lanes of `mask`: results 8..15 of the tile replace the second half of the snapshot */
__device__ __forceinline__ void copy_second_half_where(uint64_t mask, float (&snap)[SNAP_ROWS], const f32x16& a)
{
	uint64_t saved;
	KMX_SNAPSHOT_PAIRS(8);
	asm volatile("s_and_saveexec_b64 %[saved], %[mask]\n\tv_mov_b64 %[d0], %[s0]\n\tv_mov_b64 %[d1], %[s1]\n\tv_mov_b64 %[d2], %[s2]\n\t"
	             "v_mov_b64 %[d3], %[s3]\n\ts_mov_b64 exec, %[saved]"
	             : [d0] "+v"(d0), [d1] "+v"(d1), [d2] "+v"(d2), [d3] "+v"(d3), [saved] "=&s"(saved)
	             : [s0] "v"(s0), [s1] "v"(s1), [s2] "v"(s2), [s3] "v"(s3), [mask] "s"(mask)
	             : "scc");
	KMX_SNAPSHOT_UNPAIR(8);
}
#undef KMX_SNAPSHOT_PAIRS
#undef KMX_SNAPSHOT_UNPAIR

/* Tracking with the snapshot: the minimum of the lane's 16 results of a tile (NaN-propagating tree, see track_tile), the two
 * smallest tile minima so far (m1 <= m2), the tile that holds m1 and its 16 results. MASKED: the copies under a narrowed
 * execution mask (above) instead of selections the compiler schedules freely; the wide-row step, whose MFMAs hide its
 * tracking anyway, is faster with the latter (N = 1M, d = 64, k = 512: 0.182 against 0.186 ms). */
template <bool MASKED>
__device__ __forceinline__ void track_snapshot(const f32x16& acc, Track& s, float (&snap)[SNAP_ROWS], uint32_t tile)
{
	auto lowest = [](float a, float b) { return __builtin_elementwise_minimum(a, b); };
	float t = acc[0];
#pragma unroll
	for (int i = 1; i < 16; ++i) t = lowest(t, acc[i]);
	s.m2 = __builtin_amdgcn_fmed3f(s.m1, s.m2, t); /* second smallest of {m1, m2, t} as m1 <= m2 */
	if constexpr (MASKED) {
		const uint64_t leads = settled_mask(tile == 0 ? ~0ull : __builtin_amdgcn_ballot_w64(t < s.m1)); /* tile 0 fills the snapshot, whatever its values */
		take_lead_where(leads, s.m1, s.tile, t, tile, snap, acc);
		copy_second_half_where(leads, snap, acc);
	}
	else {
		const bool lt = t < s.m1 || tile == 0; /* tile 0 fills the snapshot, whatever its values */
		s.tile = lt ? tile : s.tile;
		s.m1 = lt ? t : s.m1;
#pragma unroll
		for (int i = 0; i < 16; ++i) snap[i] = lt ? acc[i] : snap[i];
	}
}

/* which kernel instances sweep with the fenced, prefetching step (unpacked rows of up to 48 dimensions, ten centroid tiles or
 * more, all centroids resident) and which of those track with the snapshot: all of them. (Measured on one box at N = 2M, d = 32,
 * k = 1024: 0.325 ms with the snapshot and two point tiles against 0.344 ms with group minima, a refinement and three point
 * tiles, which spills 9 registers; KMX_SNAPSHOT_FROM_KB = 3 builds the latter for rows of 17 to 32 dimensions. Rows of 5 to 16
 * dimensions, three MFMAs per tile: N = 2M, d = 16: k = 320 0.136 -> 0.110 ms, k = 1024 0.238 -> 0.235 ms; d = 12, k = 512:
 * 0.160 -> 0.144 ms; no shape slower.) */
#ifndef KMX_SNAPSHOT_FROM_KB
#define KMX_SNAPSHOT_FROM_KB 1
#endif
/* the wide-row step (wide_sweep): rows of 49 dimensions and more */
template <int KB> constexpr bool wide_rows_sweep() { return KB >= 4; }
/* ... which of them track with the snapshot (track_snapshot: 29 operations per tile instead of the 66 of the row-by-row
 * tracking, 16 registers per point tile): rows of 49 to 64 dimensions, whose 12 MFMAs per tile are short of hiding 66 */
#ifndef KMX_WIDE_SNAPSHOT_UP_TO_KB
#define KMX_WIDE_SNAPSHOT_UP_TO_KB 4
#endif
template <int KB> constexpr bool wide_rows_snapshot() { return wide_rows_sweep<KB>() && KB <= KMX_WIDE_SNAPSHOT_UP_TO_KB; }
template <int KB, bool STREAM, bool COARSE, bool PACKED> constexpr bool pipelined_sweep() { return COARSE && !PACKED && !STREAM && KB <= 3; }
template <int KB, bool STREAM, bool COARSE, bool PACKED> constexpr bool snapshot_sweep() { return pipelined_sweep<KB, STREAM, COARSE, PACKED>() && KB >= KMX_SNAPSHOT_FROM_KB; }

/*
 * A sweep may cover a slice of the centroids only (rows slice.row_base .. slice.row_base + kp of the packed block; `packed`
 * and `norms` then point at the slice). The launcher cuts the centroids into slices that fit the LDS when streaming them
 * through it would be slower than sweeping the points once per slice. Between the launches a point's leader and its two
 * smallest ranking values travel in `carried` (three arrays of n words); the last slice decides. tau is the same in every
 * slice: its coefficients are maxima over all centroids.
 */
struct CentroidSlice {
	const float* all_norms; /* the norms block of all centroids (the maxima of the certificate, the frame) */
	uint32_t* carried;      /* [3][n]: leader, smallest and second smallest ranking value over the earlier slices */
	uint32_t all_k, all_kp;
	uint32_t row_base;      /* first centroid of the slice */
	uint32_t mode;          /* CARRY_IN: earlier slices have been swept; CARRY_OUT: later ones follow, nothing is decided yet */
};
constexpr uint32_t CARRY_IN = 1u, CARRY_OUT = 2u;

/*
 * The two-level sweep (rows of 17 to 32 dimensions, resident centroids, many points). Level 1 multiplies the hi parts only:
 * a third of the matrix work, half the operand registers and LDS reads, and a certificate about two hundred times wider
 * (cert_coeffs_level1), which still settles the points whose two nearest centroids are far apart -- 86 % at the headline
 * configuration. The points it cannot settle go to a list (`queue` and `counters` of that launch are the list and its
 * length), and level 2, the three-product sweep, covers the points of that list instead of all points; what level 2
 * cannot settle goes to the exact pass as before. A point's result does not depend on the level that settles it: every
 * level writes the serial scan's index or passes the point on.
 */
struct LevelOne {
	uint32_t unused;
};
struct ListedPoints {
	const uint32_t* list;    /* entries of two words, the first one the point number */
	const uint32_t* length;  /* entries in the list (written by the launch of level 1) */
};
template <class T, class... Extra> constexpr bool extra_is() { return sizeof...(Extra) == 1 && (std::is_same<T, Extra>::value || ...); }
__device__ __forceinline__ CentroidSlice slice_of() { return CentroidSlice{ nullptr, nullptr, 0u, 0u, 0u, 0u }; }
__device__ __forceinline__ CentroidSlice slice_of(const CentroidSlice& s) { return s; }
__device__ __forceinline__ CentroidSlice slice_of(const LevelOne&) { return slice_of(); }
__device__ __forceinline__ CentroidSlice slice_of(const ListedPoints&) { return slice_of(); }
__device__ __forceinline__ ListedPoints listed_of() { return ListedPoints{ nullptr, nullptr }; }
__device__ __forceinline__ ListedPoints listed_of(const ListedPoints& l) { return l; }
template <class T> __device__ __forceinline__ ListedPoints listed_of(const T&) { return listed_of(); }

/* (Slice: nothing; CentroidSlice for the instances that sweep slices; LevelOne / ListedPoints for the two levels of the
 * two-level sweep; the others are compiled without any of it) */
template <int KB, int P, int LD, bool VEC, bool STREAM, bool COARSE, bool PREFETCH, bool PACKED = false, class... Slice>
__global__ void __launch_bounds__(MFMA_WAVES * WAVE)
assign_bf16_kernel(const float* __restrict__ data, size_t stride, const float* __restrict__ packed, const float* __restrict__ norms,
                   uint32_t* __restrict__ assignment, uint32_t* __restrict__ queue, uint32_t* __restrict__ counters,
                   uint32_t dim, uint32_t k, uint32_t kp, uint32_t n_given, uint32_t chunk_rows, float kd, float neg_inf, uint32_t shifted_cap,
                   float kd_unmoved, Slice... slice_argument)
{
	static_assert(sizeof...(Slice) <= 1, "at most one slice");
	constexpr bool SLICED = extra_is<CentroidSlice, Slice...>();
	constexpr bool LEVEL1 = extra_is<LevelOne, Slice...>();
	constexpr bool LISTED = extra_is<ListedPoints, Slice...>();
	static_assert(!(LEVEL1 || LISTED) || (COARSE && !PACKED && !STREAM && KB <= 3 && PREFETCH) || (wide_rows_sweep<KB>() && STREAM && !PREFETCH),
	              "the two-level sweep is built on the pipelined step with prefetched points and on the wide-row step");
	[[maybe_unused]] const CentroidSlice slice = slice_of(slice_argument...);
	[[maybe_unused]] const ListedPoints listed = listed_of(slice_argument...);
	/* LISTED: the points of the list (never more than the caller's n) */
	const uint32_t n = LISTED ? min(listed.length[0], n_given) : n_given;
	const float* __restrict__ all_norms = SLICED ? slice.all_norms : norms;
	const uint32_t all_k = SLICED ? slice.all_k : k, all_kp = SLICED ? slice.all_kp : kp;
	constexpr uint32_t RS = row_floats<KB, PACKED>();
	extern __shared__ __attribute__((aligned(16))) float lds[];
	Frame frame = { { 0.0f, 0.0f, 0.0f, 0.0f } }; /* PACKED: the rows are swept as x - frame (pack_means_bf16_kernel moved the centroids alike) */
	if constexpr (PACKED) {
#pragma unroll
		for (int j = 0; j < 4; ++j) frame.m[j] = all_norms[frame_offset(all_kp) + j];
	}
	__shared__ __attribute__((aligned(16))) float frame_lds[PACKED ? 4 : KB * KBLOCK]; /* unpacked rows: m, see convert_split_points */
	if constexpr (!PACKED) {
		for (uint32_t i = threadIdx.x; i < KB * KBLOCK; i += blockDim.x) frame_lds[i] = all_norms[frame_offset(all_kp) + i];
	}
	const float frame_m2 = PACKED ? 0.0f : all_norms[frame_offset(all_kp) + FRAME_DIMS];        /* |m|^2 */
	const float frame_norm = PACKED ? 0.0f : all_norms[frame_offset(all_kp) + FRAME_DIMS + 1];  /* an upper bound of |m| */
	__shared__ uint32_t wave_max[4][MFMA_WAVES]; /* rows 0..2: maxima per wavefront; [3][0]: items of this work-group handed out so far */
	__shared__ uint32_t flag_list[MFMA_WAVES][2 * FLAG_CAP]; /* (point, threshold) pairs */
	uint32_t& claimed = wave_max[3][0]; /* (kept inside an array whose size is a multiple of 16 bytes: the tiles behind the static data must stay 16-byte aligned for their 128-bit reads) */

	const uint32_t lane = threadIdx.x & (WAVE - 1);
	const uint32_t wave = threadIdx.x / WAVE;
	const uint32_t col = lane & 31; /* point within a tile (B column) / centroid row fed to A */
	const uint32_t h = lane >> 5;   /* half-wave: K split and the +4 row group of the result    */
	if (threadIdx.x == 0) claimed = 0u; /* (the barrier below publishes it) */

	/* max_j of |c_j|^2, sum_i c'mid_i^2 and sum_i c'rest_i^2 (bit pattern maxima: they propagate NaN and +inf, which then flag every point) */
	CertCoeffs cert;
	{
		const float* part_norms = all_norms + split_norms_offset(all_kp);
		uint32_t cmax[3] = { 0u, 0u, 0u };
		for (uint32_t j = threadIdx.x; j < all_k; j += blockDim.x) {
			cmax[0] = max(cmax[0], __float_as_uint(all_norms[norm_at(j)]));
			cmax[1] = max(cmax[1], __float_as_uint(part_norms[j]));
			cmax[2] = max(cmax[2], __float_as_uint(part_norms[all_kp + j]));
		}
#pragma unroll
		for (int q = 0; q < 3; ++q) {
			for (int off = WAVE / 2; off > 0; off >>= 1) cmax[q] = max(cmax[q], (uint32_t)__shfl_xor((int)cmax[q], off));
			if (lane == 0) wave_max[q][wave] = cmax[q];
		}
		__syncthreads();
#pragma unroll
		for (int q = 0; q < 3; ++q) {
			cmax[q] = 0;
			for (uint32_t w = 0; w < MFMA_WAVES; ++w) cmax[q] = max(cmax[q], wave_max[q][w]);
		}
		const CentroidBounds cb{ __uint_as_float(cmax[0]), __uint_as_float(cmax[1]), __uint_as_float(cmax[2]) };
		cert = PACKED ? cert_coeffs_packed(cb) : LEVEL1 ? cert_coeffs_level1(cb) : cert_coeffs_split(cb);
		/* the same in every lane of the work-group: kept in scalar registers */
		cert.c2max = __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(cert.c2max)));
		cert.a = __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(cert.a)));
		cert.b = __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(cert.b)));
	}
	const float c2max = cert.c2max;

	const uint32_t chunk_tiles = chunk_rows / TILE;
	const uint32_t chunks = (kp + chunk_rows - 1) / chunk_rows;
	/* STREAM: two LDS buffers of chunk_tiles packed tiles followed by their norms; `cur` is the one in use */
	const uint32_t buf_floats = chunk_tiles * (tile_floats(RS) + NORM_TILE);
	uint32_t cur = 0;

	/* one chunk on its way from global memory to LDS: this lane's share, held in registers while the previous
	 * chunk is being used (requested before, committed after the tile steps of that chunk) */
	struct Staged {
		f32x4 v[STAGE_VECS];
		f32x4 nv;
	};
	auto request = [&](Staged& sg, uint32_t row0, uint32_t rows) {
		const f32x4* src = (const f32x4*)(packed + packed_row(row0, RS));
		const uint32_t vecs = (rows / TILE) * tile_floats(RS) / 4;
#pragma unroll
		for (int i = 0; i < STAGE_VECS; ++i) {
			const uint32_t at = threadIdx.x + i * (MFMA_WAVES * WAVE);
			if (at < vecs) sg.v[i] = src[at];
		}
		const f32x4* nsrc = (const f32x4*)(norms + (size_t)(row0 / TILE) * NORM_TILE);
		if (threadIdx.x < (rows / TILE) * NORM_TILE / 4) sg.nv = nsrc[threadIdx.x];
	};
	auto commit = [&](const Staged& sg, uint32_t buffer, uint32_t rows) {
		f32x4* dst = (f32x4*)(lds + (size_t)buffer * buf_floats);
		const uint32_t vecs = (rows / TILE) * tile_floats(RS) / 4;
#pragma unroll
		for (int i = 0; i < STAGE_VECS; ++i) {
			const uint32_t at = threadIdx.x + i * (MFMA_WAVES * WAVE);
			if (at < vecs) dst[at] = sg.v[i];
		}
		f32x4* ndst = (f32x4*)(lds + (size_t)buffer * buf_floats + (size_t)chunk_tiles * tile_floats(RS));
		if (threadIdx.x < (rows / TILE) * NORM_TILE / 4) ndst[threadIdx.x] = sg.nv;
	};

	if (!STREAM) {
		/* everything resident: flat 16-byte copies of all packed tiles and norms */
		const f32x4* src = (const f32x4*)packed;
		f32x4* dst = (f32x4*)lds;
		const uint32_t vecs = (kp / TILE) * tile_floats(RS) / 4;
		for (uint32_t i = threadIdx.x; i < vecs; i += blockDim.x) dst[i] = src[i];
		const f32x4* nsrc = (const f32x4*)norms;
		f32x4* ndst = (f32x4*)(lds + (size_t)chunk_tiles * tile_floats(RS));
		const uint32_t nvecs = (kp / TILE) * NORM_TILE / 4;
		for (uint32_t i = threadIdx.x; i < nvecs; i += blockDim.x) ndst[i] = nsrc[i];
		__syncthreads();
	}
	else {
		Staged first;
		request(first, 0, min(chunk_rows, kp));
		commit(first, 0, min(chunk_rows, kp));
		__syncthreads();
	}

	uint32_t flagged = 0; /* wave-uniform */
	auto flush_flags = [&]() {
		__builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
		__builtin_amdgcn_wave_barrier();
		uint32_t slot = 0;
		if (lane == 0) slot = atomicAdd(&counters[0], flagged);
		slot = (uint32_t)__shfl((int)slot, 0);
		/* (entries from shifted_cap on: thresholds of a moved frame mean nothing to the kernels that will read them) */
		for (uint32_t i = lane; i < 2 * flagged; i += WAVE)
			queue[2 * (size_t)slot + i] = ((i & 1u) && slot + i / 2 >= shifted_cap) ? __float_as_uint(__builtin_inff()) : flag_list[wave][i];
		__builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
		__builtin_amdgcn_wave_barrier();
		flagged = 0;
	};

	const uint32_t unit_points = MFMA_WAVES * P * TILE;
	const uint32_t units = (n + unit_points - 1) / unit_points;

	/*
	 * Rows of 49 dimensions and more (two point tiles per wavefront up to 128 dimensions, one above, where the split operands
	 * of a tile take half of the register file; rows of more than 64 dimensions are always streamed, the narrower ones when
	 * their centroids do not fit the LDS). Per centroid tile and point tile: one chain of 3 KB MFMAs into a single accumulator that starts from the norms;
	 * the centroid operands of block kb + 2 are requested from LDS before the MFMAs of block kb are issued
	 * (sched_group_barrier pins that order: left to itself the scheduler reads each block right before its MFMAs and the
	 * matrix pipe waits out an LDS round trip per block). The next chunk travels in pieces, one per tile step: requested
	 * from global memory before the step's MFMAs, written to the other LDS buffer after them (a few registers instead of a
	 * whole chunk's share). Lanes beyond the end of the chunk repeat its last piece, so the step has no branches.
	 * (Rows of 49 to 64 dimensions had the step of the narrower rows before, tracking groups of 8 rows behind the MFMAs of
	 * the next tile with a refinement at the end: 255 registers resident, spills when streamed. This step measured faster
	 * at every k: N = 1M, d = 64: k = 512 0.202 -> 0.187 ms, k = 1024 0.50 -> 0.40 ms, k = 2048 1.0 -> 0.745 ms.)
	 */
	constexpr int AHEAD = 2; /* blocks of centroid operands requested before the first MFMA of a step (one in flight behind the one in use; a deeper pipeline measured no faster) */
	constexpr uint32_t PIECE_VECS = (tile_floats(RS) / 4 + MFMA_WAVES * WAVE - 1) / (MFMA_WAVES * WAVE); /* 16-byte pieces per lane that cover one tile */
	constexpr bool WSNAP = wide_rows_snapshot<KB>();
	auto wide_sweep = [&](const SplitPoints<KB> (&x)[P], Track (&st)[P], float (&snap)[P][WSNAP ? SNAP_ROWS : 1]) {
		for (uint32_t chunk = 0; chunk < chunks; ++chunk) {
			const uint32_t row0 = chunk * chunk_rows;
			const uint32_t rows = min(chunk_rows, kp - row0);
			const uint32_t next_row0 = chunk + 1 < chunks ? row0 + chunk_rows : 0;
			const uint32_t next_rows = min(chunk_rows, kp - next_row0);
			const float* lds_tiles = lds + (size_t)cur * buf_floats;
			const float* lds_norms = lds_tiles + (size_t)chunk_tiles * tile_floats(RS);
			const uint32_t tiles = rows / TILE;
			const uint32_t tile0 = row0 / TILE;
			const f32x4* src = (const f32x4*)(packed + packed_row(next_row0, RS));
			const f32x4* nsrc = (const f32x4*)(norms + (size_t)(next_row0 / TILE) * NORM_TILE);
			f32x4* dst = (f32x4*)(lds + (size_t)(cur ^ 1u) * buf_floats);
			f32x4* ndst = (f32x4*)(lds + (size_t)(cur ^ 1u) * buf_floats + (size_t)chunk_tiles * tile_floats(RS));
			const uint32_t last_vec = (next_rows / TILE) * tile_floats(RS) / 4 - 1;
			const uint32_t norm_vec = min((uint32_t)threadIdx.x, (next_rows / TILE) * NORM_TILE / 4 - 1);
			uint32_t piece = threadIdx.x; /* first 16-byte piece of this lane in the current step */
			for (uint32_t t = 0; t < tiles; ++t) {
				f32x4 pv[PIECE_VECS], nv;
				if constexpr (STREAM) {
#pragma unroll
					for (uint32_t i = 0; i < PIECE_VECS; ++i) pv[i] = src[min(piece + i * (MFMA_WAVES * WAVE), last_vec)];
					nv = nsrc[norm_vec];
				}
				const float* arow = lds_tiles + (size_t)t * tile_floats(RS) + (size_t)col * RS;
				f32x16 acc[P];
#pragma unroll
				for (int g = 0; g < 4; ++g) {
					f32x4 v = *(const f32x4*)(lds_norms + t * NORM_TILE + 8 * g + 4 * h);
					acc[0][4 * g] = v.x; acc[0][4 * g + 1] = v.y; acc[0][4 * g + 2] = v.z; acc[0][4 * g + 3] = v.w;
				}
#pragma unroll
				for (int p = 1; p < P; ++p) acc[p] = acc[0];
				bf16x8 chi[KB], cmid[LEVEL1 ? 1 : KB]; /* (the first level of a two-level sweep multiplies the hi parts only) */
#pragma unroll
				for (int kb = 0; kb < AHEAD; ++kb) {
					chi[kb] = row_unit(arow, 4 * kb + 2 * h);
					if constexpr (!LEVEL1) cmid[kb] = row_unit(arow, 4 * kb + 2 * h + 1);
				}
#pragma unroll
				for (int kb = 0; kb < KB; ++kb) {
					if (kb + AHEAD < KB) {
						chi[kb + AHEAD] = row_unit(arow, 4 * (kb + AHEAD) + 2 * h);
						if constexpr (!LEVEL1) cmid[kb + AHEAD] = row_unit(arow, 4 * (kb + AHEAD) + 2 * h + 1);
					}
					if constexpr (!LEVEL1) {
#pragma unroll
						for (int p = 0; p < P; ++p) acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(chi[kb], x[p].mid[kb], acc[p], 0, 0, 0);
#pragma unroll
						for (int p = 0; p < P; ++p) acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(cmid[kb], x[p].hi[kb], acc[p], 0, 0, 0);
					}
#pragma unroll
					for (int p = 0; p < P; ++p) acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(chi[kb], x[p].hi[kb], acc[p], 0, 0, 0);
				}
#pragma unroll
				for (int p = 0; p < P; ++p) {
					if constexpr (WSNAP) track_snapshot<false>(acc[p], st[p], snap[p], tile0 + t);
					else track_tile<false, false>(acc[p], st[p], tile0 + t, neg_inf);
				}
				if constexpr (STREAM) {
#pragma unroll
					for (uint32_t i = 0; i < PIECE_VECS; ++i) dst[min(piece + i * (MFMA_WAVES * WAVE), last_vec)] = pv[i];
					ndst[norm_vec] = nv;
					piece += PIECE_VECS * (MFMA_WAVES * WAVE);
				}
				/* the order of the step: global requests; norms and AHEAD blocks of operands; then per block its MFMAs
				 * and the request for the block AHEAD blocks on; tracking and the LDS writes come last by their dependences */
				constexpr int PARTS = LEVEL1 ? 1 : 2, PRODUCTS = LEVEL1 ? 1 : 3; /* LDS reads and MFMAs per block of 16 dimensions */
				if constexpr (STREAM) __builtin_amdgcn_sched_group_barrier(0x020, PIECE_VECS + 1, 0);
				__builtin_amdgcn_sched_group_barrier(0x100, 4 + PARTS * AHEAD, 0);
#pragma unroll
				for (int kb = 0; kb < KB; ++kb) {
					__builtin_amdgcn_sched_group_barrier(0x008, PRODUCTS * P, 0);
					if (kb + AHEAD < KB) __builtin_amdgcn_sched_group_barrier(0x100, PARTS, 0);
				}
			}
			if constexpr (STREAM) {
				/* a short chunk (the last one) has fewer steps than the next chunk has tiles: the remaining pieces */
				for (; piece - threadIdx.x <= last_vec; piece += PIECE_VECS * (MFMA_WAVES * WAVE)) {
#pragma unroll
					for (uint32_t i = 0; i < PIECE_VECS; ++i) {
						const uint32_t at = min(piece + i * (MFMA_WAVES * WAVE), last_vec);
						dst[at] = src[at];
					}
				}
				__syncthreads();
				cur ^= 1u;
			}
		}
	};

	auto sweep = [&](const SplitPoints<KB> (&b)[P], const float (&xx)[P], const float (&xalong)[P], uint32_t base, [[maybe_unused]] const float* xlow = nullptr) {
		float x2[P], along_m[P];
		Track st[P];
#pragma unroll
		for (int p = 0; p < P; ++p) {
			/* PACKED: the half-waves hold |x|^2 and sum_i xrest_i^2 of the same point; the pair is taken apart again below */
			x2[p] = PACKED ? xx[p] : xx[p] + __shfl_xor(xx[p], 32);
			along_m[p] = PACKED ? 0.0f : xalong[p] + __shfl_xor(xalong[p], 32); /* (x - m) . m of the point */
			st[p].m1 = __builtin_inff();
			st[p].m2 = __builtin_inff();
			st[p].tile = 0;
			st[p].loc = 0;
		}
		f32x16 acc0[P], acc1[P];
		constexpr bool PIPE = pipelined_sweep<KB, STREAM, COARSE, PACKED>();
		constexpr bool SNAP = snapshot_sweep<KB, STREAM, COARSE, PACKED>() || WSNAP;
		float snap[P][SNAP ? SNAP_ROWS : 1];
		if constexpr (wide_rows_sweep<KB>()) {
			if constexpr (WSNAP) {
#pragma unroll
				for (int p = 0; p < P; ++p) {
#pragma unroll
					for (int i = 0; i < SNAP_ROWS; ++i) asm volatile("" : "=v"(snap[p][i])); /* no value yet: tile 0 always takes the lead */
				}
			}
			wide_sweep(b, st, snap);
		}
		else if constexpr (PIPE) {
#pragma unroll
			for (int p = 0; p < P; ++p) {
#pragma unroll
				for (int i = 0; i < (SNAP ? SNAP_ROWS : 1); ++i) asm volatile("" : "=v"(snap[p][i])); /* no value yet: tile 0 always takes the lead */
			}
			for (uint32_t chunk = 0; chunk < chunks; ++chunk) {
				const uint32_t row0 = chunk * chunk_rows;
				const uint32_t rows = min(chunk_rows, kp - row0);
				const uint32_t next_row0 = chunk + 1 < chunks ? row0 + chunk_rows : 0;
				const uint32_t next_rows = min(chunk_rows, kp - next_row0);
				Staged incoming;
				if (STREAM) request(incoming, next_row0, next_rows);
				const float* lds_tiles = lds + (size_t)cur * buf_floats;
				const float* lds_norms = lds_tiles + (size_t)chunk_tiles * tile_floats(RS);
				const uint32_t tiles = rows / TILE;
				const uint32_t tile0 = row0 / TILE;
				constexpr int MFMAS = (LEVEL1 ? 1 : 3) * KB * P;
				/* Tracking comes in pieces that are issued one behind each MFMA, so that a wavefront is back with its next MFMA before
				 * the matrix pipe has finished the last one. With the snapshot a point tile costs 20 operations (SNAP_OPS), spread
				 * evenly over its share of the step's MFMAs; without it, two pieces of 11 operations. */
				constexpr int SLOTS = MFMAS / P;                             /* MFMAs per point tile and step */
				constexpr int SNAP_OPS = 12 + SNAP_ROWS / 2;
				constexpr int OPS_PER_SLOT = (SNAP_OPS + SLOTS - 1) / SLOTS;
				constexpr int CHUNKS = SNAP ? MFMAS : 2 * P;
				constexpr int NORMS_AFTER = SNAP ? SLOTS - 1 : CHUNKS - 1;   /* acc_old[0] is free once point tile 0 has been tracked */
				static_assert(CHUNKS <= MFMAS, "a step has at least as many MFMAs as pieces of tracking");
				/* One step: tile `t_new` is computed into acc_new (which holds its norms) with the centroid parts in `use`,
				 * the centroid parts of the tile after it are requested into `fetch_into`, the tile in acc_old is tracked, and
				 * then acc_old receives the norms of the tile that will be computed into it in the next step. The order of
				 * the instructions is written out and fenced: the request first, then one piece of tracking behind each MFMA
				 * (a wavefront issues them while the matrix pipe works on the MFMA), the request for the norms as soon as
				 * acc_old[0] has been tracked: the remaining MFMAs give its answer time to arrive. */
				auto step = [&](StepOperands<KB>& fetch_into, uint32_t t_new, f32x16 (&acc_new)[P], const StepOperands<KB>& use,
				                f32x16 (&acc_old)[P], uint32_t tile_old) {
					fetch_operands<KB, LEVEL1>(fetch_into, lds_tiles, min(t_new + 1, tiles - 1), col, h);
					__builtin_amdgcn_sched_barrier(0);
					bool better[P][2];
					float lowest_of_tile[P];
					uint64_t leads[P]; /* lanes whose tile took the lead, as a mask in scalar registers */
					int issued = 0;
					auto lowest = [](float a, float b) { return __builtin_elementwise_minimum(a, b); };
					/* operation u of the snapshot tracking of point tile p: 0..7 the minimum of the lane's 16 results (NaN-propagating
					 * tree, see track_tile), 8 the second smallest tile minimum so far, 9 the lanes whose tile took the lead, as a mask in
					 * scalar registers; 12 and 16 stand for the two masked statements of six and four moves that make the tile the
					 * leader in those lanes and its results the snapshot (take_lead_where, copy_second_half_where: from a condition
					 * the compiler makes one branch around all copies, which undoes the spreading). */
					auto snapshot_op = [&](int p, int u) {
						const f32x16& a = acc_old[p];
						if (u == 0) lowest_of_tile[p] = lowest(a[0], a[1]);
						else if (u < 8) lowest_of_tile[p] = lowest(lowest(lowest_of_tile[p], a[2 * u]), a[2 * u + 1]);
						else if (u == 8) st[p].m2 = __builtin_amdgcn_fmed3f(st[p].m1, st[p].m2, lowest_of_tile[p]);
						else if (u == 9) leads[p] = settled_mask(tile_old == 0 ? ~0ull : __builtin_amdgcn_ballot_w64(lowest_of_tile[p] < st[p].m1)); /* (tile 0 fills the snapshot, whatever its values) */
						else if (u == 12) take_lead_where(leads[p], st[p].m1, st[p].tile, lowest_of_tile[p], tile_old, snap[p], a);
						else if (u == 16) copy_second_half_where(leads[p], snap[p], a);
					};
					auto after_mfma = [&](int i) {
						__builtin_amdgcn_sched_barrier(0);
						if (i < CHUNKS) {
							if constexpr (SNAP) {
								const int p = i / SLOTS, first_op = (i % SLOTS) * OPS_PER_SLOT;
#pragma unroll
								for (int u = first_op; u < first_op + OPS_PER_SLOT; ++u)
									if (u < SNAP_OPS) snapshot_op(p, u);
							}
							else {
								/* the minimum of a group of 8 results (NaN-propagating tree, see track_tile), the two smallest group
								 * minima so far and the group of the smallest */
								const int p = i / 2, g = i % 2, r = 8 * g;
								const f32x16& a = acc_old[p];
								const float t = lowest(lowest(lowest(lowest(lowest(lowest(lowest(a[r], a[r + 1]), a[r + 2]), a[r + 3]), a[r + 4]), a[r + 5]), a[r + 6]), a[r + 7]);
								st[p].m2 = __builtin_amdgcn_fmed3f(st[p].m1, st[p].m2, t);
								better[p][g] = t < st[p].m1;
								st[p].tile = better[p][g] ? 2 * tile_old + g : st[p].tile;
								st[p].m1 = better[p][g] ? t : st[p].m1;
							}
							__builtin_amdgcn_sched_barrier(0);
						}
						if (i == NORMS_AFTER) {
							fetch_norms(acc_old[0], lds_norms, min(t_new + 1, tiles - 1), h);
							__builtin_amdgcn_sched_barrier(0);
						}
					};
					if constexpr (LEVEL1) {
#pragma unroll
						for (int kb = 0; kb < KB; ++kb) {
#pragma unroll
							for (int p = P - 1; p >= 0; --p) {
								acc_new[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(use.chi[kb], b[p].hi[kb], kb == 0 ? acc_new[0] : acc_new[p], 0, 0, 0);
								after_mfma(issued++);
							}
						}
					}
					else {
#pragma unroll
					for (int p = P - 1; p >= 0; --p) {
						acc_new[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(use.chi[0], b[p].mid[0], acc_new[0], 0, 0, 0);
						after_mfma(issued++);
					}
#pragma unroll
					for (int kb = 0; kb < KB; ++kb) {
						if (kb > 0) {
#pragma unroll
							for (int p = P - 1; p >= 0; --p) {
								acc_new[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(use.chi[kb], b[p].mid[kb], acc_new[p], 0, 0, 0);
								after_mfma(issued++);
							}
						}
#pragma unroll
						for (int p = P - 1; p >= 0; --p) {
							acc_new[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(use.cmid[kb], b[p].hi[kb], acc_new[p], 0, 0, 0);
							after_mfma(issued++);
						}
#pragma unroll
						for (int p = P - 1; p >= 0; --p) {
							acc_new[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(use.chi[kb], b[p].hi[kb], acc_new[p], 0, 0, 0);
							after_mfma(issued++);
						}
					}
					}
				};
				StepOperands<KB> o0, o1;
				fetch_operands<KB, LEVEL1>(o0, lds_tiles, 0, col, h);
				fetch_norms(acc0[0], lds_norms, 0, h);
				fetch_operands<KB, LEVEL1>(o1, lds_tiles, min(1u, tiles - 1), col, h);
				fetch_norms(acc1[0], lds_norms, min(1u, tiles - 1), h);
				mfma_tile<KB, P, LEVEL1>(acc0, o0, b);
				uint32_t t = 0; /* acc0 holds tile t, not yet tracked; o1 and acc1[0] hold the centroid parts and norms of tile t + 1 */
				while (t + 2 < tiles) {
					step(o0, t + 1, acc1, o1, acc0, tile0 + t);
					step(o1, t + 2, acc0, o0, acc1, tile0 + t + 1);
					t += 2;
				}
				auto track = [&](const f32x16& acc, int p, uint32_t tile) {
					if constexpr (SNAP) track_snapshot<true>(acc, st[p], snap[p], tile);
					else track_tile<true, true>(acc, st[p], tile, neg_inf);
				};
				if (t + 1 < tiles) {
					mfma_tile<KB, P, LEVEL1>(acc1, o1, b);
#pragma unroll
					for (int p = 0; p < P; ++p) track(acc0[p], p, tile0 + t);
#pragma unroll
					for (int p = 0; p < P; ++p) track(acc1[p], p, tile0 + t + 1);
				}
				else {
#pragma unroll
					for (int p = 0; p < P; ++p) track(acc0[p], p, tile0 + t);
				}
				if (STREAM) {
					commit(incoming, cur ^ 1u, next_rows);
					__syncthreads();
					cur ^= 1u;
				}
			}
		}
		else if constexpr (PACKED && COARSE && !STREAM) {
			/* Packed rows, all centroids resident: the fenced step of the wider rows with one MFMA per point tile. The tile's
			 * 16-byte piece of centroid parts is requested a tile ahead; its norms go into the accumulator of the first
			 * point tile as soon as that one has been tracked, three MFMAs before they are needed. */
			const float* lds_norms = lds + (size_t)chunk_tiles * tile_floats(RS);
			const uint32_t tiles = kp / TILE;
			auto fetch_piece = [&](uint32_t tile) -> bf16x8 { return *(const bf16x8*)(lds + (size_t)tile * tile_floats(RS) + packed_half(col, h)); };
			auto step = [&](bf16x8& fetch_into, uint32_t t_new, f32x16 (&acc_new)[P], const bf16x8& use, f32x16 (&acc_old)[P], uint32_t tile_old) {
				fetch_into = fetch_piece(min(t_new + 1, tiles - 1));
				__builtin_amdgcn_sched_barrier(0);
#pragma unroll
				for (int i = 0; i < P; ++i) {
					acc_new[P - 1 - i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(use, b[P - 1 - i].hi[0], acc_new[0], 0, 0, 0);
					__builtin_amdgcn_sched_barrier(0);
					track_tile<true, false>(acc_old[i], st[i], tile_old, neg_inf);
					__builtin_amdgcn_sched_barrier(0);
					if (i == 0) {
						fetch_norms(acc_old[0], lds_norms, min(t_new + 1, tiles - 1), h);
						__builtin_amdgcn_sched_barrier(0);
					}
				}
			};
			bf16x8 o0 = fetch_piece(0), o1 = fetch_piece(min(1u, tiles - 1));
			fetch_norms(acc0[0], lds_norms, 0, h);
			fetch_norms(acc1[0], lds_norms, min(1u, tiles - 1), h);
#pragma unroll
			for (int p = P - 1; p >= 0; --p) acc0[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(o0, b[p].hi[0], acc0[0], 0, 0, 0);
			uint32_t t = 0; /* acc0 holds tile t, not yet tracked; o1 and acc1[0] hold the centroid parts and norms of tile t + 1 */
			while (t + 2 < tiles) {
				step(o0, t + 1, acc1, o1, acc0, t);
				step(o1, t + 2, acc0, o0, acc1, t + 1);
				t += 2;
			}
			if (t + 1 < tiles) {
#pragma unroll
				for (int p = P - 1; p >= 0; --p) acc1[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(o1, b[p].hi[0], acc1[0], 0, 0, 0);
#pragma unroll
				for (int p = 0; p < P; ++p) track_tile<true, false>(acc0[p], st[p], t, neg_inf);
#pragma unroll
				for (int p = 0; p < P; ++p) track_tile<true, false>(acc1[p], st[p], t + 1, neg_inf);
			}
			else {
#pragma unroll
				for (int p = 0; p < P; ++p) track_tile<true, false>(acc0[p], st[p], t, neg_inf);
			}
		}
		else
		for (uint32_t chunk = 0; chunk < chunks; ++chunk) {
			const uint32_t row0 = chunk * chunk_rows;
			const uint32_t rows = min(chunk_rows, kp - row0);
			/* STREAM: while this chunk is used, the next one (after the last: the first one, for the next sweep) is on
			 * its way; it is written to the other buffer once the tile steps are done */
			const uint32_t next_row0 = chunk + 1 < chunks ? row0 + chunk_rows : 0;
			const uint32_t next_rows = min(chunk_rows, kp - next_row0);
			Staged incoming;
			if (STREAM) request(incoming, next_row0, next_rows);
			const float* lds_tiles = lds + (size_t)cur * buf_floats;
			const float* lds_norms = lds_tiles + (size_t)chunk_tiles * tile_floats(RS);
			const uint32_t tiles = rows / TILE;
			const uint32_t tile0 = row0 / TILE;
			tile_step_bf16<KB, P, false, COARSE, PACKED>(lds_tiles, lds_norms, 0, col, h, b, acc0, acc1, 0, st, neg_inf);
			uint32_t t = 0; /* acc0 holds tile t, not yet tracked */
			while (t + 2 < tiles) {
				tile_step_bf16<KB, P, true, COARSE, PACKED>(lds_tiles, lds_norms, t + 1, col, h, b, acc1, acc0, tile0 + t, st, neg_inf);
				tile_step_bf16<KB, P, true, COARSE, PACKED>(lds_tiles, lds_norms, t + 2, col, h, b, acc0, acc1, tile0 + t + 1, st, neg_inf);
				t += 2;
			}
			if (t + 1 < tiles) {
				tile_step_bf16<KB, P, true, COARSE, PACKED>(lds_tiles, lds_norms, t + 1, col, h, b, acc1, acc0, tile0 + t, st, neg_inf);
#pragma unroll
				for (int p = 0; p < P; ++p) track_tile<COARSE, fine8_bf16<KB>()>(acc1[p], st[p], tile0 + t + 1, neg_inf);
			}
			else {
#pragma unroll
				for (int p = 0; p < P; ++p) track_tile<COARSE, fine8_bf16<KB>()>(acc0[p], st[p], tile0 + t, neg_inf);
			}
			if (STREAM) {
				/* the other buffer was last read one chunk ago, before the barrier that ended that chunk */
				commit(incoming, cur ^ 1u, next_rows);
				__syncthreads();
				cur ^= 1u;
			}
		}

#pragma unroll
		for (int p = 0; p < P; ++p) {
			const float o1 = __shfl_xor(st[p].m1, 32);
			const float o2 = __shfl_xor(st[p].m2, 32);
			const uint32_t ot = (uint32_t)__shfl_xor((int)st[p].tile, 32);
			const bool win = st[p].m1 < o1 || (st[p].m1 == o1 && h == 0);
			uint32_t idx;
			float first, second;
			if constexpr (SNAP) {
				/* the leading tile's 16 results are in registers: the winner's row and the runner-up among them; the half-wave
				 * that holds the smaller minimum decides, everything outside its 16 rows is bounded below by W */
				float v1 = __builtin_inff(), v2 = __builtin_inff();
				uint32_t rbest = 0;
#pragma unroll
				for (int r = 0; r < SNAP_ROWS; ++r) {
					const float v = snap[p][r];
					v2 = __builtin_amdgcn_fmed3f(v1, v2, v);
					const bool lt = v < v1;
					rbest = lt ? (uint32_t)r : rbest;
					v1 = lt ? v : v1;
				}
				const uint32_t mine_idx = st[p].tile * TILE + 8 * (rbest / 4) + 4 * h + (rbest % 4);
				const uint32_t oi = (uint32_t)__shfl_xor((int)mine_idx, 32);
				const float ov1 = __shfl_xor(v1, 32), ov2 = __shfl_xor(v2, 32);
				const float W = win ? fminf(o1, st[p].m2) : fminf(st[p].m1, o2);
				idx = win ? mine_idx : oi;
				first = win ? v1 : ov1;
				second = fminf(win ? v2 : ov2, W);
			}
			else if (COARSE) {
				/* refinement of the winning group of 8 or 16 rows (see assign_mfma_impl.h); the rows are re-evaluated with
				 * v_dot2c_f32_bf16 on the same three products, so the error bound of the MFMA results covers them */
				constexpr bool FINE8 = fine8_bf16<KB>();
				constexpr int ROWS = FINE8 ? 8 : 16;
				const uint32_t code = win ? st[p].tile : ot;
				const uint32_t ts = FINE8 ? code >> 1 : code;      /* tile */
				const uint32_t sub = FINE8 ? 2 * (code & 1u) : 0u; /* first group of 4 rows of the tracked group */
				const uint32_t wh = win ? h : 1u - h;
				const float W = win ? fminf(o1, st[p].m2) : fminf(st[p].m1, o2);
				const float* tile_base = STREAM ? packed + (size_t)ts * tile_floats(RS) : lds + (size_t)ts * tile_floats(RS);
				const float* norm_base = STREAM ? norms + ts * NORM_TILE : lds + (size_t)chunk_tiles * tile_floats(RS) + ts * NORM_TILE;
				/* all rows of the group are requested before the first one is used: one round trip to the local data share
				 * (or to global memory) per point tile instead of one per row, which was most of the 15 000 cycles this phase
				 * took per 96 points */
				constexpr int UNITS = PACKED ? 1 : 2 * KB; /* 16-byte pieces of a row this half-wave multiplies */
				constexpr int BATCH = UNITS >= 4 ? 4 : ROWS;  /* rows requested together (their pieces wait in registers) */
				f32x4 group_norms[ROWS / 4];
#pragma unroll
				for (int g = 0; g < ROWS / 4; ++g) group_norms[g] = *(const f32x4*)(norm_base + 8 * (sub + g) + 4 * wh);
				float tot[ROWS];
#pragma unroll
				for (int r0 = 0; r0 < ROWS; r0 += BATCH) {
					bf16x8 piece[BATCH][UNITS];
#pragma unroll
					for (int r = 0; r < BATCH; ++r) {
						const uint32_t row = 8 * (sub + (r0 + r) / 4) + 4 * wh + ((r0 + r) % 4);
						const float* at = tile_base + (PACKED ? packed_half(row, h) : row * RS);
#pragma unroll
						for (int u = 0; u < UNITS; ++u) piece[r][u] = PACKED ? *(const bf16x8*)at : row_unit(at, 4 * (u / 2) + 2 * h + (u % 2));
					}
					__builtin_amdgcn_sched_barrier(0);
#pragma unroll
					for (int r = 0; r < BATCH; ++r) tot[r0 + r] = pieces_dot_bf16<KB, PACKED>(piece[r], b[p]);
					__builtin_amdgcn_sched_barrier(0);
				}
				float v1 = __builtin_inff(), v2 = __builtin_inff();
				uint32_t rbest = 0;
#pragma unroll
				for (int g = 0; g < ROWS / 4; ++g) {
					const f32x4 c2 = group_norms[g];
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
			/* the certificate (certificate.h): the norms of the parts of the point that the products drop */
			float xsq, tau;
			if constexpr (PACKED) {
				const float other = __shfl_xor(x2[p], 32);
				xsq = h == 0 ? x2[p] : other;
				tau = cert_tau(kd, xsq, h == 0 ? other : x2[p], cert);
			}
			else if constexpr (LEVEL1) {
				xsq = x2[p];
				tau = cert_tau(kd, xsq, xlow[p] + __shfl_xor(xlow[p], 32), cert);
			}
			else {
				float xmid2 = 0.0f;
#pragma unroll
				for (int kb = 0; kb < KB; ++kb) {
					const bf16x8 xm = b[p].mid[kb];
					xmid2 = KMX_DOT2_PAIR(xmid2, xm, xm, 0); xmid2 = KMX_DOT2_PAIR(xmid2, xm, xm, 1);
					xmid2 = KMX_DOT2_PAIR(xmid2, xm, xm, 2); xmid2 = KMX_DOT2_PAIR(xmid2, xm, xm, 3);
				}
				xmid2 += __shfl_xor(xmid2, 32);
				xsq = x2[p];
				tau = cert_tau(kd, xsq, xmid2, cert);
			}
			const float along = along_m[p];
			const uint32_t slot = base + p * TILE + col;
			const bool mine = h == 0 && slot < n;
			const uint32_t pt = LISTED ? (mine ? listed.list[2 * (size_t)slot] : 0u) : slot;
			if constexpr (SLICED) {
			idx += slice.row_base;
			if (slice.mode & CARRY_IN) {
				/* the smallest two of both pairs; on equal values either leader will do: such a point is not decided here */
				const uint32_t ci = mine ? slice.carried[pt] : 0u;
				const float cf = mine ? __uint_as_float(slice.carried[(size_t)n + pt]) : 0.0f;
				const float cs = mine ? __uint_as_float(slice.carried[2 * (size_t)n + pt]) : 0.0f;
				const bool theirs = cf <= first;
				second = fminf(fminf(cs, second), theirs ? first : cf);
				idx = theirs ? ci : idx;
				first = theirs ? cf : first;
			}
			if (slice.mode & CARRY_OUT) {
				if (mine) {
					slice.carried[pt] = idx;
					slice.carried[(size_t)n + pt] = __float_as_uint(first);
					slice.carried[2 * (size_t)n + pt] = __float_as_uint(second);
				}
				continue;
			}
			}
			const bool decided = (second - first > tau) && (xsq + c2max > 1e-30f);
			if (mine) assignment[pt] = idx < all_k ? idx : 0u;
			const bool flag = mine && !decided;
			const unsigned long long mask = __ballot(flag);
			if (mask) {
				const uint32_t add = (uint32_t)__builtin_popcountll(mask);
				if (flagged + add > FLAG_CAP) flush_flags();
				if (flag) {
					const uint32_t at = 2 * (flagged + __builtin_popcountll(mask & ((1ull << lane) - 1ull)));
					flag_list[wave][at] = pt;
					/* kd_unmoved > 0: for kernels that evaluate in the frame of the data (certificate.h) */
					flag_list[wave][at + 1] = kd_unmoved > 0.0f
						? screening_threshold(cert_unmoved_threshold(first, tau, xsq, along, c2max, frame_m2, frame_norm, kd_unmoved), 0.0f)
						: screening_threshold(first, tau);
				}
				flagged += add;
			}
		}
	};

	static_assert(!PACKED || KB == 1, "the packed form is one block of 16 slots");
	auto load_points = [&](SplitPoints<KB> (&bb)[P], float (&xs)[P], float (&xa)[P], uint32_t first, [[maybe_unused]] float* xlp = nullptr) {
		if constexpr (PACKED) {
			load_packed_points<P, LD, VEC>(bb, xs, data, stride, first, col, h, dim, n, frame);
#pragma unroll
			for (int p = 0; p < P; ++p) xa[p] = 0.0f; /* (the thresholds of the packed rows stay in the moved frame) */
		}
		else load_split_points<KB, P, LD, VEC, (KB > 4), LISTED, LEVEL1>(bb, xs, xa, data, stride, first, col, h, dim, n, frame_lds, listed.list, xlp);
	};

	/*
	 * A work-group takes the units blockIdx.x, blockIdx.x + gridDim.x, ... (8 items of P tiles of 32 points each). With
	 * resident centroids its wavefronts take those items one at a time from a counter in LDS instead of a fixed eighth
	 * each: the matrix pipe of a SIMD serves its older wavefront first, so with equal shares the first four wavefronts of a
	 * work-group were done after 70 % of the kernel's time and the other four swept the rest alone (measured with the
	 * cycle counter: 440 k against 632 k cycles). (One global counter for all wavefronts was worse than either: 32768
	 * returning atomics on one address take 14 ns each, longer than the whole sweep.) The next item is claimed, and its
	 * points requested, before the current one is swept. Streamed centroids keep equal shares: every wavefront of the
	 * work-group has to arrive at the barrier of every chunk, so all of them sweep the same number of times.
	 */
	const uint32_t my_units = blockIdx.x < units ? (units - blockIdx.x + gridDim.x - 1) / gridDim.x : 0u;
	/* The listed points of a second level are few units per work-group (14 % of N = 2M points: 567 units for 256
	 * work-groups, three for some and two for the others): there the work-groups share the ITEMS evenly, a contiguous
	 * range each (N = 2M, d = 32, k = 1024: 0.077 -> 0.072 ms). */
	constexpr bool EVEN_ITEMS = LISTED && !STREAM;
	const uint32_t all_items = (n + P * TILE - 1) / (P * TILE);
	const uint32_t item0 = (uint32_t)((uint64_t)blockIdx.x * all_items / gridDim.x);
	const uint32_t item1 = (uint32_t)((uint64_t)(blockIdx.x + 1) * all_items / gridDim.x);
	const uint32_t items = EVEN_ITEMS ? item1 - item0 : STREAM ? my_units : my_units * MFMA_WAVES;
	uint32_t static_item = 0;
	auto claim = [&]() -> uint32_t {
		if (STREAM) return static_item++;
		uint32_t item = 0;
		if (lane == 0) item = atomicAdd(&claimed, 1u);
		return item; /* lane 0's value; made uniform by the caller when it is needed */
	};
	auto uniform = [&](uint32_t v) -> uint32_t { return STREAM ? v : (uint32_t)__builtin_amdgcn_readfirstlane((int)v); };
	/* first point of an item: unit blockIdx.x + (item / 8) gridDim.x, slice item % 8 (streamed: the wavefront's own slice of unit `item`) */
	auto first_point = [&](uint32_t item) -> uint32_t {
		if (EVEN_ITEMS) return (item0 + item) * P * TILE;
		const uint32_t unit = blockIdx.x + (STREAM ? item : item / MFMA_WAVES) * gridDim.x;
		const uint32_t slice = STREAM ? wave : item % MFMA_WAVES;
		return (unit * MFMA_WAVES + slice) * P * TILE;
	};
	if (PREFETCH) {
		/* one set of split operands; the raw coordinates of the next item travel while the current one is swept */
		RawPoints<KB, PACKED> raw[P];
		SplitPoints<KB> b0[P];
		float xx0[P], xm0[P];
		auto request_points = [&](uint32_t first) {
			if constexpr (PACKED) request_packed_points<P, LD, VEC>(raw, data, stride, first, col, dim, n);
			else request_split_points<KB, P, LD, VEC, LISTED>(raw, data, stride, first, col, h, dim, n, listed.list);
		};
		[[maybe_unused]] float xl0[P];
		auto convert_points = [&]() {
			if constexpr (PACKED) {
				convert_packed_points<P>(b0, xx0, raw, h, frame);
#pragma unroll
				for (int p = 0; p < P; ++p) xm0[p] = 0.0f;
			}
			else convert_split_points<KB, P, LEVEL1>(b0, xx0, xm0, raw, frame_lds, h, xl0);
		};
		uint32_t item = uniform(claim());
		uint32_t next = uniform(claim());
		if (item < items) {
			request_points(first_point(item));
			convert_points();
		}
		while (item < items) {
			const uint32_t after = claim();
			if (next < items) request_points(first_point(next));
			if constexpr (LEVEL1) sweep(b0, xx0, xm0, first_point(item), xl0);
			else sweep(b0, xx0, xm0, first_point(item));
			item = next;
			next = uniform(after);
			if (item < items) convert_points();
		}
	}
	else {
		SplitPoints<KB> b0[P];
		float xx0[P], xm0[P];
		[[maybe_unused]] float xl0[P];
		uint32_t item = uniform(claim());
		while (item < items) {
			const uint32_t after = claim();
			if constexpr (LEVEL1) {
				load_points(b0, xx0, xm0, first_point(item), xl0);
				sweep(b0, xx0, xm0, first_point(item), xl0);
			}
			else {
				load_points(b0, xx0, xm0, first_point(item));
				sweep(b0, xx0, xm0, first_point(item));
			}
			item = uniform(after);
		}
	}
	if (flagged) flush_flags();
}

/*
 * The screen of the exact pass: a second sweep over the queued points only. Their rows lie in a compact AoS block
 * (row e of the block = entry e of the queue, `dim` floats apart) with the threshold the first sweep gave them
 * (its best ranking value + tau). The same MFMAs on the same operands reproduce the ranking values a[j] of the first
 * sweep, and every centroid with a[j] <= threshold -- the only ones that can win or tie the serial comparison, two
 * or three of k -- is noted as a (row, centroid) pair for the kernel that evaluates the serial arithmetic. A NaN
 * a[j] and an infinite threshold (values the sweep could not cover) pass the screen. Per tile the lane only takes
 * the minimum of its 16 results and compares it with the threshold; the pairs are picked out on the rare hit.
 * Every work item has a slice of the pair list to itself (no atomics); pairs beyond it (many coincident centroids)
 * are evaluated when the wavefront hands its pairs over.
 * The centroid operands are read from global memory (they stay in the caches; this kernel sees a small share of
 * the points), one wavefront per P tiles of 32 rows.
 */
/* the rare pair beyond its slice's capacity; not inlined, so that the sweep's registers are not sized for it */
static __device__ __attribute__((noinline)) void evaluate_pair_of_row(const float* __restrict__ rows, uint32_t dim, const float* __restrict__ means_t,
                                                                      uint32_t kp, uint32_t row, uint32_t j, unsigned long long* __restrict__ keys)
{
	evaluate_pair<KMX_AOS>(rows, dim, means_t, dim, kp, row, j, &keys[row]);
}

template <int KB, int P, bool PACKED = false>
__global__ void __launch_bounds__(SCREEN_WAVES * WAVE) __attribute__((amdgpu_waves_per_eu((KB <= 3 || KB == 8) ? 2 : 1)))
screen_bf16_kernel(const float* __restrict__ rows, const float* __restrict__ packed, const float* __restrict__ norms,
                   const float* __restrict__ means_t, const uint32_t* __restrict__ row_queue, const uint32_t* __restrict__ row_count,
                   uint32_t* __restrict__ pairs, uint32_t* __restrict__ item_pairs,
                   unsigned long long* __restrict__ keys, uint32_t dim, uint32_t k, uint32_t kp)
{
	static_assert(!PACKED || KB == 1, "the packed form is one block of 16 slots");
	constexpr uint32_t RS = row_floats<KB, PACKED>();
	constexpr int G = KB < 4 ? KB : 4; /* blocks of 16 dimensions whose centroid operands travel together */
	constexpr int GROUPS = KB / G;     /* 1, 2 or 4 */
	static_assert(KB % G == 0 && (GROUPS == 1 || GROUPS % 2 == 0), "operand groups");
	constexpr uint32_t unit_rows = P * TILE;
	constexpr uint32_t SLICE = SCREEN_SLICE_PER_ROW * unit_rows; /* pairs an item can note */
	const uint32_t lane = threadIdx.x & (WAVE - 1);
	const uint32_t col = lane & 31, h = lane >> 5;
	const uint32_t count = row_count[0];
	const uint32_t tiles = kp / TILE;
	const uint32_t waves = gridDim.x * SCREEN_WAVES;
	const ScreenItems work = screen_items(count, unit_rows, tiles, waves);
	Frame frame = { { 0.0f, 0.0f, 0.0f, 0.0f } }; /* PACKED: the frame of the first sweep */
	if constexpr (PACKED) {
#pragma unroll
		for (int j = 0; j < 4; ++j) frame.m[j] = norms[frame_offset(kp) + j];
	}

	struct Operands { bf16x8 hi[G], mid[G]; };

	/* the pairs a wavefront notes wait in LDS and go to the item's slice of the list a few hundred at a time; pairs
	 * beyond the slice are evaluated then and there */
	constexpr uint32_t HIT_LIST = 256;
	__shared__ uint32_t hit_list[SCREEN_WAVES][2 * HIT_LIST];
	const uint32_t wave = threadIdx.x / WAVE;
	uint32_t listed = 0, written = 0; /* wave-uniform: pairs in LDS, pairs of the current item handed over */
	uint32_t* slice = pairs;
	auto flush = [&]() {
		__builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
		__builtin_amdgcn_wave_barrier();
		for (uint32_t i = lane; i < listed; i += WAVE) {
			const uint32_t row = hit_list[wave][2 * i], j = hit_list[wave][2 * i + 1];
			if (written + i < SLICE) { slice[2 * (written + i)] = row; slice[2 * (written + i) + 1] = j; }
			else evaluate_pair_of_row(rows, dim, means_t, kp, row, j, keys);
		}
		__builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
		__builtin_amdgcn_wave_barrier();
		written += listed;
		listed = 0;
	};

	for (uint32_t item = blockIdx.x * SCREEN_WAVES + threadIdx.x / WAVE; item < work.items; item += waves) {
		const uint32_t base = (item / work.parts) * unit_rows;
		const uint32_t tile_begin = (item % work.parts) * work.part_tiles, tile_end = min(tiles, tile_begin + work.part_tiles);
		slice = pairs + 2 * (size_t)item * SLICE;
		written = 0;
		SplitPoints<KB> b[P];
		float xx[P];
		if constexpr (PACKED) load_packed_points<P, KMX_AOS, false>(b, xx, rows, dim, base, col, h, dim, count, frame);
		else {
			float along[P]; /* (not needed here: the thresholds of these rows are values of the moved frame) */
			load_split_points<KB, P, KMX_AOS, false, false>(b, xx, along, rows, dim, base, col, h, dim, count, norms + frame_offset(kp));
			__builtin_amdgcn_sched_barrier(0); /* (the operands of the first tiles are not requested before the rows are split) */
		}
		float thr[P];
		bool valid[P];
#pragma unroll
		for (int p = 0; p < P; ++p) {
			const uint32_t row = base + p * TILE + col;
			valid[p] = row < count;
			thr[p] = valid[p] ? __uint_as_float(row_queue[2 * (size_t)row + 1]) : 0.0f;
		}

		auto fetch = [&](Operands& o, uint32_t tile, int group) {
			const float* arow = packed + (size_t)tile * tile_floats(RS) + (PACKED ? packed_half(col, h) : col * RS);
#pragma unroll
			for (int i = 0; i < G; ++i) {
				o.hi[i] = PACKED ? *(const bf16x8*)arow : row_unit(arow, 4 * (group * G + i) + 2 * h);
				if (!PACKED) o.mid[i] = row_unit(arow, 4 * (group * G + i) + 2 * h + 1);
			}
		};
		auto fetch_norms = [&](f32x16& c, uint32_t tile) { /* |c|^2 of the 16 rows this lane receives */
#pragma unroll
			for (int g = 0; g < 4; ++g) {
				const f32x4 v = *(const f32x4*)(norms + tile * NORM_TILE + 8 * g + 4 * h);
				c[4 * g] = v.x; c[4 * g + 1] = v.y; c[4 * g + 2] = v.z; c[4 * g + 3] = v.w;
			}
		};
		auto screen = [&](const f32x16& a, int p, uint32_t tile) {
			float t = a[0]; /* NaN-propagating minimum of the lane's 16 results */
#pragma unroll
			for (int r = 1; r < 16; ++r) t = __builtin_elementwise_minimum(t, a[r]);
			const bool near = valid[p] && !(t > thr[p]);
			if (__builtin_amdgcn_ballot_w64(near) == 0) return;
			const uint32_t row = base + p * TILE + col;
#pragma unroll
			for (int r = 0; r < 16; ++r) {
				const uint32_t j = tile * TILE + 8 * (r / 4) + 4 * h + (r % 4);
				const bool hit = near && j < k && !(a[r] > thr[p]);
				const unsigned long long mask = __builtin_amdgcn_ballot_w64(hit);
				if (mask == 0) continue;
				const uint32_t more = (uint32_t)__popcll(mask);
				if (listed + more > HIT_LIST) flush();
				if (hit) {
					const uint32_t slot = listed + (uint32_t)__popcll(mask & ((1ull << lane) - 1ull));
					hit_list[wave][2 * slot] = row;
					hit_list[wave][2 * slot + 1] = j;
				}
				listed += more;
			}
		};

		f32x16 acc[P], norms_next;
		fetch_norms(norms_next, tile_begin);
		/* the MFMAs of one operand group (the order of tile_step_bf16: hi*mid, mid*hi, hi*hi per block) */
		auto compute = [&](const Operands& o, uint32_t tile, auto group_c) {
			constexpr int group = decltype(group_c)::value;
			if (group == 0) {
#pragma unroll
				for (int p = 0; p < P; ++p) acc[p] = norms_next;
				if (tile + 1 < tile_end) fetch_norms(norms_next, tile + 1);
			}
			if constexpr (PACKED) { /* one MFMA holds every product of the row (load_packed_points) */
#pragma unroll
				for (int p = 0; p < P; ++p) acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(o.hi[0], b[p].hi[0], acc[p], 0, 0, 0);
			}
			else
#pragma unroll
			for (int i = 0; i < G; ++i) {
#pragma unroll
				for (int p = 0; p < P; ++p) acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(o.hi[i], b[p].mid[group * G + i], acc[p], 0, 0, 0);
#pragma unroll
				for (int p = 0; p < P; ++p) acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(o.mid[i], b[p].hi[group * G + i], acc[p], 0, 0, 0);
#pragma unroll
				for (int p = 0; p < P; ++p) acc[p] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(o.hi[i], b[p].hi[group * G + i], acc[p], 0, 0, 0);
			}
			if (group == GROUPS - 1) {
#pragma unroll
				for (int p = 0; p < P; ++p) screen(acc[p], p, tile);
			}
		};

		/* two operand buffers: while one feeds the MFMAs the other one is on its way from the caches */
		Operands o0, o1;
		fetch(o0, tile_begin, 0);
		if constexpr (GROUPS == 1) {
			for (uint32_t tile = tile_begin; tile < tile_end; tile += 2) {
				if (tile + 1 < tile_end) fetch(o1, tile + 1, 0);
				compute(o0, tile, std::integral_constant<int, 0>());
				if (tile + 2 < tile_end) fetch(o0, tile + 2, 0);
				if (tile + 1 < tile_end) compute(o1, tile + 1, std::integral_constant<int, 0>());
			}
		}
		else {
			for (uint32_t tile = tile_begin; tile < tile_end; ++tile) {
				fetch(o1, tile, 1);
				compute(o0, tile, std::integral_constant<int, 0>());
				if constexpr (GROUPS == 2) {
					if (tile + 1 < tile_end) fetch(o0, tile + 1, 0);
					compute(o1, tile, std::integral_constant<int, 1>());
				}
				else {
					fetch(o0, tile, 2);
					compute(o1, tile, std::integral_constant<int, 1>());
					fetch(o1, tile, 3);
					compute(o0, tile, std::integral_constant<int, 2>());
					if (tile + 1 < tile_end) fetch(o0, tile + 1, 0);
					compute(o1, tile, std::integral_constant<int, 3>());
				}
			}
		}
		flush();
		if (lane == 0) item_pairs[item] = min(written, SLICE);
	}
}

template <int KB> struct ScreenShape { static constexpr int P = KB <= 4 ? 2 : 1; };

template <int KB>
static int launch_screen_bf16_kb(const float* rows, const Workspace* ws, const uint32_t* row_queue, const uint32_t* row_count,
                                 uint32_t* pairs, uint32_t* item_pairs, unsigned long long* keys, uint32_t dim, uint32_t k, uint32_t kp,
                                 const DeviceInfo& dev, uint32_t* waves)
{
	auto kernel = screen_bf16_kernel<KB, ScreenShape<KB>::P>;
	if constexpr (KB == 1) {
		if (packed_rows(dim)) kernel = screen_bf16_kernel<KB, ScreenShape<KB>::P, true>;
	}
	/* as many wavefronts as the device holds at once: the partition of the work counts on all of them running together */
	int per_cu = 1;
	KMX_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, (const void*)kernel, (int)(SCREEN_WAVES * WAVE), 0));
	const uint32_t grid = std::min<uint32_t>(dev.compute_units * (uint32_t)std::max(1, per_cu), SCREEN_MAX_WAVES / SCREEN_WAVES);
	*waves = grid * SCREEN_WAVES;
	KMX_LAUNCH_KERNEL(kernel, dim3(grid), dim3(SCREEN_WAVES * WAVE), 0, stream(),
	                   rows, ws->packed_means, ws->norms, ws->means_t, row_queue, row_count, pairs, item_pairs, keys, dim, k, kp);
	KMX_LAUNCH_CHECK("screen_bf16_kernel");
	return KMX_OK;
}

/* static LDS of assign_bf16_kernel: the flag lists, wave_max (4 x MFMA_WAVES words) and the frame of the rows */
template <int KB, bool PACKED> constexpr uint32_t sweep_static_lds_bytes()
{
	return (2 * FLAG_CAP * MFMA_WAVES + 4 * MFMA_WAVES + (PACKED ? 4 : KB * KBLOCK)) * 4;
}

/*
 * What a sweep is about to be launched with, checked on the host against what the kernel assumes: every offset the
 * kernel forms from these numbers -- the packed rows and norms of each chunk or slice, the frame behind the norms, the
 * two LDS buffers, the staged pieces, the values carried between slices, the queue -- must lie inside its allocation.
 * A kernel that runs off one of them faults the GPU for everybody; a launch refused here costs an error message.
 */
struct SweepPlan {
	uint32_t kb, rs, kp, k, n, chunk_rows, slices, lds_bytes, static_bytes, grid;
	bool stream_mode, packed_form, wide;
};

inline int check_sweep_plan(const SweepPlan& p, const Workspace* ws, const DeviceInfo& dev, const void* data, bool vec)
{
#define KMX_PLAN(cond) do { if (!(cond)) return fail(KMX_ERR_DEVICE, "assign (split-bf16 MFMA): launch refused, the plan breaks \"%s\" (dim blocks %u, k %u, kp %u, n %u, chunk rows %u, slices %u, LDS %u + %u)", \
	#cond, p.kb, p.k, p.kp, p.n, p.chunk_rows, p.slices, p.lds_bytes, p.static_bytes); } while (0)
	const uint32_t tile_words = tile_floats(p.rs);
	KMX_PLAN(p.kp % TILE == 0 && p.kp >= p.k && p.kp - p.k < TILE);
	KMX_PLAN(p.chunk_rows > 0 && p.chunk_rows % TILE == 0 && p.chunk_rows <= p.kp);
	KMX_PLAN(tile_words % 4 == 0 && NORM_TILE % 4 == 0);                                  /* 16-byte copies of tiles and norms */
	KMX_PLAN(p.grid >= 1 && p.n >= 1);
	KMX_PLAN((uint64_t)p.lds_bytes + p.static_bytes <= dev.lds_bytes);
	KMX_PLAN(ws->packed_means && (size_t)(p.kp / TILE) * tile_words <= ws->packed_cap);  /* the last chunk or slice ends with the block */
	KMX_PLAN(ws->norms && split_norms_floats(p.kp) <= ws->norms_cap);
	KMX_PLAN(p.packed_form || (p.kb * KBLOCK <= FRAME_DIMS && FRAME_DIMS + 2 <= FRAME_FLOATS)); /* the frame read behind the norms */
	KMX_PLAN(ws->queue && 2 * (size_t)p.n <= ws->queue_cap && ws->counters);
	KMX_PLAN(!vec || ((uintptr_t)data & 15) == 0);
	const uint32_t chunk_tiles = p.chunk_rows / TILE;
	if (p.slices > 1) {
		KMX_PLAN(!p.stream_mode && p.slices <= SLICED_MAX_SLICES);
		KMX_PLAN(ws->carried && 3 * (size_t)p.n <= ws->carried_cap);
		KMX_PLAN((uint64_t)(p.slices - 1) * p.chunk_rows < p.kp);                         /* the last slice is not empty */
		KMX_PLAN((uint64_t)chunk_tiles * (tile_words + NORM_TILE) * 4 <= p.lds_bytes);
	}
	else if (!p.stream_mode) {
		KMX_PLAN(p.chunk_rows == p.kp);
		KMX_PLAN((uint64_t)chunk_tiles * (tile_words + NORM_TILE) * 4 <= p.lds_bytes);
	}
	else {
		KMX_PLAN((uint64_t)2 * chunk_tiles * (tile_words + NORM_TILE) * 4 <= p.lds_bytes); /* two buffers */
		KMX_PLAN(chunk_tiles * NORM_TILE / 4 <= MFMA_WAVES * WAVE);                        /* one 16-byte piece of norms per lane */
		if (!p.wide)
			KMX_PLAN((uint64_t)chunk_tiles * tile_words / 4 <= (uint64_t)STAGE_VECS * MFMA_WAVES * WAVE); /* a chunk staged in registers */
		/* every chunk, the short last one too: whole tiles inside the block */
		for (uint32_t row0 = 0; row0 < p.kp; row0 += p.chunk_rows) {
			const uint32_t rows = std::min(p.chunk_rows, p.kp - row0);
			KMX_PLAN(rows % TILE == 0 && packed_row(row0, p.rs) + (size_t)(rows / TILE) * tile_words <= ws->packed_cap);
			KMX_PLAN((size_t)(row0 / TILE + rows / TILE) * NORM_TILE <= split_norms_offset(p.kp));
		}
	}
#undef KMX_PLAN
	return KMX_OK;
}

/* point tiles per wavefront and sweep, and whether the next sweep's points are prefetched: bounded by the register file */
template <int KB> struct SplitSweepShape {
	static constexpr int P = KB <= 8 ? 2 : 1; /* (rows of 65 to 128 dimensions: 128 registers of split operands; measured 6 % faster than one tile, whose centroid operands serve half the MFMAs) */
	static constexpr bool PREFETCH = KB <= 2;
};

template <int KB, int LD, bool VEC, bool PACKED = false>
static int launch_bf16_t(const AssignArgs& a, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev, uint32_t kp, float kd)
{
	constexpr uint32_t RS = row_floats<KB, PACKED>();
	constexpr int P = PACKED ? 4 : SplitSweepShape<KB>::P; /* one MFMA per tile: four point tiles share the centroid operand and the norms */
	/* resident centroids and rows of 17 to 32 dimensions: a third point tile fits the registers (255, no spills; the
	 * streamed kernel would spill) and the LDS reads of a step serve 18 MFMAs instead of 12: 0.348 against 0.356 ms at
	 * N = 2M, d = 32, k = 1024 */
	constexpr int PR = (!PACKED && KB == 2 && KMX_SNAPSHOT_FROM_KB > 2) ? 3 : P; /* a third point tile fits where the tracking keeps no snapshot */
	constexpr bool PF = SplitSweepShape<KB>::PREFETCH;
	uint32_t budget = exec->shared_mem_bytes ? std::min(exec->shared_mem_bytes, dev.lds_bytes) : dev.lds_bytes;
	const uint32_t static_bytes = sweep_static_lds_bytes<KB, PACKED>();
	const uint32_t tile_bytes = (tile_floats(RS) + NORM_TILE) * 4;
	if (budget < static_bytes + tile_bytes) return fail(KMX_ERR_UNSUPPORTED, "assign (split-bf16 MFMA): LDS budget of %u bytes is too small", budget);
	/* everything resident if it fits (rows up to 64 dimensions only: the wider kernels always stream); otherwise two
	 * buffers of as many tiles as fit, bounded by what a work-group carries in registers (STAGE_VECS) */
	uint32_t chunk_rows = std::min<uint32_t>(kp, (budget - static_bytes) / tile_bytes * TILE);
	bool stream_mode = KB > 4 || chunk_rows < kp;
	/* Rows of 17 to 64 dimensions whose centroids do not fit: slices of centroids that do, one launch of the resident kernel
	 * each (see CentroidSlice), when the points are many enough to pay for the launches. The resident kernels hand out their
	 * items dynamically and keep the pipelined step; the streamed one has a barrier per chunk and item. (N = 1M: d = 48,
	 * k = 1024 0.373 -> 0.270 ms; d = 32, k = 2048 0.429 -> 0.350 ms, k = 4096 no difference; SoA points gain as much. Rows
	 * of up to 16 dimensions stream as fast as they sweep resident centroids.) */
	uint32_t slices = 1;
	if (stream_mode && KB >= 2 && KB <= 4 && !PACKED && a.n >= SLICED_MIN_POINTS) {
		const uint32_t tiles = kp / TILE, fit = chunk_rows / TILE;
		const uint32_t wanted = (tiles + fit - 1) / fit;
		if (wanted <= (KB < 4 ? SLICED_MAX_SLICES : LD == KMX_AOS ? SLICED_MAX_SLICES_WIDE : 1u)) {
			slices = wanted;
			chunk_rows = (tiles + slices - 1) / slices * TILE; /* equal slices; the last one may be shorter */
			stream_mode = false;
			int rc = reserve_carried(ws, 3 * (size_t)a.n);
			if (rc) return rc;
		}
	}
	if (stream_mode) {
		const uint32_t by_lds = (budget - static_bytes) / (2 * tile_bytes);
		const uint32_t by_regs = (uint32_t)STAGE_VECS * MFMA_WAVES * WAVE * 16 / (tile_floats(RS) * 4);
		const uint32_t by_norms = MFMA_WAVES * WAVE * 4 / NORM_TILE;
		const uint32_t chunk_tiles = std::min({ by_lds, by_regs, by_norms, kp / TILE });
		if (chunk_tiles == 0) return fail(KMX_ERR_UNSUPPORTED, "assign (split-bf16 MFMA): two tiles of %u-dimension rows do not fit the LDS budget of %u bytes", KBLOCK * KB, budget);
		chunk_rows = chunk_tiles * TILE;
	}
	const uint32_t swept_tiles = (slices > 1 ? chunk_rows : kp) / TILE;
	/* per-tile tracking pays from COARSE_MIN_TILES tiles on where a refinement follows the sweep; the snapshot needs none
	 * (N = 2-4M: d = 16, k = 256 0.219 -> 0.174 ms; d = 32, k = 256 0.150 -> 0.127 ms, k = 128 0.105 -> 0.096 ms; two tiles,
	 * k = 64: 0.108 -> 0.110 ms, left with the row-by-row tracking) */
	constexpr uint32_t SNAPSHOT_MIN_TILES = 3;
	const uint32_t coarse_from = (snapshot_sweep<KB, false, true, PACKED>() && !stream_mode) ? SNAPSHOT_MIN_TILES : COARSE_MIN_TILES;
	const bool coarse = swept_tiles >= coarse_from && !wide_rows_sweep<KB>(); /* (the wide-row step tracks single rows) */
	const uint32_t lds_bytes = (stream_mode ? 2u : 1u) * (chunk_rows / TILE) * tile_bytes;
	const uint32_t unit_points = MFMA_WAVES * (stream_mode ? P : PR) * TILE;
	const uint32_t units = (a.n + unit_points - 1) / unit_points;
	void (*kernel)(const float*, size_t, const float*, const float*, uint32_t*, uint32_t*, uint32_t*,
	               uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, float, float, uint32_t, float) = nullptr;
	void (*sliced_kernel)(const float*, size_t, const float*, const float*, uint32_t*, uint32_t*, uint32_t*,
	                      uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, float, float, uint32_t, float, CentroidSlice) = nullptr;
	if constexpr (KB == 4) {
		if (slices > 1) sliced_kernel = assign_bf16_kernel<KB, PR, LD, VEC, false, false, PF, PACKED, CentroidSlice>;
	}
	else if constexpr (KB >= 2 && KB <= 3 && !PACKED) {
		if (slices > 1) sliced_kernel = coarse ? assign_bf16_kernel<KB, PR, LD, VEC, false, true, PF, PACKED, CentroidSlice> : assign_bf16_kernel<KB, PR, LD, VEC, false, false, PF, PACKED, CentroidSlice>;
	}
	if constexpr (KB == 4) {
		kernel = stream_mode ? assign_bf16_kernel<KB, P, LD, VEC, true, false, PF, PACKED> : assign_bf16_kernel<KB, PR, LD, VEC, false, false, PF, PACKED>;
	}
	else if constexpr (KB <= 4) {
		if (stream_mode) kernel = coarse ? assign_bf16_kernel<KB, P, LD, VEC, true, true, PF, PACKED> : assign_bf16_kernel<KB, P, LD, VEC, true, false, PF, PACKED>;
		else kernel = coarse ? assign_bf16_kernel<KB, PR, LD, VEC, false, true, PF, PACKED> : assign_bf16_kernel<KB, PR, LD, VEC, false, false, PF, PACKED>;
	}
	else {
		kernel = assign_bf16_kernel<KB, P, LD, VEC, true, false, PF>;
	}
	/* two levels: hi * hi for everybody, then the three products for the points that level could not settle */
	constexpr bool TWO_LEVEL_WIDE = KB == 16; /* rows of 129 to 256 dimensions: the wide-row step */
	constexpr bool TWO_LEVEL_BUILT = (KB == 2 && !PACKED && PF) || TWO_LEVEL_WIDE;
	constexpr int P1 = TWO_LEVEL_WIDE ? 1 : PR; /* point tiles per wavefront in the first level (two tiles of hi parts would fit the registers of 256-dimension rows by count, but the compiler spills 300 to 700 of them) */
	[[maybe_unused]] void (*level1_kernel)(const float*, size_t, const float*, const float*, uint32_t*, uint32_t*, uint32_t*,
	                                      uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, float, float, uint32_t, float, LevelOne) = nullptr;
	[[maybe_unused]] void (*level2_kernel)(const float*, size_t, const float*, const float*, uint32_t*, uint32_t*, uint32_t*,
	                                      uint32_t, uint32_t, uint32_t, uint32_t, uint32_t, float, float, uint32_t, float, ListedPoints) = nullptr;
	bool two_level = false;
	if constexpr (TWO_LEVEL_BUILT) {
		const int mode = two_level_mode(); /* kmx_set_two_level_sweep: 0 never, 1 where it pays, 2 wherever the kernels allow it */
		two_level = (TWO_LEVEL_WIDE ? stream_mode : (!stream_mode && coarse)) && slices == 1 && a.two_level && mode != 0 &&
		            (mode == 2 || (swept_tiles >= TWO_LEVEL_MIN_TILES && a.n >= KMX_TWO_LEVEL_MIN_POINTS));
		if constexpr (TWO_LEVEL_WIDE) {
			level1_kernel = assign_bf16_kernel<KB, P1, LD, VEC, true, false, PF, PACKED, LevelOne>;
			level2_kernel = assign_bf16_kernel<KB, P, LD, VEC, true, false, PF, PACKED, ListedPoints>;
		}
		else {
			level1_kernel = assign_bf16_kernel<KB, PR, LD, VEC, false, true, PF, PACKED, LevelOne>;
			level2_kernel = assign_bf16_kernel<KB, PR, LD, VEC, false, true, PF, PACKED, ListedPoints>;
		}
	}
	if (two_level) {
		int rc = reserve_listed(ws, 2 * (size_t)a.n);
		if (rc) return rc;
	}
	const void* launched = slices > 1 ? (const void*)sliced_kernel : (const void*)kernel;
	KMX_HIP(hipFuncSetAttribute(launched, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
	int per_cu = 1;
	KMX_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, launched, (int)(MFMA_WAVES * WAVE), lds_bytes));
	per_cu = std::max(1, std::min(per_cu, 4));
	const uint32_t grid = std::min(units, dev.compute_units * (uint32_t)per_cu);
	exec->block_count = grid;
	const float kd_unmoved = a.unmoved_thresholds ? cert_kd_unmoved(a.dim) : 0.0f;
	int rc = KMX_OK;
	if (!sizing_only()) {
		const SweepPlan plan = { (uint32_t)KB, RS, kp, a.k, a.n, chunk_rows, slices, lds_bytes, static_bytes, grid, stream_mode, PACKED, wide_rows_sweep<KB>() };
		if ((rc = check_sweep_plan(plan, ws, dev, a.data, VEC))) return rc;
		if (slices > 1 ? !sliced_kernel : !kernel) return fail(KMX_ERR_DEVICE, "assign (split-bf16 MFMA): no kernel instance for this plan");
	}
	if ((rc = profile_begin(0))) return rc;
	if (two_level) {
		if constexpr (TWO_LEVEL_BUILT) {
			if (!sizing_only() && (!ws->listed || ws->listed_cap < 2 * (size_t)a.n)) return fail(KMX_ERR_DEVICE, "assign (split-bf16 MFMA): no list for the two levels");
			KMX_HIP(hipFuncSetAttribute((const void*)level1_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
			KMX_HIP(hipFuncSetAttribute((const void*)level2_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
			/* level 1: its "queue" is the list, its counter the list's length; thresholds mean nothing there */
			const float kd1 = kd - cert_kd_split(a.dim) + cert_kd_level1(a.dim);
			const uint32_t unit_points1 = MFMA_WAVES * (stream_mode ? P1 : PR) * TILE;
			const uint32_t grid1 = std::min((a.n + unit_points1 - 1) / unit_points1, dev.compute_units * (uint32_t)per_cu);
			KMX_LAUNCH_KERNEL(level1_kernel, dim3(grid1), dim3(MFMA_WAVES * WAVE), lds_bytes, stream(),
			                   a.data, a.stride, ws->packed_means, ws->norms, a.assignment, ws->listed, ws->counters + LISTED_COUNTER,
			                   a.dim, a.k, kp, a.n, chunk_rows, kd1, -__builtin_inff(), 0xFFFFFFFFu, 0.0f, LevelOne{ 0u });
			KMX_LAUNCH_CHECK("assign_bf16_kernel (first level)");
			/* level 2: the listed points only; as many work-groups as the device runs at once, those without work leave */
			const ListedPoints listed = { ws->listed, ws->counters + LISTED_COUNTER };
			KMX_LAUNCH_KERNEL(level2_kernel, dim3(std::min(grid, dev.compute_units * (uint32_t)per_cu)), dim3(MFMA_WAVES * WAVE), lds_bytes, stream(),
			                   a.data, a.stride, ws->packed_means, ws->norms, a.assignment, ws->queue, ws->counters,
			                   a.dim, a.k, kp, a.n, chunk_rows, kd, -__builtin_inff(), a.shifted_cap, kd_unmoved, listed);
			KMX_LAUNCH_CHECK("assign_bf16_kernel (second level)");
		}
	}
	else if (slices == 1) {
		KMX_LAUNCH_KERNEL(kernel, dim3(grid), dim3(MFMA_WAVES * WAVE), lds_bytes, stream(),
		                   a.data, a.stride, ws->packed_means, ws->norms, a.assignment, ws->queue, ws->counters,
		                   a.dim, a.k, kp, a.n, chunk_rows, kd, -__builtin_inff(), a.shifted_cap, kd_unmoved);
		KMX_LAUNCH_CHECK("assign_bf16_kernel");
	}
	else {
		for (uint32_t s = 0; s < slices; ++s) {
			const uint32_t row0 = s * chunk_rows;
			const uint32_t rows = std::min(chunk_rows, kp - row0);
			const CentroidSlice slice = { ws->norms, ws->carried, a.k, kp, row0, (s > 0 ? CARRY_IN : 0u) | (s + 1 < slices ? CARRY_OUT : 0u) };
			if (row0 >= kp || rows == 0 || rows % TILE != 0) return fail(KMX_ERR_DEVICE, "assign (split-bf16 MFMA): slice %u of %u is empty or ragged", s, slices);
			/* (the kernel's view: `rows` resident centroids, all of them one chunk) */
			KMX_LAUNCH_KERNEL(sliced_kernel, dim3(grid), dim3(MFMA_WAVES * WAVE), lds_bytes, stream(),
			                   a.data, a.stride, ws->packed_means + packed_row(row0, RS), ws->norms + (size_t)(row0 / TILE) * NORM_TILE,
			                   a.assignment, ws->queue, ws->counters,
			                   a.dim, std::min(a.k - std::min(a.k, row0), rows), rows, a.n, rows, kd, -__builtin_inff(), a.shifted_cap, kd_unmoved, slice);
			KMX_LAUNCH_CHECK("assign_bf16_kernel (a slice of the centroids)");
		}
	}
	return profile_end(0);
}

template <int KB>
static int launch_bf16_kb(const AssignArgs& a, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev, uint32_t kp, float kd)
{
	const bool aligned = a.dim % 4 == 0 && a.stride % 4 == 0 && ((uintptr_t)a.data % 16) == 0;
	if constexpr (KB == 1) {
		if (packed_rows(a.dim)) {
			if (a.layout == KMX_SOA) return launch_bf16_t<KB, KMX_SOA, false, true>(a, exec, ws, dev, kp, kd);
			if (aligned) return launch_bf16_t<KB, KMX_AOS, true, true>(a, exec, ws, dev, kp, kd);
			return launch_bf16_t<KB, KMX_AOS, false, true>(a, exec, ws, dev, kp, kd);
		}
	}
	if (a.layout == KMX_SOA) return launch_bf16_t<KB, KMX_SOA, false>(a, exec, ws, dev, kp, kd);
	if (aligned) return launch_bf16_t<KB, KMX_AOS, true>(a, exec, ws, dev, kp, kd);
	return launch_bf16_t<KB, KMX_AOS, false>(a, exec, ws, dev, kp, kd);
}

} // namespace kmx

#endif
