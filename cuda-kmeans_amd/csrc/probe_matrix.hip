/*
 * kmx_probe_matrix_chain: one wavefront runs a chain of matrix-core instructions on operands the caller chooses and
 * hands back the raw accumulators. The certificates of the ranking sweeps (certificate.h) allow one u' = 2^-23 of the
 * running magnitude per accumulated product "for any rounding or truncation inside the matrix core"; that is a statement
 * about hardware, and this probe is how the tests hold the hardware to it: products of very different exponents inside
 * one block, cancelling pairs next to small terms, long chains -- in the instructions, operand layout and order the
 * sweeps use (assign_mfma_impl.h: v_mfma_f32_32x32x2_f32; assign_bf16_impl.h: v_mfma_f32_32x32x16_bf16; fused_small.hip:
 * v_mfma_f32_16x16x4_f32; centroids as the rows of A, points as the columns of B, the accumulator started from the norms).
 */
#include "kmx_internal.h"

namespace kmx {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4v __attribute__((ext_vector_type(4)));

/* a: 32 rows x depth (row-major), b: 32 columns x depth (each column's values contiguous), c, d: 32 x 32 row-major.
 * d[i][j] = c[i][j] + sum_q a[i][q] b[j][q], accumulated block by block in ascending q by one instruction per block. */
template <int KIND>
__global__ void __launch_bounds__(64)
matrix_chain_probe_kernel(const float* __restrict__ a, const float* __restrict__ b, const float* __restrict__ c, float* __restrict__ d,
                          uint32_t blocks)
{
	constexpr uint32_t BLOCK = KIND == 0 ? 2 : KIND == 1 ? 16 : 4;
	const uint32_t lane = threadIdx.x, col = lane & 31, h = lane >> 5;
	const uint32_t depth = blocks * BLOCK;
	if (KIND == 2) { /* the 32 x 32 result as four tiles of 16 x 16, one chain each */
		const uint32_t c16 = lane & 15, quad = lane >> 4;
		for (uint32_t ti = 0; ti < 2; ++ti)
			for (uint32_t tj = 0; tj < 2; ++tj) {
				f32x4v t;
#pragma unroll
				for (int r = 0; r < 4; ++r) t[r] = c[(16 * ti + 4 * quad + r) * 32 + 16 * tj + c16];
				for (uint32_t blk = 0; blk < blocks; ++blk)
					t = __builtin_amdgcn_mfma_f32_16x16x4f32(a[(size_t)(16 * ti + c16) * depth + blk * 4 + quad],
					                                         b[(size_t)(16 * tj + c16) * depth + blk * 4 + quad], t, 0, 0, 0);
#pragma unroll
				for (int r = 0; r < 4; ++r) d[(16 * ti + 4 * quad + r) * 32 + 16 * tj + c16] = t[r];
			}
		return;
	}
	f32x16 acc;
#pragma unroll
	for (int g = 0; g < 4; ++g) {
#pragma unroll
		for (int t = 0; t < 4; ++t) acc[4 * g + t] = c[(8 * g + 4 * h + t) * 32 + col];
	}
	for (uint32_t blk = 0; blk < blocks; ++blk) {
		if (KIND == 0) {
			const float av = a[(size_t)col * depth + blk * 2 + h], bv = b[(size_t)col * depth + blk * 2 + h];
			acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc, 0, 0, 0);
		}
		else {
			bf16x8 av, bv;
#pragma unroll
			for (int j = 0; j < 8; ++j) {
				/* the caller passes values a bf16 holds exactly: dropping the low half of the word loses nothing */
				const uint32_t aw = __float_as_uint(a[(size_t)col * depth + blk * 16 + h * 8 + j]) >> 16;
				const uint32_t bw = __float_as_uint(b[(size_t)col * depth + blk * 16 + h * 8 + j]) >> 16;
				av[j] = __builtin_bit_cast(__bf16, (unsigned short)aw);
				bv[j] = __builtin_bit_cast(__bf16, (unsigned short)bw);
			}
			acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, bv, acc, 0, 0, 0);
		}
	}
#pragma unroll
	for (int g = 0; g < 4; ++g) {
#pragma unroll
		for (int t = 0; t < 4; ++t) d[(8 * g + 4 * h + t) * 32 + col] = acc[4 * g + t];
	}
}

} // namespace kmx

using namespace kmx;

extern "C" int kmx_probe_matrix_chain(int kind, const float* a, const float* b, const float* c, float* d, uint32_t blocks)
{
	clear_error();
	if (kind < 0 || kind > 2) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_probe_matrix_chain: kind %d (0 = fp32 32x32x2, 1 = bf16 32x32x16, 2 = fp32 16x16x4)", kind);
	if (!a || !b || !c || !d) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_probe_matrix_chain: null device pointer");
	if (blocks == 0 || blocks > (1u << 20)) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_probe_matrix_chain: 1 to 2^20 blocks");
	if (kind == 0) KMX_LAUNCH_KERNEL((matrix_chain_probe_kernel<0>), dim3(1), dim3(WAVE), 0, stream(), a, b, c, d, blocks);
	else if (kind == 1) KMX_LAUNCH_KERNEL((matrix_chain_probe_kernel<1>), dim3(1), dim3(WAVE), 0, stream(), a, b, c, d, blocks);
	else KMX_LAUNCH_KERNEL((matrix_chain_probe_kernel<2>), dim3(1), dim3(WAVE), 0, stream(), a, b, c, d, blocks);
	KMX_LAUNCH_CHECK("matrix_chain_probe_kernel");
	return KMX_OK;
}
