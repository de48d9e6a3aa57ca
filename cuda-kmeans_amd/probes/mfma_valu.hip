/*
 * Probe: does VALU work hide behind fp32 MFMA on the current device?
 *
 * Every wavefront runs chains of v_mfma_f32_32x32x2_f32 with NV independent (or dependent) VALU
 * fused multiply-adds placed after each MFMA (sched_group_barrier keeps them there), at 1, 2 and 4
 * wavefronts per SIMD. The report is TFLOP/s of the MFMAs alone and cycles per MFMA per SIMD. On
 * gfx950 the times ADD UP (about 2.3-3 cycles per VALU operation on top of 64-66 per MFMA) at every
 * occupancy: fp32 MFMA does not free the vector ALUs. It decided the per-tile tracking of the assignment
 * kernel (as few VALU operations per MFMA result as possible).
 *
 *     make -C cuda-kmeans_amd/probes && cuda-kmeans_amd/probes/mfma_valu
 */
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("%s: %s\n", #x, hipGetErrorString(e)); exit(1);} } while(0)
typedef float f32x16 __attribute__((ext_vector_type(16)));
// NV = VALU ops per MFMA, fine-grained interleave forced with sched_group_barrier; CHAINS independent acc chains
template <int NV, int CHAINS, bool DEP>
__global__ void __launch_bounds__(1024) k(float* out, int iters, float seed)
{
	float a = seed + threadIdx.x, b = seed * 2 + threadIdx.x;
	f32x16 acc[CHAINS];
	for (int p = 0; p < CHAINS; ++p) for (int r = 0; r < 16; ++r) acc[p][r] = 0;
	float m[8]; for (int i = 0; i < 8; ++i) m[i] = seed * i;
	for (int it = 0; it < iters; ++it) {
#pragma unroll
		for (int s = 0; s < 16; ++s) {
#pragma unroll
			for (int p = 0; p < CHAINS; ++p) {
				acc[p] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[p], 0, 0, 0);
#pragma unroll
				for (int v = 0; v < NV; ++v) {
					if (DEP) m[0] = __builtin_fmaf(m[0], a, b);              // one serial chain
					else m[v % 8] = __builtin_fmaf(m[v % 8], a, b);          // 8 independent chains
				}
			}
		}
#pragma unroll
		for (int i = 0; i < 16 * CHAINS; ++i) { __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); if (NV) __builtin_amdgcn_sched_group_barrier(0x002, NV, 0); }
	}
	float s = 0; for (int i = 0; i < 8; ++i) s += m[i];
	for (int p = 0; p < CHAINS; ++p) for (int r = 0; r < 16; ++r) s += acc[p][r];
	if (s == 12345.f) out[0] = s;
}
int main()
{
	float* out; CK(hipMalloc(&out, 4));
	hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
	auto run = [&](const char* name, auto kern, int threads, int chains) {
		int iters = 1000, blocks = 256;
		hipLaunchKernelGGL(kern, dim3(blocks), dim3(threads), 0, 0, out, 10, 1.0f); CK(hipDeviceSynchronize());
		CK(hipEventRecord(e0)); hipLaunchKernelGGL(kern, dim3(blocks), dim3(threads), 0, 0, out, iters, 1.0f); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
		float ms; CK(hipEventElapsedTime(&ms, e0, e1));
		double mfmas = (double)blocks * (threads / 64) * iters * 16.0 * chains;
		double cyc_per_mfma_per_simd = ms * 1e-3 * 2.4e9 / (mfmas / (blocks * 4.0));
		printf("%-44s waves/SIMD %d: %7.2f ms %7.1f TFLOP/s  %6.1f cycles/MFMA/SIMD\n", name, threads / 256, ms, mfmas * 4096 / ms / 1e9, cyc_per_mfma_per_simd);
	};
	for (int thr : {256, 512, 1024}) {
		run("0 VALU, 2 chains", k<0, 2, false>, thr, 2);
		run("0 VALU, 1 chain (dependent MFMAs)", k<0, 1, false>, thr, 1);
		run("2 indep VALU per MFMA, 2 chains", k<2, 2, false>, thr, 2);
		run("4 indep VALU per MFMA, 2 chains", k<4, 2, false>, thr, 2);
		run("8 indep VALU per MFMA, 2 chains", k<8, 2, false>, thr, 2);
		run("12 indep VALU per MFMA, 2 chains", k<12, 2, false>, thr, 2);
		run("4 dep VALU per MFMA, 2 chains", k<4, 2, true>, thr, 2);
		run("8 dep VALU per MFMA, 2 chains", k<8, 2, true>, thr, 2);
	}
	return 0;
}
