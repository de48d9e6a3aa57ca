/*
 * Probe: throughput of LDS read-modify-write flavours on the current device.
 *
 * Counterpart of the reference's raw atomic-throughput probes (atomicFakeKernel / atomicShmFakeKernel,
 * experimental/bucketing-cuda/bucketing-cuda/kernels/kernels.cu:454-531). One work-group of 1024 lanes per
 * CU issues 4096 wavefront-level LDS operations per wavefront with five address patterns; the report is
 * cycles per wavefront instruction per CU (2.4 GHz assumed). It decided the design of the update kernels:
 * on gfx950 ds_add_f32 costs ~194 cycles whatever the pattern, ds_add_u32 4.4, a plain
 * read + add + write 8.2.
 *
 *     make -C cuda-kmeans_amd/probes && cuda-kmeans_amd/probes/lds_atomics
 */
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <cstdint>
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("%s: %s\n", #x, hipGetErrorString(e)); exit(1);} } while(0)
constexpr int ITERS = 4096;
// mode 0: ds_add_f32, 1: ds_add_u32, 2: read+add+write (non atomic), 3: ds_add_f32 via returning atomic
template <int MODE>
__global__ void __launch_bounds__(1024) k(const uint32_t* __restrict__ idx, float* out, uint32_t words)
{
	extern __shared__ float lds[];
	for (uint32_t i = threadIdx.x; i < words; i += blockDim.x) lds[i] = 0;
	__syncthreads();
	uint32_t a[8];
	for (int u = 0; u < 8; ++u) a[u] = idx[(blockIdx.x * 8 + u) * blockDim.x + threadIdx.x] % words;
	float acc = 0;
	for (int it = 0; it < ITERS / 8; ++it) {
#pragma unroll
		for (int u = 0; u < 8; ++u) {
			if (MODE == 0) unsafeAtomicAdd(&lds[a[u]], 1.0f);
			else if (MODE == 1) atomicAdd((uint32_t*)&lds[a[u]], 1u);
			else if (MODE == 2) { float v = lds[a[u]]; lds[a[u]] = v + 1.0f; }
			else acc += atomicAdd(&lds[a[u]], 1.0f);
		}
	}
	__syncthreads();
	if (lds[threadIdx.x] == 123.f || acc == 5.f) out[0] = 1;
}
int main()
{
	const uint32_t blocks = 256, threads = 1024, words = 32768;
	uint32_t* hidx = (uint32_t*)malloc(blocks * 8 * threads * 4);
	uint32_t* didx; float* out; CK(hipMalloc(&didx, blocks * 8 * threads * 4)); CK(hipMalloc(&out, 4));
	hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
	const char* pats[] = {"linear(conflict-free)", "rows32 random (kmeans d=32)", "random word", "same address per wave", "rows16 random (d=16,k=16)"};
	for (int pat = 0; pat < 5; ++pat) {
		srand(3);
		for (uint32_t b = 0; b < blocks * 8; ++b) for (uint32_t t = 0; t < threads; ++t) {
			uint32_t v;
			if (pat == 0) v = t;
			else if (pat == 1) { static uint32_t rows[32]; if (t % 32 == 0) rows[t / 32] = rand() % 1024; v = rows[t / 32] * 32 + t % 32; }
			else if (pat == 2) v = rand() % words;
			else if (pat == 3) v = (t / 64) * 64;
			else { static uint32_t rows[64]; if (t % 16 == 0) rows[t / 16] = (rand() % 4 == 0) ? rand() % 16 : 0; v = rows[t / 16] * 16 + t % 16; }
			hidx[b * threads + t] = v;
		}
		CK(hipMemcpy(didx, hidx, blocks * 8 * threads * 4, hipMemcpyHostToDevice));
		printf("pattern: %s\n", pats[pat]);
		auto run = [&](const char* name, auto kern) {
			CK(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, words * 4));
			hipLaunchKernelGGL(kern, dim3(blocks), dim3(threads), words * 4, 0, didx, out, words); CK(hipDeviceSynchronize());
			CK(hipEventRecord(e0)); hipLaunchKernelGGL(kern, dim3(blocks), dim3(threads), words * 4, 0, didx, out, words); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
			float ms; CK(hipEventElapsedTime(&ms, e0, e1));
			double cyc = ms * 1e-3 * 2.4e9;
			double wave_instr = (double)ITERS * (threads / 64);
			printf("  %-22s %8.1f us  %6.1f cycles per wave-instr per CU\n", name, ms * 1e3, cyc / wave_instr);
		};
		run("ds_add_f32", k<0>); run("ds_add_u32", k<1>); run("read+add+write", k<2>); run("ds_add_rtn_f32", k<3>);
	}
	return 0;
}
