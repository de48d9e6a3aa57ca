/*
 * C ABI entry points of libkmx_hip.so: device / memory / stream / event plumbing, argument
 * validation and dispatch to the kernel launchers. Declared in include/kmx.h.
 */
#include "kmx_internal.h"
#include "certificate.h"

#include <cstdarg>
#include <cstring>

namespace kmx {

static thread_local char g_error[512] = "";
static hipStream_t g_stream = nullptr;
static DeviceInfo g_dev;
static Workspace g_ws;

int fail(int code, const char* fmt, ...)
{
	va_list ap;
	va_start(ap, fmt);
	vsnprintf(g_error, sizeof(g_error), fmt, ap);
	va_end(ap);
	return code;
}

void clear_error() { g_error[0] = '\0'; }

/* while a graph is being recorded every launch goes to the library's own capture stream */
static hipStream_t g_capture_stream = nullptr;
static bool g_capturing = false;

hipStream_t stream() { return g_capturing ? g_capture_stream : g_stream; }
bool recording_graph() { return g_capturing; }

#define KMX_NOT_WHILE_CAPTURING(name)                                                                          \
	do {                                                                                                       \
		if (g_capturing) return fail(KMX_ERR_INVALID_ARGUMENT, name ": not allowed between kmx_graph_begin and kmx_graph_end"); \
	} while (0)

static bool g_sizing = false;
bool sizing_only() { return g_sizing; }

static bool g_profiling = false;
static bool g_profiling_suspended = false;
void suspend_profiling(bool suspended) { g_profiling_suspended = suspended; }
static hipEvent_t g_prof[2][2] = { { nullptr, nullptr }, { nullptr, nullptr } };
static bool g_prof_valid[2] = { false, false };

int profile_begin(int which)
{
	if (!g_profiling || g_capturing || g_profiling_suspended || g_sizing) return KMX_OK;
	for (int i = 0; i < 2; ++i)
		if (!g_prof[which][i]) KMX_HIP(hipEventCreate(&g_prof[which][i]));
	KMX_HIP(hipEventRecord(g_prof[which][0], g_stream));
	return KMX_OK;
}

int profile_end(int which)
{
	if (!g_profiling || g_capturing || g_profiling_suspended || g_sizing) return KMX_OK;
	KMX_HIP(hipEventRecord(g_prof[which][1], g_stream));
	g_prof_valid[which] = true;
	return KMX_OK;
}

int device_info(const DeviceInfo** out)
{
	int dev = 0;
	KMX_HIP(hipGetDevice(&dev));
	if (g_dev.device != dev) {
		hipDeviceProp_t p;
		KMX_HIP(hipGetDeviceProperties(&p, dev));
		g_dev.device = dev;
		g_dev.compute_units = (uint32_t)p.multiProcessorCount;
		g_dev.lds_bytes = (uint32_t)p.sharedMemPerBlock;
		g_dev.max_threads = (uint32_t)p.maxThreadsPerBlock;
	}
	*out = &g_dev;
	return KMX_OK;
}

int workspace(Workspace** ws)
{
	if (!g_ws.counters) {
		KMX_HIP(hipMalloc((void**)&g_ws.counters, 16 * sizeof(uint32_t)));
		KMX_HIP(hipMemset(g_ws.counters, 0, 16 * sizeof(uint32_t)));
	}
	*ws = &g_ws;
	return KMX_OK;
}

template <typename T>
static int grow(T** ptr, size_t* cap, size_t want)
{
	if (want <= *cap) return KMX_OK;
	if (g_capturing)
		return fail(KMX_ERR_INVALID_ARGUMENT, "the call needs a larger work space, which cannot be allocated while a graph is recorded: "
		                                      "make the same call once before kmx_graph_begin");
	if (*ptr) {
		/* earlier launches may still be reading the old buffer */
		KMX_HIP(hipStreamSynchronize(g_stream));
		KMX_HIP(hipFree(*ptr));
		*ptr = nullptr;
		*cap = 0;
	}
	KMX_HIP(hipMalloc((void**)ptr, want * sizeof(T)));
	*cap = want;
	return KMX_OK;
}

int reserve_queue(Workspace* ws, size_t entries) { return grow(&ws->queue, &ws->queue_cap, entries); }

int reserve_packed(Workspace* ws, size_t packed_floats, size_t norm_floats, size_t transposed_floats)
{
	int rc = grow(&ws->packed_means, &ws->packed_cap, packed_floats);
	if (rc) return rc;
	rc = grow(&ws->norms, &ws->norms_cap, norm_floats);
	if (rc) return rc;
	return grow(&ws->means_t, &ws->means_t_cap, transposed_floats);
}

int reserve_partials(Workspace* ws, size_t floats)
{
	if (ws->fixed) {
		if (floats <= ws->partials_cap) return KMX_OK;
		return fail(KMX_ERR_UNSUPPORTED, "the call needs %zu bytes of scratch memory for its partial sums; the entry point that allocates nothing holds %zu",
		            floats * sizeof(float), ws->partials_cap * sizeof(float));
	}
	return grow(&ws->partials, &ws->partials_cap, floats);
}
int reserve_fused_assignment(Workspace* ws, size_t entries) { return grow(&ws->fused_assignment, &ws->fused_cap, entries); }
int reserve_bucket_sizes(Workspace* ws, size_t entries) { return grow(&ws->bucket_sizes, &ws->bucket_cap, entries); }
int reserve_f64(double** ptr, size_t* cap, size_t doubles) { return grow(ptr, cap, doubles); }
int reserve_rows_copy(Workspace* ws, size_t floats) { return grow(&ws->rows_copy, &ws->rows_copy_cap, floats); }
int reserve_queued_rows(Workspace* ws, size_t rows, size_t dim, size_t extra_words)
{
	int rc = grow(&ws->queued_rows, &ws->queued_rows_cap, rows * dim);
	if (rc) return rc;
	return grow(&ws->queued_index, &ws->queued_index_cap, 4 * rows + extra_words);
}

int reserve_carried(Workspace* ws, size_t words) { return grow(&ws->carried, &ws->carried_cap, words); }
int reserve_listed(Workspace* ws, size_t words) { return grow(&ws->listed, &ws->listed_cap, words); }
static int g_two_level_mode = 1;
int two_level_mode() { return g_two_level_mode; }

static int release_workspace()
{
	if (g_ws.queue) KMX_HIP(hipFree(g_ws.queue));
	if (g_ws.counters) KMX_HIP(hipFree(g_ws.counters));
	if (g_ws.packed_means) KMX_HIP(hipFree(g_ws.packed_means));
	if (g_ws.norms) KMX_HIP(hipFree(g_ws.norms));
	if (g_ws.means_t) KMX_HIP(hipFree(g_ws.means_t));
	if (g_ws.partials) KMX_HIP(hipFree(g_ws.partials));
	if (g_ws.fused_assignment) KMX_HIP(hipFree(g_ws.fused_assignment));
	if (g_ws.bucket_sizes) KMX_HIP(hipFree(g_ws.bucket_sizes));
	if (g_ws.rows_copy) KMX_HIP(hipFree(g_ws.rows_copy));
	if (g_ws.queued_rows) KMX_HIP(hipFree(g_ws.queued_rows));
	if (g_ws.queued_index) KMX_HIP(hipFree(g_ws.queued_index));
	if (g_ws.carried) KMX_HIP(hipFree(g_ws.carried));
	if (g_ws.listed) KMX_HIP(hipFree(g_ws.listed));
	g_ws = Workspace();
	return release_f64_workspace();
}

/* counterpart of fillZeros (reference kernels.cu:12-17), grid-stride, 128-bit stores where aligned */
__global__ void fill_zero_kernel(uint32_t* __restrict__ p, size_t count)
{
	size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
	size_t step = (size_t)gridDim.x * blockDim.x;
	for (; i < count; i += step) p[i] = 0u;
}

} // namespace kmx

using namespace kmx;

static int g_last_assign_variant = -1; /* concrete variant of the last assignment sweep (kmx_assign_f32, or the ranking stage of kmx_assign_f64) */

namespace kmx {

int dispatch_assign(int variant, const AssignArgs& a, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev, int* chosen)
{
	if (variant == KMX_ASSIGN_BEST) {
		/* counterpart of BestCachedAssignmentKernel::run (reference kernels.cu:706-717): pick by shape.
		 * Measured (one call, exact pass included, N = 2-4M): the split-bf16 sweep is about twice as fast as the fp32 one
		 * wherever the sweep dominates; it hands 2-3 times as many points to the exact pass. Rows of 16 dimensions and more:
		 * ahead or level at every k (d = 64, k = 16: 0.25 against 0.32 ms; d = 32, k = 33: 0.108 against 0.137 ms; d = 16,
		 * k = 32: level). Rows of 5 to 15 dimensions: ahead from three centroid tiles on (d = 5, k = 100: 0.153 against
		 * 0.181 ms; k = 1024: 0.279 against 0.385 ms), behind with one or two (d = 8, k = 64: 0.120 against 0.116 ms).
		 * Rows of 2 to 4 dimensions: all their products fit one MFMA per tile (the packed form), which beats the fp32 sweep
		 * from 128 centroids on (512 for two dimensions; 1.14 against 1.53 ms per iteration at N = 4M, d = 4, k = 4096).
		 * The plain-VALU variant, which reads a small centroid block through the scalar cache, wins with at most 16
		 * centroids of at most 16 dimensions (d = 16, k = 16: 0.086 against 0.105 ms; d = 8, k = 8: 0.049 against 0.080 ms)
		 * and loses from there on (d = 16, k = 32: 0.128 against 0.110 ms; d = 32, k = 16: 0.183 against 0.161 ms).
		 * The double path, which pays more per queued point: the packed form from 256 centroids on, where its exact pass
		 * works in batches (N = 4M doubles, d = 4, k = 4096: 1.09 against 1.64 ms per call; d = 3, k = 1024: 0.40 against
		 * 0.52 ms; d = 4, k = 256: 0.25 against 0.29 ms; d = 2, k = 1024: level); the plain-VALU variant
		 * up to 32 centroids (N = 2M doubles, d = 16, k = 32: 0.134 against 0.153 ms; d = 32, k = 16: level); the split
		 * sweep from there as for floats (d = 64, k = 48: 0.547 against 0.625 ms; d = 32, k = 33: 0.302 against 0.326 ms;
		 * d = 5, k = 1024: 0.427 against 0.438 ms). */
		const bool packed_wins = (a.dim >= 3 && a.dim <= 4 && a.k >= (a.ranking_only ? 256u : 128u)) || (a.dim == 2 && a.k >= 512);
		const bool split_wins = a.dim >= 16 || (a.dim >= 5 && a.k > 64);
		const bool few = a.ranking_only ? a.k <= 32 : (a.k <= 16 && a.dim <= 16);
		if (few && lds_fma_supports(a, dev) && lds_fma_reads_through_scalar_cache(a)) variant = KMX_ASSIGN_LDS_FMA;
		else if (bf16_supports(a, dev) && (split_wins || packed_wins)) variant = KMX_ASSIGN_MFMA_BF16X3;
		else if (mfma_supports(a, dev)) variant = KMX_ASSIGN_MFMA;
		else if (lds_fma_supports(a, dev)) variant = KMX_ASSIGN_LDS_FMA;
		else variant = KMX_ASSIGN_BASE;
	}
	g_last_assign_variant = variant;
	if (chosen) *chosen = variant;
	switch (variant) {
	case KMX_ASSIGN_BASE:
		return launch_assign_base(a, exec);
	case KMX_ASSIGN_LDS_FMA:
		if (!lds_fma_supports(a, dev))
			return fail(KMX_ERR_UNSUPPORTED, "kmx_assign_f32: shape dim=%u k=%u is not supported by the LDS/FMA variant", a.dim, a.k);
		return launch_assign_lds_fma(a, exec, ws, dev);
	case KMX_ASSIGN_MFMA:
		if (!mfma_supports(a, dev))
			return fail(KMX_ERR_UNSUPPORTED, "kmx_assign_f32: shape dim=%u k=%u is not supported by the MFMA variant", a.dim, a.k);
		return launch_assign_mfma(a, exec, ws, dev);
	case KMX_ASSIGN_MFMA_BF16X3:
		if (!bf16_supports(a, dev))
			return fail(KMX_ERR_UNSUPPORTED, "kmx_assign_f32: shape dim=%u k=%u is not supported by the split-bf16 MFMA variant", a.dim, a.k);
		return launch_assign_bf16(a, exec, ws, dev);
	default:
		return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_assign_f32: unknown variant %d", variant);
	}
}

} // namespace kmx

extern "C" {

const char* kmx_last_error(void) { return g_error; }

int kmx_device_count(int* count)
{
	clear_error();
	if (!count) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_device_count: null pointer");
	int c = 0;
	hipError_t e = hipGetDeviceCount(&c);
	if (e != hipSuccess) { (void)hipGetLastError(); c = 0; }
	*count = c;
	return KMX_OK;
}

int kmx_set_device(int device)
{
	clear_error();
	KMX_NOT_WHILE_CAPTURING("kmx_set_device");
	int c = 0;
	if (hipGetDeviceCount(&c) != hipSuccess || c == 0) {
		(void)hipGetLastError();
		return fail(KMX_ERR_NO_DEVICE, "No HIP devices found!");
	}
	/* the work space, the cached device properties and the stream belong to the device they were made on */
	if (g_ws.counters && g_dev.device >= 0 && g_dev.device != device)
		return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_set_device: the library holds a work space on device %d; call kmx_shutdown() before moving to device %d",
		            g_dev.device, device);
	KMX_HIP(hipSetDevice(device));
	/* the address of this device's scratch array of kmx_update_f32_noalloc, now rather than inside its first call (looking
	 * it up loads the library's code onto the device, which is no work for a call that promises to allocate nothing) */
	Workspace* scratch = nullptr;
	return noalloc_workspace(&scratch);
}

int kmx_device_props(kmx_props* props)
{
	clear_error();
	if (!props) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_device_props: null pointer");
	int dev = 0;
	KMX_HIP(hipGetDevice(&dev));
	hipDeviceProp_t p;
	KMX_HIP(hipGetDeviceProperties(&p, dev));
	std::memset(props, 0, sizeof(*props));
	std::strncpy(props->name, p.name, sizeof(props->name) - 1);
	std::strncpy(props->arch, p.gcnArchName, sizeof(props->arch) - 1);
	props->compute_units = (uint32_t)p.multiProcessorCount;
	props->wavefront_size = (uint32_t)p.warpSize;
	props->max_threads_per_block = (uint32_t)p.maxThreadsPerBlock;
	props->lds_bytes_per_block = (uint32_t)p.sharedMemPerBlock;
	props->clock_khz = (uint32_t)p.clockRate;
	props->global_mem_bytes = (uint64_t)p.totalGlobalMem;
	return KMX_OK;
}

int kmx_malloc(void** dptr, size_t bytes)
{
	clear_error();
	KMX_NOT_WHILE_CAPTURING("kmx_malloc");
	if (!dptr) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_malloc: null pointer");
	*dptr = nullptr;
	if (bytes == 0) return KMX_OK;
	KMX_HIP(hipMalloc(dptr, bytes));
	return KMX_OK;
}

int kmx_free(void* dptr)
{
	clear_error();
	KMX_NOT_WHILE_CAPTURING("kmx_free");
	if (!dptr) return KMX_OK;
	{
		/* points announced with kmx_prepare_points_f64 that live in this allocation are gone with it */
		void* base = nullptr;
		size_t size = 0;
		if (hipMemGetAddressRange(&base, &size, dptr) == hipSuccess && base && size) forget_prepared_points_f64(base, size);
		else {
			(void)hipGetLastError();
			forget_prepared_points_f64(dptr, 0);
		}
	}
	KMX_HIP(hipFree(dptr));
	return KMX_OK;
}

int kmx_h2d(void* dst_device, const void* src_host, size_t bytes)
{
	clear_error();
	KMX_NOT_WHILE_CAPTURING("kmx_h2d");
	if (bytes == 0) return KMX_OK;
	if (!dst_device || !src_host) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_h2d: null pointer");
	forget_prepared_points_f64(dst_device, bytes);
	KMX_HIP(hipMemcpyAsync(dst_device, src_host, bytes, hipMemcpyHostToDevice, stream()));
	return KMX_OK;
}

int kmx_d2h(void* dst_host, const void* src_device, size_t bytes)
{
	clear_error();
	KMX_NOT_WHILE_CAPTURING("kmx_d2h");
	if (bytes == 0) return KMX_OK;
	if (!dst_host || !src_device) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_d2h: null pointer");
	KMX_HIP(hipMemcpyAsync(dst_host, src_device, bytes, hipMemcpyDeviceToHost, stream()));
	KMX_HIP(hipStreamSynchronize(stream()));
	return KMX_OK;
}

int kmx_d2d(void* dst_device, const void* src_device, size_t bytes)
{
	clear_error();
	KMX_NOT_WHILE_CAPTURING("kmx_d2d");
	if (bytes == 0) return KMX_OK;
	if (!dst_device || !src_device) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_d2d: null pointer");
	forget_prepared_points_f64(dst_device, bytes);
	KMX_HIP(hipMemcpyAsync(dst_device, src_device, bytes, hipMemcpyDeviceToDevice, stream()));
	return KMX_OK;
}

int kmx_sync(void)
{
	clear_error();
	KMX_NOT_WHILE_CAPTURING("kmx_sync");
	KMX_HIP(hipDeviceSynchronize());
	return KMX_OK;
}

int kmx_set_stream(void* hip_stream)
{
	clear_error();
	KMX_NOT_WHILE_CAPTURING("kmx_set_stream");
	g_stream = (hipStream_t)hip_stream;
	return KMX_OK;
}

int kmx_shutdown(void)
{
	clear_error();
	KMX_NOT_WHILE_CAPTURING("kmx_shutdown");
	KMX_HIP(hipDeviceSynchronize());
	return release_workspace();
}

int kmx_fill_zero_u32(void* dptr, size_t count)
{
	clear_error();
	if (count == 0) return KMX_OK;
	if (!dptr) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_fill_zero_u32: null pointer");
	forget_prepared_points_f64(dptr, count * sizeof(uint32_t));
	const unsigned block = 256;
	size_t blocks = (count + block - 1) / block;
	if (blocks > 4096) blocks = 4096;
	KMX_LAUNCH_KERNEL(fill_zero_kernel, dim3((unsigned)blocks), dim3(block), 0, stream(), (uint32_t*)dptr, count);
	KMX_LAUNCH_CHECK("fill_zero_kernel");
	return KMX_OK;
}


static int check_update_variant(const char* who, int variant, bool bucket_sum)
{
	const int base = variant & ~KMX_UPDATE_EMULATED_ATOMICS;
	if (base < KMX_UPDATE_ATOMIC_POINT || base > KMX_UPDATE_SERIAL_ORDER) return fail(KMX_ERR_INVALID_ARGUMENT, "%s: unknown variant %d", who, variant);
	if ((base == KMX_UPDATE_FAKE || base == KMX_UPDATE_FAKE_SHM) && !bucket_sum)
		return fail(KMX_ERR_INVALID_ARGUMENT, "%s: variant %d ignores its inputs; it exists for kmx_bucket_sum_f32 only", who, variant);
	if ((variant & KMX_UPDATE_EMULATED_ATOMICS) &&
	    (base == KMX_UPDATE_ATOMIC_SHM || base == KMX_UPDATE_BASE || base == KMX_UPDATE_ATOMIC_SHM2 || base == KMX_UPDATE_FAKE_SHM ||
	     base == KMX_UPDATE_SERIAL_ORDER))
		return fail(KMX_ERR_UNSUPPORTED, "%s: emulated atomics exist for the point, fine, wavefront and fake variants only", who);
	return KMX_OK;
}

static int check_layout(const char* who, const char* what, int layout, size_t stride, uint32_t count, uint32_t dim)
{
	if (layout != KMX_AOS && layout != KMX_SOA) return fail(KMX_ERR_INVALID_ARGUMENT, "%s: unknown %s layout %d", who, what, layout);
	if (layout == KMX_AOS && stride < dim) return fail(KMX_ERR_INVALID_ARGUMENT, "%s: %s stride %zu < dim %u", who, what, stride, dim);
	if (layout == KMX_SOA && stride < count) return fail(KMX_ERR_INVALID_ARGUMENT, "%s: %s stride %zu < count %u", who, what, stride, count);
	return KMX_OK;
}

int kmx_assign_f32(int variant,
                   const float* data, int layout, size_t stride,
                   const float* means, int layout_means, size_t stride_means,
                   const uint32_t* last_assignment, uint32_t* assignment,
                   uint32_t dim, uint32_t k, uint32_t n, kmx_exec_params* exec)
{
	clear_error();
	(void)last_assignment;
	if (!exec) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_assign_f32: exec is null");
	if (dim == 0 || k == 0) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_assign_f32: dim and k must be positive");
	if (n == 0) { exec->block_count = 0; return KMX_OK; }
	if (!data || !means || !assignment) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_assign_f32: null device pointer");
	int rc = check_layout("kmx_assign_f32", "data", layout, stride, n, dim);
	if (rc) return rc;
	rc = check_layout("kmx_assign_f32", "means", layout_means, stride_means, k, dim);
	if (rc) return rc;

	const DeviceInfo* dev = nullptr;
	rc = device_info(&dev);
	if (rc) return rc;
	Workspace* ws = nullptr;
	rc = workspace(&ws);
	if (rc) return rc;

	AssignArgs a{ data, layout, stride, means, layout_means, stride_means, assignment, dim, k, n };
	return dispatch_assign(variant, a, exec, ws, *dev, nullptr);
}

int kmx_reserve_f32(int assign_variant, int update_variant, int layout, int layout_means, uint32_t dim, uint32_t k, uint32_t n)
{
	clear_error();
	KMX_NOT_WHILE_CAPTURING("kmx_reserve_f32");
	if (dim == 0 || k == 0) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_reserve_f32: dim and k must be positive");
	if (n == 0) return KMX_OK;
	/* the launchers themselves say what they need: they are walked with the launches switched off, on pointers that are
	 * never followed (16-byte aligned, like buffers from kmx_malloc) */
	float* const points = (float*)(uintptr_t)4096;
	uint32_t* const words = (uint32_t*)(uintptr_t)4096;
	const size_t stride = layout == KMX_AOS ? dim : n, stride_means = layout_means == KMX_AOS ? dim : k;
	kmx_exec_params exec = { 256, 0, 0, 1, 1, 1 };
	const int last_variant = g_last_assign_variant;
	g_sizing = true;
	int rc = kmx_assign_f32(assign_variant, points, layout, stride, points, layout_means, stride_means, nullptr, words, dim, k, n, &exec);
	if (rc == KMX_OK) rc = kmx_update_f32(update_variant, points, layout, stride, words, points, layout_means, stride_means, words, dim, k, n, &exec);
	if (rc == KMX_OK) {
		Workspace* ws = nullptr;
		rc = workspace(&ws);
		if (rc == KMX_OK) rc = reserve_fused_assignment(ws, n); /* kmx_fused_f32 keeps its assignment vector in the work space */
	}
	if (rc == KMX_OK) {
		Workspace* scratch = nullptr;
		rc = noalloc_workspace(&scratch); /* kmx_update_f32_noalloc: the address of its scratch array on this device */
	}
	g_sizing = false;
	g_last_assign_variant = last_variant;
	return rc;
}

int kmx_assign_last_variant(int* variant)
{
	clear_error();
	if (!variant) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_assign_last_variant: null pointer");
	*variant = g_last_assign_variant;
	return KMX_OK;
}

int kmx_assign_last_rechecked(uint64_t* count)
{
	clear_error();
	KMX_NOT_WHILE_CAPTURING("kmx_assign_last_rechecked");
	if (!count) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_assign_last_rechecked: null pointer");
	*count = 0;
	Workspace* ws = nullptr;
	int rc = workspace(&ws);
	if (rc) return rc;
	uint32_t c = 0;
	KMX_HIP(hipMemcpyAsync(&c, ws->counters, sizeof(c), hipMemcpyDeviceToHost, stream()));
	KMX_HIP(hipStreamSynchronize(stream()));
	*count = c;
	return KMX_OK;
}

int kmx_update_f32(int variant,
                   const float* data, int layout, size_t stride,
                   const uint32_t* assignment,
                   float* means, int layout_means, size_t stride_means,
                   uint32_t* cluster_sizes,
                   uint32_t dim, uint32_t k, uint32_t n, kmx_exec_params* exec)
{
	clear_error();
	if (!exec) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_update_f32: exec is null");
	if (dim == 0 || k == 0) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_update_f32: dim and k must be positive");
	if (!means || !cluster_sizes) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_update_f32: null device pointer");
	if (n > 0 && (!data || !assignment)) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_update_f32: null device pointer");
	int rc = check_layout("kmx_update_f32", "data", layout, stride, n, dim);
	if (rc) return rc;
	rc = check_layout("kmx_update_f32", "means", layout_means, stride_means, k, dim);
	if (rc) return rc;
	rc = check_update_variant("kmx_update_f32", variant, false);
	if (rc) return rc;
	if (exec->privatized_copies == 0) exec->privatized_copies = 1;

	const DeviceInfo* dev = nullptr;
	rc = device_info(&dev);
	if (rc) return rc;
	Workspace* ws = nullptr;
	rc = workspace(&ws);
	if (rc) return rc;

	UpdateArgs u{ data, layout, stride, assignment, means, layout_means, stride_means, cluster_sizes, dim, k, n };
	return launch_update(variant, u, exec, ws, *dev);
}

int kmx_update_f32_noalloc(int variant,
                           const float* data, int layout, size_t stride,
                           const uint32_t* assignment,
                           float* means, int layout_means, size_t stride_means,
                           uint32_t* cluster_sizes,
                           uint32_t dim, uint32_t k, uint32_t n, kmx_exec_params* exec)
{
	clear_error();
	if (!exec) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_update_f32_noalloc: exec is null");
	if (dim == 0 || k == 0) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_update_f32_noalloc: dim and k must be positive");
	if (!means || !cluster_sizes) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_update_f32_noalloc: null device pointer");
	if (n > 0 && (!data || !assignment)) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_update_f32_noalloc: null device pointer");
	int rc = check_layout("kmx_update_f32_noalloc", "data", layout, stride, n, dim);
	if (rc) return rc;
	rc = check_layout("kmx_update_f32_noalloc", "means", layout_means, stride_means, k, dim);
	if (rc) return rc;
	rc = check_update_variant("kmx_update_f32_noalloc", variant, false);
	if (rc) return rc;
	if (exec->privatized_copies == 0) exec->privatized_copies = 1;

	const DeviceInfo* dev = nullptr;
	rc = device_info(&dev);
	if (rc) return rc;
	Workspace* ws = nullptr;
	rc = noalloc_workspace(&ws); /* the static scratch array of this device; set up on the first call */
	if (rc) return rc;

	UpdateArgs u{ data, layout, stride, assignment, means, layout_means, stride_means, cluster_sizes, dim, k, n };
	suspend_profiling(true);
	rc = launch_update(variant, u, exec, ws, *dev);
	suspend_profiling(false);
	return rc;
}

int kmx_bucket_sum_f32(int variant,
                       const float* data, int layout, size_t stride,
                       const uint32_t* indices,
                       float* result, int layout_result, size_t stride_result,
                       uint32_t dim, uint32_t k, uint32_t n, kmx_exec_params* exec)
{
	clear_error();
	if (!exec) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_bucket_sum_f32: exec is null");
	if (dim == 0 || k == 0) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_bucket_sum_f32: dim and k must be positive");
	if (!result) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_bucket_sum_f32: null device pointer");
	if (n > 0 && (!data || !indices)) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_bucket_sum_f32: null device pointer");
	int rc = check_layout("kmx_bucket_sum_f32", "data", layout, stride, n, dim);
	if (rc) return rc;
	rc = check_layout("kmx_bucket_sum_f32", "result", layout_result, stride_result, k, dim);
	if (rc) return rc;
	rc = check_update_variant("kmx_bucket_sum_f32", variant, true);
	if (rc) return rc;
	if (exec->privatized_copies == 0) exec->privatized_copies = 1;

	const DeviceInfo* dev = nullptr;
	rc = device_info(&dev);
	if (rc) return rc;
	Workspace* ws = nullptr;
	rc = workspace(&ws);
	if (rc) return rc;
	/* the kernels count members as they go; the counts land in a scratch array */
	rc = reserve_bucket_sizes(ws, k);
	if (rc) return rc;
	rc = kmx_fill_zero_u32(ws->bucket_sizes, k);
	if (rc) return rc;

	UpdateArgs u{ data, layout, stride, indices, result, layout_result, stride_result, ws->bucket_sizes, dim, k, n };
	u.divide = false;
	return launch_update(variant, u, exec, ws, *dev);
}

int kmx_fused_f32(int variant,
                  const float* data, int layout, size_t stride,
                  const float* means_in, float* means_out, int layout_means, size_t stride_means,
                  uint32_t* cluster_sizes,
                  uint32_t dim, uint32_t k, uint32_t n, kmx_exec_params* exec)
{
	clear_error();
	if (!exec) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_fused_f32: exec is null");
	if (variant < KMX_FUSED_TWO_PASS || variant > KMX_FUSED_BEST) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_fused_f32: unknown variant %d", variant);
	if (!means_in || !means_out || !cluster_sizes) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_fused_f32: null device pointer");
	if (means_in == means_out) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_fused_f32: means_in and means_out must differ");
	Workspace* ws = nullptr;
	int rc = workspace(&ws);
	if (rc) return rc;
	rc = reserve_fused_assignment(ws, n);
	if (rc) return rc;

	const bool one_pass_fits = fused_small_supports(dim, k, layout, stride, n);
	if (variant == KMX_FUSED_ONE_PASS && !one_pass_fits)
		return fail(KMX_ERR_UNSUPPORTED, "kmx_fused_f32: shape dim=%u k=%u is not supported by the single-pass kernel", dim, k);
	if (variant != KMX_FUSED_TWO_PASS && one_pass_fits && n > 0) {
		if (dim == 0 || k == 0) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_fused_f32: dim and k must be positive");
		if (!data) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_fused_f32: null device pointer");
		rc = check_layout("kmx_fused_f32", "data", layout, stride, n, dim);
		if (rc) return rc;
		rc = check_layout("kmx_fused_f32", "means", layout_means, stride_means, k, dim);
		if (rc) return rc;
		const DeviceInfo* dev = nullptr;
		rc = device_info(&dev);
		if (rc) return rc;
		AssignArgs a{ data, layout, stride, means_in, layout_means, stride_means, ws->fused_assignment, dim, k, n };
		rc = launch_fused_small(a, means_out, cluster_sizes, exec, ws, *dev);
		if (rc) return rc;
		UpdateArgs u{ data, layout, stride, ws->fused_assignment, means_out, layout_means, stride_means, cluster_sizes, dim, k, n };
		return launch_divide_means(u);
	}
	/* argument checks of the two halves apply unchanged (their messages name the half that objects) */
	rc = kmx_assign_f32(KMX_ASSIGN_BEST, data, layout, stride, means_in, layout_means, stride_means, nullptr, ws->fused_assignment, dim, k, n, exec);
	if (rc) return rc;
	return kmx_update_f32(KMX_UPDATE_ATOMIC_SHM, data, layout, stride, ws->fused_assignment, means_out, layout_means, stride_means,
	                      cluster_sizes, dim, k, n, exec);
}

static int g_last_iteration_passes = 0;

int kmx_iteration_f32(const float* data, int layout, size_t stride,
                      const float* means_in, float* means_out, int layout_means, size_t stride_means,
                      uint32_t* assignment, uint32_t* cluster_sizes,
                      uint32_t dim, uint32_t k, uint32_t n, kmx_exec_params* exec)
{
	clear_error();
	if (!exec) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_iteration_f32: exec is null");
	if (dim == 0 || k == 0) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_iteration_f32: dim and k must be positive");
	if (!means_in || !means_out || !cluster_sizes) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_iteration_f32: null device pointer");
	if (n > 0 && (!data || !assignment)) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_iteration_f32: null device pointer");
	if (means_in == means_out) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_iteration_f32: means_in and means_out must differ");
	g_last_iteration_passes = 2;
	if (fused_small_supports(dim, k, layout, stride, n) && n > 0) {
		int rc = check_layout("kmx_iteration_f32", "data", layout, stride, n, dim);
		if (rc) return rc;
		rc = check_layout("kmx_iteration_f32", "means", layout_means, stride_means, k, dim);
		if (rc) return rc;
		const DeviceInfo* dev = nullptr;
		rc = device_info(&dev);
		if (rc) return rc;
		Workspace* ws = nullptr;
		rc = workspace(&ws);
		if (rc) return rc;
		UpdateArgs u{ data, layout, stride, assignment, means_out, layout_means, stride_means, cluster_sizes, dim, k, n };
		rc = clear_update_outputs(u); /* the single-pass kernel accumulates into them */
		if (rc) return rc;
		AssignArgs a{ data, layout, stride, means_in, layout_means, stride_means, assignment, dim, k, n };
		a.emit_assignment = true;
		g_last_assign_variant = KMX_ASSIGN_LDS_FMA; /* the ranking of the single-pass kernel: fused multiply-adds on scalar operands */
		rc = launch_fused_small(a, means_out, cluster_sizes, exec, ws, *dev);
		if (rc) return rc;
		g_last_iteration_passes = 1;
		return launch_divide_means(u);
	}
	int rc = kmx_assign_f32(KMX_ASSIGN_BEST, data, layout, stride, means_in, layout_means, stride_means, nullptr, assignment, dim, k, n, exec);
	if (rc) return rc;
	return kmx_update_f32(KMX_UPDATE_ATOMIC_SHM, data, layout, stride, assignment, means_out, layout_means, stride_means, cluster_sizes, dim, k, n, exec);
}

int kmx_iteration_last_passes(int* passes)
{
	clear_error();
	if (!passes) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_iteration_last_passes: null pointer");
	*passes = g_last_iteration_passes;
	return KMX_OK;
}

int kmx_graph_begin(void)
{
	clear_error();
	KMX_NOT_WHILE_CAPTURING("kmx_graph_begin");
	if (!g_capture_stream) KMX_HIP(hipStreamCreateWithFlags(&g_capture_stream, hipStreamNonBlocking));
	/* work already queued on the caller's stream stays ahead of whatever the graph will do: the graph is launched
	 * on that stream; recording itself runs nothing */
	KMX_HIP(hipStreamBeginCapture(g_capture_stream, hipStreamCaptureModeRelaxed));
	g_capturing = true;
	return KMX_OK;
}

int kmx_graph_end(void** graph)
{
	clear_error();
	if (!g_capturing) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_graph_end: no recording in progress");
	g_capturing = false;
	hipGraph_t recorded = nullptr;
	hipError_t e = hipStreamEndCapture(g_capture_stream, &recorded);
	if (e != hipSuccess) {
		(void)hipGetLastError(); /* a failed recording must not poison the launch checks that follow */
		return fail(KMX_ERR_DEVICE, "hipStreamEndCapture failed: %s", hipGetErrorString(e));
	}
	if (!graph) {
		(void)hipGraphDestroy(recorded);
		return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_graph_end: null pointer");
	}
	hipGraphExec_t exec = nullptr;
	e = hipGraphInstantiate(&exec, recorded, nullptr, nullptr, 0);
	(void)hipGraphDestroy(recorded);
	if (e != hipSuccess) {
		(void)hipGetLastError();
		return fail(KMX_ERR_DEVICE, "hipGraphInstantiate failed: %s", hipGetErrorString(e));
	}
	*graph = (void*)exec;
	return KMX_OK;
}

int kmx_graph_launch(void* graph)
{
	clear_error();
	KMX_NOT_WHILE_CAPTURING("kmx_graph_launch");
	if (!graph) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_graph_launch: null graph");
	KMX_HIP(hipGraphLaunch((hipGraphExec_t)graph, g_stream));
	return KMX_OK;
}

int kmx_graph_destroy(void* graph)
{
	clear_error();
	if (!graph) return KMX_OK;
	KMX_HIP(hipGraphExecDestroy((hipGraphExec_t)graph));
	return KMX_OK;
}

int kmx_set_queued_rows_limit(size_t bytes)
{
	clear_error();
	set_queued_rows_limit(bytes);
	return KMX_OK;
}

int kmx_certificate_tau(int form, uint32_t dim, float x2, float xpart2, float c2max, float cmid2max, float crest2max, float* tau)
{
	clear_error();
	if (!tau) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_certificate_tau: null pointer");
	const CentroidBounds cb{ c2max, cmid2max, crest2max };
	switch (form) {
	case 0: *tau = cert_kd_fp32(dim) * (x2 + c2max); return KMX_OK;
	case 3: *tau = cert_kd_fma(dim) * (x2 + c2max); return KMX_OK;
	case 1: *tau = cert_tau(cert_kd_split(dim), x2, xpart2, cert_coeffs_split(cb)); return KMX_OK;
	case 2: *tau = cert_tau(cert_kd_packed(dim), x2, xpart2, cert_coeffs_packed(cb)); return KMX_OK;
	case 4: *tau = cert_tau(cert_kd_level1(dim), x2, xpart2, cert_coeffs_level1(cb)); return KMX_OK;
	case 5: /* the single-pass iteration kernels: forms 3 and 0 with the lowest xpart2 (4 or 5) bits of a value replaced by its centroid's number */
	case 6:
		if (!(xpart2 == 4.0f || xpart2 == 5.0f)) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_certificate_tau: forms 5 and 6 take 4 or 5 replaced bits in xpart2");
		*tau = ((form == 5 ? cert_kd_fma(dim) : cert_kd_fp32(dim)) + cert_kd_keyed((unsigned)xpart2)) * (x2 + c2max);
		return KMX_OK;
	default: return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_certificate_tau: unknown form %d", form);
	}
}

int kmx_certificate_unmoved_threshold(uint32_t dim, float first, float tau, float x2, float along, float c2max, float m2, float mnorm,
                                      float* threshold)
{
	clear_error();
	if (!threshold) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_certificate_unmoved_threshold: null pointer");
	*threshold = cert_unmoved_threshold(first, tau, x2, along, c2max, m2, mnorm, cert_kd_unmoved(dim));
	return KMX_OK;
}

int kmx_set_two_level_sweep(int mode)
{
	clear_error();
	if (mode < 0 || mode > 2) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_set_two_level_sweep: mode %d (0 = never, 1 = where it pays, 2 = wherever the kernels allow it)", mode);
	g_two_level_mode = mode;
	return KMX_OK;
}

int kmx_set_profiling(int enabled)
{
	clear_error();
	g_profiling = enabled != 0;
	if (!g_profiling) g_prof_valid[0] = g_prof_valid[1] = false;
	return KMX_OK;
}

int kmx_last_kernel_ms(int which, float* ms)
{
	clear_error();
	if (which < 0 || which > 1 || !ms) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_last_kernel_ms: bad argument");
	if (!g_prof_valid[which]) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_last_kernel_ms: no profiled call (kmx_set_profiling(1) first)");
	KMX_HIP(hipEventSynchronize(g_prof[which][1]));
	KMX_HIP(hipEventElapsedTime(ms, g_prof[which][0], g_prof[which][1]));
	return KMX_OK;
}

int kmx_event_create(void** event)
{
	clear_error();
	if (!event) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_event_create: null pointer");
	hipEvent_t e;
	KMX_HIP(hipEventCreate(&e));
	*event = (void*)e;
	return KMX_OK;
}

int kmx_event_destroy(void* event)
{
	clear_error();
	if (!event) return KMX_OK;
	KMX_HIP(hipEventDestroy((hipEvent_t)event));
	return KMX_OK;
}

int kmx_event_record(void* event)
{
	clear_error();
	KMX_NOT_WHILE_CAPTURING("kmx_event_record");
	if (!event) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_event_record: null event");
	KMX_HIP(hipEventRecord((hipEvent_t)event, stream()));
	return KMX_OK;
}

int kmx_event_elapsed_ms(void* start, void* stop, float* ms)
{
	clear_error();
	KMX_NOT_WHILE_CAPTURING("kmx_event_elapsed_ms");
	if (!start || !stop || !ms) return fail(KMX_ERR_INVALID_ARGUMENT, "kmx_event_elapsed_ms: null argument");
	KMX_HIP(hipEventSynchronize((hipEvent_t)stop));
	KMX_HIP(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
	return KMX_OK;
}

} // extern "C"
