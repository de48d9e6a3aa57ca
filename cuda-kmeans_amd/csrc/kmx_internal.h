/*
 * Internal declarations shared by the HIP sources of libkmx_hip.so (not part of the C ABI).
 */
#ifndef KMX_INTERNAL_H
#define KMX_INTERNAL_H

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>
#include <cstdio>

#include "kmx.h"

namespace kmx {

constexpr int WAVE = 64; /* gfx950 wavefront width */

typedef float f32x4 __attribute__((ext_vector_type(4)));

/* Records the message returned by kmx_last_error() and passes `code` through. */
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
void clear_error();

/* The stream every kernel of the library is launched on. */
hipStream_t stream();

/* Brackets the dominant kernel of a call with events when kmx_set_profiling(1) is active (which: 0 assign, 1 update). */
int profile_begin(int which);
int profile_end(int which);
/* while set, profile_begin / profile_end do nothing (they create events on first use: not for the entry point that allocates nothing) */
void suspend_profiling(bool suspended);

/* Properties of the current device, queried once. */
struct DeviceInfo {
	int device = -1;
	uint32_t compute_units = 0;
	uint32_t lds_bytes = 0;      /* LDS available to one work-group */
	uint32_t max_threads = 0;
};
int device_info(const DeviceInfo** out);

/*
 * Work space owned by the library (grown on demand, released by kmx_shutdown):
 *   recheck queue : indices of the points the fast assignment kernels hand to the exact pass
 *   counters      : [0] = queue length of the current call, [4] = length of the list between the two levels of a two-level sweep
 *   packed means  : centroids re-laid-out (scaled by -2, padded) for the fast assignment kernels
 *   norms         : |c|^2 per (padded) centroid followed by max_j |c_j|^2
 *   partials      : per-work-group partial sums/counts of the update kernels that need them
 *   queued rows   : the rows of the queued points as a compact AoS block for the exact pass, with a
 *                   queue and an assignment vector of their own (counters[1] = rows taken, counters[2] = entries left
 *                   over); the split-bf16 sweep uses the block for every layout
 */
struct Workspace {
	uint32_t* queue = nullptr;      size_t queue_cap = 0;      /* entries */
	uint32_t* counters = nullptr;                               /* 16 words */
	float* packed_means = nullptr;  size_t packed_cap = 0;     /* floats  */
	float* norms = nullptr;         size_t norms_cap = 0;      /* floats  */
	float* means_t = nullptr;       size_t means_t_cap = 0;    /* floats: exact transposed centroids [dim][kp] */
	float* partials = nullptr;      size_t partials_cap = 0;   /* floats  */
	uint32_t* fused_assignment = nullptr; size_t fused_cap = 0; /* entries: assignment vector of kmx_fused_f32 */
	uint32_t* bucket_sizes = nullptr;     size_t bucket_cap = 0; /* entries: member counts nobody asked for (kmx_bucket_sum_f32) */
	float* rows_copy = nullptr;           size_t rows_copy_cap = 0;     /* floats: AoS copy of SoA points for the tuned update */
	float* queued_rows = nullptr;         size_t queued_rows_cap = 0;   /* floats */
	uint32_t* queued_index = nullptr;     size_t queued_index_cap = 0;  /* words: per row 2 (queue) + 2 (assignment or 64-bit key), then the screen's pair counters and pairs */
	uint32_t* carried = nullptr;          size_t carried_cap = 0;       /* words: per point the leader and the two smallest ranking values over the slices of centroids swept so far */
	uint32_t* listed = nullptr;           size_t listed_cap = 0;        /* words: two per point the first level of a two-level sweep could not settle (its length: counters[LISTED_COUNTER]) */
	const float* exact_norms = nullptr; /* |c|^2 of the centroids as given, in the layout of `norms`, for the exact pass of a sweep that moved its frame (points into `norms`; null: `norms` holds them) */
	bool fixed = false; /* the work space of the entry point that allocates nothing: its buffers never grow, a call that needs more is refused */
};
int workspace(Workspace** ws);
int reserve_queue(Workspace* ws, size_t entries);
int reserve_packed(Workspace* ws, size_t packed_floats, size_t norm_floats, size_t transposed_floats);
int reserve_partials(Workspace* ws, size_t floats);
int reserve_fused_assignment(Workspace* ws, size_t entries);
int reserve_bucket_sizes(Workspace* ws, size_t entries);
int reserve_rows_copy(Workspace* ws, size_t floats);
int reserve_queued_rows(Workspace* ws, size_t rows, size_t dim, size_t extra_words);
int reserve_carried(Workspace* ws, size_t words);
int reserve_listed(Workspace* ws, size_t words);
int two_level_mode(); /* kmx_set_two_level_sweep */
constexpr uint32_t LISTED_COUNTER = 4; /* word of Workspace::counters that holds the length of Workspace::listed */

#define KMX_HIP(call)                                                                                         \
	do {                                                                                                      \
		hipError_t kmx_e_ = (call);                                                                           \
		if (kmx_e_ != hipSuccess)                                                                             \
			return ::kmx::fail(KMX_ERR_DEVICE, "%s failed: %s", #call, hipGetErrorString(kmx_e_));           \
	} while (0)

/* Every kernel of the library is launched through this: while kmx_reserve_f32 walks the launchers to size the work space
 * (sizing_only()), the reservations happen and the kernels do not run. */
bool sizing_only();
#define KMX_LAUNCH_KERNEL(...)                                                                                \
	do {                                                                                                      \
		if (!::kmx::sizing_only()) hipLaunchKernelGGL(__VA_ARGS__);                                           \
	} while (0)

#define KMX_LAUNCH_CHECK(name)                                                                                \
	do {                                                                                                      \
		hipError_t kmx_e_ = hipGetLastError();                                                                \
		if (kmx_e_ != hipSuccess)                                                                             \
			return ::kmx::fail(KMX_ERR_DEVICE, "launch of %s failed: %s", name, hipGetErrorString(kmx_e_));  \
	} while (0)

/* Element address in either layout (layout_policies.hpp:22-25 SoA, :46-49 AoS of the reference). */
template <int LAYOUT>
__host__ __device__ __forceinline__ size_t elem(size_t stride, size_t idx, size_t dim)
{
	return LAYOUT == KMX_AOS ? idx * stride + dim : dim * stride + idx;
}

/* Argument bundle of one assignment call after validation. */
struct AssignArgs {
	const float* data; int layout; size_t stride;
	const float* means; int layout_means; size_t stride_means;
	uint32_t* assignment;
	uint32_t dim, k, n;
	/* The double-precision entry point runs the float sweeps on rounded copies of its inputs as a ranking stage:
	 * kd_extra widens the certificate by the effect of that rounding, and ranking_only leaves the queue of
	 * uncertified points (pairs of point number and threshold, length in counters[0]) to the caller. */
	float kd_extra = 0.0f;
	bool ranking_only = false;
	/* The split-bf16 sweep may work in a frame moved to the middle of the centroids (shift_rows). Where the screen follows,
	 * the thresholds of the queue stay values of that frame, which only the screen shares, so entries from position
	 * shifted_cap on -- those the screen has no rows for -- get an infinite threshold; where the other kernels of the exact
	 * pass follow, the sweep takes the thresholds back to the frame of the data (unmoved_thresholds). */
	bool shift_rows = false;
	uint32_t shifted_cap = 0xFFFFFFFFu;
	bool unmoved_thresholds = false;
	/* rows of 17 to 32 dimensions: the sweep may run in two levels (one product per dimension for all points, three for
	 * those the first level cannot settle); off for measurements of the one-level sweep */
	bool two_level = true;
	/* the single-pass fused kernel: write the result of every point to `assignment`, not only those of the exact pass */
	bool emit_assignment = false;
};

struct UpdateArgs {
	const float* data; int layout; size_t stride;
	const uint32_t* assignment;
	float* means; int layout_means; size_t stride_means;
	uint32_t* cluster_sizes;
	uint32_t dim, k, n;
	bool divide = true; /* false: leave the member sums in `means` (the update micro-benchmark) */
};

/* kmx_runtime.hip: runs one assignment variant (KMX_ASSIGN_BEST: chosen by shape); *chosen receives the concrete variant */
int dispatch_assign(int variant, const AssignArgs& a, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev, int* chosen);

/* assign_exact.hip */
int launch_assign_base(const AssignArgs& a, kmx_exec_params* exec);
/* Re-evaluates the points listed in ws->queue[0 .. counters[0]) with the serial arithmetic, reading the
 * exact transposed centroids ws->means_t ([dim][kp]) that pack_means wrote for this call. */
int launch_recheck(const AssignArgs& a, Workspace* ws, uint32_t kp);
void set_queued_rows_limit(size_t bytes); /* bound of the block of copied rows */
/* The exact pass behind the split-bf16 sweep for k >= 128 and rows of more than 32 dimensions: the queued rows are copied into a compact block, a second
 * split-bf16 sweep over them notes the (row, centroid) pairs within the threshold (assign_bf16.hip), and one lane
 * per pair evaluates the serial arithmetic. */
int launch_recheck_screened(const AssignArgs& a, Workspace* ws, uint32_t kp, const DeviceInfo& dev);
uint32_t screened_rows_cap(const AssignArgs& a); /* queue entries the screened exact pass has rows for */
int launch_screen_bf16(const float* rows, const Workspace* ws, const uint32_t* row_queue, const uint32_t* row_count,
                       uint32_t* pairs, uint32_t* item_pairs, unsigned long long* keys, uint32_t dim, uint32_t k, uint32_t kp,
                       const DeviceInfo& dev, uint32_t* waves);
uint32_t screen_unit_rows(uint32_t dim);

/* assign_mfma.hip / assign_lds_fma.hip: return KMX_ERR_UNSUPPORTED (without message side effects
 * beyond kmx_last_error) when the shape does not fit the variant. */
/* shared by both fast variants: packed centroids (-2c rows of dp floats, kp rows), norms, transposed copy, empty queue */
int launch_pack_means(const AssignArgs& a, Workspace* ws, uint32_t dp, uint32_t kp, uint32_t moved); /* FRAME_KEPT, FRAME_MOVED, FRAME_MOVED_IF_FAR (assign_mfma_impl.h) */
bool mfma_supports(const AssignArgs& a, const DeviceInfo& dev);
int launch_assign_mfma(const AssignArgs& a, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev);
bool bf16_supports(const AssignArgs& a, const DeviceInfo& dev);
int launch_assign_bf16(const AssignArgs& a, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev);
bool lds_fma_supports(const AssignArgs& a, const DeviceInfo& dev);
bool lds_fma_reads_through_scalar_cache(const AssignArgs& a); /* a handful of centroids: no LDS staging */
int launch_assign_lds_fma(const AssignArgs& a, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev);

/* update.hip */
/* the work space of kmx_update_f32_noalloc on the current device: `partials` is the library's static scratch array */
int noalloc_workspace(Workspace** ws);
bool recording_graph(); /* between kmx_graph_begin and kmx_graph_end */
int launch_update(int variant, const UpdateArgs& u, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev);
int launch_divide_means(const UpdateArgs& u);
int clear_update_outputs(const UpdateArgs& u); /* means (replica 0) and cluster sizes := 0 in one launch */

/* update_ordered.hip: KMX_UPDATE_SERIAL_ORDER for floats and doubles -- stable counting sort of the point numbers by
 * cluster, then one lane per (cluster, coordinate) adds the members in ascending point order and divides: the bits of
 * the serial loop. Scratch (chunk histograms, cluster starts, the sorted point numbers: about n + 2^21 words) is taken
 * from ws->partials. */
template <typename F>
int launch_update_serial_order(const F* data, int layout, size_t stride, const uint32_t* assignment,
                               F* means, int layout_means, size_t stride_means, uint32_t* cluster_sizes,
                               uint32_t dim, uint32_t k, uint32_t n, bool divide, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev);

/* f64.hip: the double-precision calls keep their own transposed centroids; the runtime grows the buffer under the
 * rules of the work space (not while a graph is recorded, after the stream has drained) and releases it on shutdown */
int reserve_f64(double** ptr, size_t* cap, size_t doubles);
int release_f64_workspace();
/* [dst, dst + bytes) is about to be written or released (bytes = 0: extent unknown): if the points announced by
 * kmx_prepare_points_f64 lie there, their float copy is forgotten */
void forget_prepared_points_f64(const void* dst, size_t bytes);

/* fused_small.hip: one pass over the points for a handful of centroids. a.assignment is a scratch vector of n entries
 * (only the entries of the points left to the exact pass are written); means_out and sizes are zero on entry and hold
 * sums and counts on return (the caller divides). */
bool fused_small_supports(uint32_t dim, uint32_t k, int layout, size_t stride, uint32_t n);
int launch_fused_small(const AssignArgs& a, float* means_out, uint32_t* sizes, kmx_exec_params* exec, Workspace* ws, const DeviceInfo& dev);

} // namespace kmx

#endif
