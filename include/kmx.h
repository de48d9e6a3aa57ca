/*
 * kmx -- C ABI of the MI355X (gfx950) Lloyd-iteration kernels.
 *
 * This is the device boundary of the k-means harness: the only thing the C++ host side (or any
 * other caller: ctypes, cgo, JNI ...) links against. It replaces the reference's kernel-runner
 * boundary, experimental/k-means/k-means/headers/kernels.cuh, whose entry points are the static
 * `KERNEL::run(const *ProblemInstance&, CudaExecParameters&)` policy functions and runFillZeros(),
 * plus the small part of bpplib's CudaBuffer/CUCH the reference's algorithm objects use
 * (experimental/k-means/k-means/headers/cuda.hpp:25-28,44-68,105-110).
 *
 * Conventions
 *   - Every function returns 0 on success or a non-zero kmx_status; kmx_last_error() then holds a
 *     message for the calling thread. Nothing throws across this boundary; the C++ host wrappers
 *     rethrow as std::runtime_error like the reference's runners (kernels.cu:281-282,666,675,701).
 *   - Device pointers are plain `void*`/`float*`/`uint32_t*` obtained from kmx_malloc (or from any
 *     other HIP allocation of the current device). Runners borrow them and never free them.
 *   - All work is enqueued on one stream (the legacy default stream unless kmx_set_stream() was
 *     called) and the calls return without waiting, except kmx_sync, kmx_d2h and
 *     kmx_event_elapsed_ms. Stream order is the only dependency mechanism, as in the reference
 *     (cuda.hpp:70-88: one cudaDeviceSynchronize after the iteration loop).
 *   - Not thread-safe: one host thread drives one device, as in the reference. The library keeps one work space, one
 *     stream and the properties of one device per process; kmx_set_device to another device is refused until
 *     kmx_shutdown() has released the work space.
 *   - layout: KMX_AOS element (idx, dim) = base[idx*stride + dim]; KMX_SOA = base[dim*stride + idx]
 *     (layout_policies.hpp:22-25,46-49); stride = LAYOUT::precomputeConstants(count, dim).
 */
#ifndef KMX_H
#define KMX_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum kmx_status {
	KMX_OK = 0,
	KMX_ERR_INVALID_ARGUMENT = 1, /* bad pointer / size / enum value                              */
	KMX_ERR_UNSUPPORTED = 2,      /* shape not supported by the requested variant                  */
	KMX_ERR_DEVICE = 3,           /* a HIP call failed; message carries hipGetErrorString          */
	KMX_ERR_NO_DEVICE = 4         /* no GPU visible (cuda.hpp:50-51 "No CUDA devices found!")      */
} kmx_status;

typedef enum kmx_layout { KMX_AOS = 0, KMX_SOA = 1 } kmx_layout;

/* = CudaExecParameters (kernels.cuh:55-70). In/out: runners overwrite block_count like the reference
 * (kernels.cu:203,311,750). Unlike the reference (kernels.cu:384,676,713) they never write the
 * other fields back, so one struct can serve the assignment and the update of every iteration.
 * Who reads what: block_size and items_per_thread shape the launches of KMX_ASSIGN_BASE and of the update variants
 * ATOMIC_POINT / _FINE / _WARP / _SHM2 / FAKE / FAKE_SHM (one lane per point or element, as in the reference);
 * shared_mem_bytes bounds the LDS of every variant that stages data there (0 = all of it); privatized_copies is read by
 * the update variants with global replicas. The tuned variants (KMX_ASSIGN_LDS_FMA / _MFMA / _MFMA_BF16X3 / _BEST,
 * KMX_UPDATE_ATOMIC_SHM, the fused kernels) fix their own work-group shape -- 8 wavefronts around the LDS-resident
 * centroids, 16 around a sorted chunk -- and ignore block_size, items_per_thread and regs_cache: the register tile the
 * reference exposes as regs_cache is the MFMA tile here. */
typedef struct kmx_exec_params {
	uint32_t block_size;        /* work-group size for the variants that honour it (default 256)   */
	uint32_t block_count;       /* out: number of work-groups of the main kernel last launched      */
	uint32_t shared_mem_bytes;  /* LDS budget per work-group; 0 = device maximum                    */
	uint32_t privatized_copies; /* global replicas of the k x d accumulator (update variants 0, 1)  */
	uint32_t items_per_thread;
	uint32_t regs_cache;
} kmx_exec_params;

/* Assignment variants (reference counterparts: kernels.cuh:81-93). */
typedef enum kmx_assign_variant {
	KMX_ASSIGN_BASE = 0,    /* BaseAssignmentKernel: one lane per point, the serial arithmetic op for op */
	KMX_ASSIGN_LDS_FMA = 1, /* CachedFixed/CachedRegs counterpart: centroids in LDS, register tile, fp32 FMA */
	KMX_ASSIGN_MFMA = 2,    /* dense-contraction path: fp32 MFMA tiles of -2 x.c + |c|^2                */
	KMX_ASSIGN_BEST = 3,    /* BestCachedAssignmentKernel: shape-based selector between the tuned variants */
	KMX_ASSIGN_MFMA_BF16X3 = 4 /* dense-contraction path at bf16 MFMA rate: operands split into hi + mid bf16 parts,
	                              three products per term, fp32 accumulation; same exact result (certify + recheck) */
} kmx_assign_variant;

/* Update variants (reference counterparts: kernels.cuh:96-105). */
typedef enum kmx_update_variant {
	KMX_UPDATE_ATOMIC_POINT = 0, /* UpdateAtomicPointKernel: one lane per point, global atomics      */
	KMX_UPDATE_ATOMIC_FINE = 1,  /* UpdateAtomicFineKernel: one lane per (point, dim) element        */
	KMX_UPDATE_ATOMIC_SHM = 2,   /* UpdateAtomicShmKernel: LDS-privatised partial sums, wave-aggregated flush */
	/* the remaining variants of the update micro-benchmark (bucketing-cuda/headers/kernels.cuh:44-63) */
	KMX_UPDATE_BASE = 3,         /* BaseKernel: no atomics, one lane per element of the result walks all points (sums in
	                                point order, i.e. with the bits of the serial loop); O(n k dim), for small inputs */
	KMX_UPDATE_ATOMIC_WARP = 4,  /* AtomicWarpKernel: one wavefront per point, lanes stride over the dimensions */
	KMX_UPDATE_ATOMIC_SHM2 = 5,  /* AtomicShm2Kernel (bucketing-cuda/kernels/kernels.cu:381-447): the whole k x dim block in LDS, in
	                                shared_mem_bytes / (k dim 4) private copies (lane t uses copy t mod copies), LDS atomics;
	                                KMX_ERR_UNSUPPORTED "Insufficient shared memory size ..." if not even one copy fits */
	/* kmx_bucket_sum_f32 only: probes of the raw cost of atomic additions, inputs ignored (kernels.cu:452-541). Element i adds
	 * 0.1 to dimension i mod dim of bucket (i / dim) mod k, so result[b][d] = 0.1 * #{points congruent to b modulo k} */
	KMX_UPDATE_FAKE = 6,         /* AtomicFakeKernel: global atomics (may be or-ed with KMX_UPDATE_EMULATED_ATOMICS) */
	KMX_UPDATE_FAKE_SHM = 7,     /* AtomicShmFakeKernel: the first shared_mem_bytes / (dim 4) buckets cached in LDS */
	/* no kernel of the reference: the sums of its SERIAL loop (serial.hpp:44-73) -- the members of a cluster added one after
	 * the other in ascending point number, then the guarded divide -- in O(n dim) work: stable counting sort of the point
	 * numbers by cluster, then one lane per (cluster, coordinate) walks its members in order. Same bits as
	 * SerialKMeansAlgorithm (and as KMX_UPDATE_BASE, which costs O(n k dim)), so a whole run with this update and any
	 * assignment variant equals the reference's serial run bit for bit. No precondition on the outputs. Floats and doubles.
	 * Time grows with the largest cluster (a chain of that many dependent additions). */
	KMX_UPDATE_SERIAL_ORDER = 8,
	/* flag, or-ed to ATOMIC_POINT / ATOMIC_FINE / ATOMIC_WARP / FAKE: additions as compare-and-swap loops instead of the hardware
	 * atomic (the micro-benchmark's --emul, AtomicEmulTrait, bucketing-cuda/kernels/kernels.cu:83-91) */
	KMX_UPDATE_EMULATED_ATOMICS = 0x100
} kmx_update_variant;

typedef struct kmx_props {
	char name[128];
	char arch[64];             /* gcnArchName, e.g. "gfx950:sramecc+:xnack-" */
	uint32_t compute_units;
	uint32_t wavefront_size;
	uint32_t max_threads_per_block;
	uint32_t lds_bytes_per_block;
	uint32_t clock_khz;
	uint64_t global_mem_bytes;
} kmx_props;

/* ---- device + memory (bpp::CudaDevice::count / cudaSetDevice / bpp::CudaBuffer; cuda.hpp:50-64,105-110;
 *      cudaGetDeviceProperties k-means.cpp:24-25) ---- */
int kmx_device_count(int* count);
int kmx_set_device(int device);
int kmx_device_props(kmx_props* props);
int kmx_malloc(void** dptr, size_t bytes);
int kmx_free(void* dptr);
int kmx_h2d(void* dst_device, const void* src_host, size_t bytes);          /* CudaBuffer::write; enqueued, host buffer must stay valid until kmx_sync */
int kmx_d2h(void* dst_host, const void* src_device, size_t bytes);          /* CudaBuffer::read; waits for the stream            */
int kmx_d2d(void* dst_device, const void* src_device, size_t bytes);        /* device copy on the stream                          */
int kmx_sync(void);                                                         /* cudaDeviceSynchronize (cuda.hpp:67,87)             */
int kmx_set_stream(void* hip_stream);                                       /* NULL = legacy default stream                       */
int kmx_shutdown(void);                                                     /* frees the library's internal work space            */

/* ---- runFillZeros<float|uint32_t> (kernels.cuh:74-75, kernels.cu:12-28): count 32-bit words := 0 ---- */
int kmx_fill_zero_u32(void* dptr, size_t count);

/*
 * ---- ASGN_KERNEL::run(AssignmentProblemInstance, CudaExecParameters&) (kernels.cuh:7-20,81-93) ----
 * assignment[i] = index of the centroid nearest to point i under the reference metric
 * sqrt(sum_d (x_d - c_d)^2) with the serial tie-break (lowest index on equal distances;
 * serial.hpp:21-35). Every variant returns exactly that index: the fast variants rank centroids
 * with |c|^2 - 2 x.c and re-evaluate with the serial arithmetic every point whose two best
 * candidates are closer than the rounding-error bound of that ranking.
 * last_assignment is accepted for signature parity and ignored (no reference kernel reads it).
 */
int kmx_assign_f32(int variant,
                   const float* data, int layout, size_t stride,
                   const float* means, int layout_means, size_t stride_means,
                   const uint32_t* last_assignment, uint32_t* assignment,
                   uint32_t dim, uint32_t k, uint32_t n, kmx_exec_params* exec);

/*
 * Sizes the library's work space (packed centroids, recheck queue, copied rows, partial sums, the values carried between
 * the sweeps of slices of centroids) for kmx_assign_f32 /
 * kmx_update_f32 / kmx_fused_f32 calls of this shape and these variants, so that those calls allocate nothing afterwards
 * (no counterpart in the reference, whose runners allocate nothing: cuda.hpp:54-64 allocates everything in initialize()).
 * Without it the first call of a shape grows the work space itself, which waits for the stream and calls hipMalloc; a
 * call with a different LDS budget (shared_mem_bytes) than the default may still grow it. Not while a graph is recorded.
 */
int kmx_reserve_f32(int assign_variant, int update_variant, int layout, int layout_means, uint32_t dim, uint32_t k, uint32_t n);

/* Number of points the last kmx_assign_f32 call re-evaluated with the serial arithmetic (waits for the stream). */
int kmx_assign_last_rechecked(uint64_t* count);

/* The concrete variant (never KMX_ASSIGN_BEST) the last kmx_assign_f32 call ran, -1 before the first call:
 * what the selector chose, for reports such as the reference's per-algorithm benchmark lines (k-means.cpp:155-169). */
int kmx_assign_last_variant(int* variant);

/*
 * ---- UPDATE_KERNEL::run(UpdateProblemInstance, CudaExecParameters&) (kernels.cuh:23-36,96-105) ----
 * Precondition as in the reference (cuda.hpp:78-79): means (k x dim, times privatized_copies for
 * variants 0 and 1) and cluster_sizes (k) are zero. Accumulates member sums and counts, merges
 * the privatised replicas and divides every non-empty cluster by its count; empty clusters stay
 * at zero (kernels.cu:149-163, serial.hpp:66-67).
 * KMX_UPDATE_ATOMIC_SHM has no precondition: it overwrites means (replica 0) and cluster_sizes, or
 * clears them itself where its kernel accumulates into them, so a driver may leave out the two
 * runFillZeros calls of cuda.hpp:78-79 (zeroing anyway is harmless).
 */
int kmx_update_f32(int variant,
                   const float* data, int layout, size_t stride,
                   const uint32_t* assignment,
                   float* means, int layout_means, size_t stride_means,
                   uint32_t* cluster_sizes,
                   uint32_t dim, uint32_t k, uint32_t n, kmx_exec_params* exec);

/*
 * kmx_update_f32 for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc). It has no counterpart in the reference, whose runners allocate nothing to begin
 * with. Same arguments, variants and results as kmx_update_f32; the difference is where the scratch memory of the tuned
 * variant (per-chunk partial sums and counts, chunks x k x (dim + 1) words) lives: in a static device array of
 * KMX_UPDATE_NOALLOC_SCRATCH_BYTES that every GPU the library runs on holds until the process ends, instead of the
 * work space that kmx_update_f32 grows with hipMalloc. The call allocates and frees nothing; a shape whose partial
 * sums do not fit is refused with KMX_ERR_UNSUPPORTED (the message names both sizes). SoA points skip the AoS copy
 * kmx_update_f32 makes of them and run the element-wise kernels (slower, same results). Per-kernel profiling
 * (kmx_set_profiling) does not cover this call. All calls on one GPU share that GPU's array: calls that overlap in
 * time on one GPU (different streams, different threads) race; calls on the library's one stream do not.
 * The address of a device's array is looked up once per device: by kmx_set_device, by kmx_reserve_f32, or else by the
 * first call of this function on the device, which is therefore refused (KMX_ERR_INVALID_ARGUMENT) between kmx_graph_begin
 * and kmx_graph_end -- make one of those calls before recording.
 */
#define KMX_UPDATE_NOALLOC_SCRATCH_BYTES (64u << 20)
int kmx_update_f32_noalloc(int variant,
                           const float* data, int layout, size_t stride,
                           const uint32_t* assignment,
                           float* means, int layout_means, size_t stride_means,
                           uint32_t* cluster_sizes,
                           uint32_t dim, uint32_t k, uint32_t n, kmx_exec_params* exec);

/*
 * ---- KERNEL::run(ProblemInstance, CudaExecParameters&) of the update micro-benchmark
 *      (experimental/bucketing-cuda/bucketing-cuda/headers/kernels.cuh:7-22,44-63; called once per batch by
 *      CudaBucketingAlgorithm::run, bucketing-cuda/headers/cuda.hpp:56-63) ----
 * result[b][d] = sum of data[i][d] over the vectors with indices[i] == b: the accumulation of kmx_update_f32 without
 * counts and without the divide, same variants (enum kmx_update_variant). Precondition as in the reference
 * (cuda.hpp:48): result (k x dim, times privatized_copies for ATOMIC_POINT / _FINE / _WARP) is zero. The sums of the replicas
 * are merged into replica 0.
 */
int kmx_bucket_sum_f32(int variant,
                       const float* data, int layout, size_t stride,
                       const uint32_t* indices,
                       float* result, int layout_result, size_t stride_result,
                       uint32_t dim, uint32_t k, uint32_t n, kmx_exec_params* exec);

/*
 * ---- FUSED_KERNEL::run(FusedProblemInstance, CudaExecParameters&) (kernels.cuh:38-53,107-116; called by
 *      CudaFusedKMeansAlgorithm::run, cuda.hpp:174-191) ----
 * One whole iteration without a caller-visible assignment vector: every point is assigned to its nearest centroid
 * of means_in (same result as kmx_assign_f32) and accumulated into means_out / cluster_sizes, which are then merged
 * and divided as by kmx_update_f32. Precondition as in the reference (cuda.hpp:178-179): means_out and cluster_sizes
 * are zero. The assignment lives in the library's work space (n words, grown on demand).
 */
typedef enum kmx_fused_variant {
	KMX_FUSED_TWO_PASS = 0, /* selector-chosen assignment sweep into the work space, then the tuned update (any shape; the
	                           points are read twice) */
	KMX_FUSED_ONE_PASS = 1, /* a single kernel reads every point once, assigns it and accumulates it (k <= 32, dim <= 32:
	                           the shapes bound by HBM; role of FusedCachedFixed / FusedCachedRegs) */
	KMX_FUSED_BEST = 2      /* ONE_PASS where it applies, else TWO_PASS */
} kmx_fused_variant;

int kmx_fused_f32(int variant,
                  const float* data, int layout, size_t stride,
                  const float* means_in, float* means_out, int layout_means, size_t stride_means,
                  uint32_t* cluster_sizes,
                  uint32_t dim, uint32_t k, uint32_t n, kmx_exec_params* exec);

/*
 * ---- one iteration of CudaKMeansAlgorithm::run's loop (cuda.hpp:72-85: assignment kernel, two zero-fills, update kernel) in
 *      one call, with the selector's assignment and the tuned update ----
 * assignment[i] = the nearest centroid of means_in (exactly as kmx_assign_f32), means_out / cluster_sizes = the centroids and
 * member counts of that assignment (as kmx_update_f32 with KMX_UPDATE_ATOMIC_SHM). No precondition on the outputs. What the
 * one call buys: where a single kernel can hold all centroids (k <= 32, dim <= 32 -- the shapes bound by HBM, where reading
 * the points twice is what an iteration costs) it reads every point ONCE, assigns it, accumulates it and writes its
 * assignment; everywhere else the call is the two calls it stands for. kmx_iteration_last_passes tells which of the two
 * ran (1 or 2 passes over the points; 0 before the first call).
 */
int kmx_iteration_f32(const float* data, int layout, size_t stride,
                      const float* means_in, float* means_out, int layout_means, size_t stride_means,
                      uint32_t* assignment, uint32_t* cluster_sizes,
                      uint32_t dim, uint32_t k, uint32_t n, kmx_exec_params* exec);
int kmx_iteration_last_passes(int* passes);

/*
 * ---- the same runners instantiated with F = double: the reference's --double switch (k-means.cpp:341-342) selects
 *      the <double> instantiations of every kernel (kernels.cu:1200-1261) ----
 * Arguments as for the _f32 entry points, with doubles for data and centroids (strides in elements).
 * kmx_assign_f64: every variant returns the serial result. KMX_ASSIGN_BASE evaluates the serial arithmetic for every pair;
 *   KMX_ASSIGN_LDS_FMA ranks with fp64 FMAs; KMX_ASSIGN_MFMA, _MFMA_BF16X3 and _BEST rank float copies of the inputs with the
 *   float sweeps (work space: n * dim + k * dim floats); all hand the points they cannot certify to the serial arithmetic
 *   on the doubles.
 * kmx_update_f64: ATOMIC_POINT / _FINE / _SHM; ATOMIC_SHM privatises the sums in LDS (whole when k * dim doubles fit 32 KB,
 *   in ranges of clusters of that size beyond), the others (and more than 256 ranges) use fp64 atomics in global memory. privatized_copies > 1: KMX_ERR_UNSUPPORTED.
 *   Precondition as for kmx_update_f32: means and cluster_sizes are zero (kmx_fill_zero_u32 with twice the count).
 * kmx_fused_f64: KMX_FUSED_TWO_PASS / KMX_FUSED_BEST (assignment into the work space, then the update);
 *   KMX_FUSED_ONE_PASS is float-only: KMX_ERR_UNSUPPORTED.
 * kmx_prepare_points_f64: the float copy of the points that the ranking sweeps of kmx_assign_f64 work on is made once, now,
 *   and kmx_assign_f64 / kmx_fused_f64 calls with the same pointer, layout, stride, dim and n reuse it instead of converting
 *   n * dim doubles per call -- the counterpart of the reference's upload in initialize() (cuda.hpp:54-64), after which the
 *   points never change. The caller promises exactly that: not to modify the points until kmx_forget_points_f64(), the next
 *   kmx_prepare_points_f64() or kmx_shutdown(). A call with other points makes the library forget by itself. Without
 *   this call every kmx_assign_f64 converts its points (correct for points that change between calls).
 */
int kmx_prepare_points_f64(const double* data, int layout, size_t stride, uint32_t dim, uint32_t n);
int kmx_forget_points_f64(void);
int kmx_assign_f64(int variant,
                   const double* data, int layout, size_t stride,
                   const double* means, int layout_means, size_t stride_means,
                   const uint32_t* last_assignment, uint32_t* assignment,
                   uint32_t dim, uint32_t k, uint32_t n, kmx_exec_params* exec);
int kmx_update_f64(int variant,
                   const double* data, int layout, size_t stride,
                   const uint32_t* assignment,
                   double* means, int layout_means, size_t stride_means,
                   uint32_t* cluster_sizes,
                   uint32_t dim, uint32_t k, uint32_t n, kmx_exec_params* exec);
/* kmx_bucket_sum_f32 on doubles (the micro-benchmark's --double): variants ATOMIC_POINT, ATOMIC_FINE, ATOMIC_SHM */
int kmx_bucket_sum_f64(int variant,
                       const double* data, int layout, size_t stride,
                       const uint32_t* indices,
                       double* result, int layout_result, size_t stride_result,
                       uint32_t dim, uint32_t k, uint32_t n, kmx_exec_params* exec);
int kmx_fused_f64(int variant,
                  const double* data, int layout, size_t stride,
                  const double* means_in, double* means_out, int layout_means, size_t stride_means,
                  uint32_t* cluster_sizes,
                  uint32_t dim, uint32_t k, uint32_t n, kmx_exec_params* exec);

/* ---- events on the library's stream (for the assignment / update split; the reference only has
 *      a wall-clock Stopwatch around run(), k-means.cpp:155-158) ---- */
int kmx_event_create(void** event);
int kmx_event_destroy(void* event);
int kmx_event_record(void* event);
int kmx_event_elapsed_ms(void* start, void* stop, float* ms); /* waits for `stop` */

/*
 * ---- recorded iterations (no counterpart in the reference, whose loop launches kernel by kernel,
 *      cuda.hpp:70-88) ----
 * Between kmx_graph_begin and kmx_graph_end the launching calls (kmx_assign_f32, kmx_update_f32, kmx_fused_f32,
 * kmx_bucket_sum_f32, kmx_fill_zero_u32) run nothing: their kernels, with the arguments of that moment, are recorded into
 * a HIP graph. kmx_graph_launch enqueues the whole recording on the library's stream as one unit, any number of times
 * (the host driver records two ping-pong iterations once and replays them). Everything that allocates, copies or
 * waits is refused while recording; a call whose work space would have to grow is refused too -- make the same
 * calls once before recording. Per-kernel profiling events are not recorded.
 */
int kmx_graph_begin(void);
int kmx_graph_end(void** graph);
int kmx_graph_launch(void* graph);
int kmx_graph_destroy(void* graph);

/*
 * Per-kernel timing for roofline reports (no counterpart in the reference). While enabled, every
 * kmx_assign_f32 / kmx_update_f32 call brackets its dominant kernel (the sweep over the centroids /
 * the accumulation pass; not the small pack, recheck, merge and divide kernels around it) with a pair of
 * events on the library's stream. kmx_last_kernel_ms(which, ...) waits for that kernel of the most
 * recent call and returns its duration; which: 0 = assignment, 1 = update.
 */
int kmx_set_profiling(int enabled);
int kmx_last_kernel_ms(int which, float* ms);

/*
 * Work-space bound (no counterpart in the reference: its kernels evaluate every point directly). With SoA points the
 * exact pass of the tuned assignment variants copies the rows of the points it has to re-evaluate into a compact
 * block in the library's work space; `bytes` bounds that block (default 1 GiB, at least 1024 rows are always kept).
 * Points beyond the bound are still re-evaluated, reading the SoA data directly (slower, same results).
 */
int kmx_set_queued_rows_limit(size_t bytes);

/*
 * The split-bf16 sweep of rows of 17 to 32 dimensions may run in two levels (no counterpart in the reference): one product
 * per dimension (hi * hi) for all points, a third of the matrix work, with a certificate wide enough for it; then the three
 * products for the points that level could not settle; then the exact pass as always. The results are the same at every
 * setting. mode 0: one level always; 1 (default): two levels where they pay (resident centroids, 97 centroids or more,
 * 2^18 points or more); 2: two levels wherever the kernels allow it (for tests and measurements on small inputs).
 */
int kmx_set_two_level_sweep(int mode);

/*
 * The certification bound of the ranking sweeps, evaluated on the host by the very function the kernels use (no
 * counterpart in the reference, whose kernels evaluate every pair directly; no device needed). A sweep decides a point
 * without the serial arithmetic only if its two smallest ranking values differ by more than tau; the tests check tau
 * against an emulation of the split operands on adversarial inputs.
 *   form 0: fp32 MFMA sweep (KMX_ASSIGN_MFMA)                      tau = kd (x2 + c2max); xpart2, cmid2max, crest2max ignored
 *   form 3: sweeps on the vector ALU (KMX_ASSIGN_LDS_FMA): the same with a smaller kd
 *   forms 5, 6: the single-pass iteration kernels (narrow rows: the chain of form 3; rows of 8, 16, 32 floats: the matrix
 *           instruction of form 0), whose ranking values carry the centroid's number in their lowest bits: xpart2 = the
 *           number of replaced bits, 4 (up to 16 centroids) or 5
 *   form 1: split-bf16 sweep, three products per dimension         xpart2 = sum_i xmid_i^2
 *   form 2: split-bf16 sweep, packed rows (dim <= 4, four products) xpart2 = sum_i xrest_i^2
 *   form 4: first level of the two-level split-bf16 sweep (one product per dimension, hi * hi) xpart2 = sum_i (x_i - xhi_i)^2
 * x2 = |x|^2, c2max = max_j |c_j|^2, cmid2max / crest2max = max_j of the squared norms of the mid / rest parts of -2 c_j;
 * all of them in the frame the sweep works in: the float sweeps subtract a vector m from points and centroids (the mean
 * of the first 16 centroids; for packed rows, with 128 centroids or more, of the first 256; the single-pass fused kernel
 * only when they lie far from the origin; the double-precision path hands them float copies of data it has moved itself, in double), so the norms are those of the moved data; forms 0, 1 and 3 then add
 * 8 * 2^-23 * (x2 + c2max) for the two roundings, which this function leaves out (form 2 contains it).
 */
int kmx_certificate_tau(int form, uint32_t dim, float x2, float xpart2, float c2max, float cmid2max, float crest2max, float* tau);

/*
 * The screening threshold that a sweep in the moved frame hands to the kernels of the exact pass that evaluate
 * |c_j|^2 - 2 c_j . x in the frame of the data (same purpose and conventions as kmx_certificate_tau: the kernels' own
 * function, on the host). first, tau, x2 = |x - m|^2 and c2max = max_j |c_j - m|^2 are values of the moved frame,
 * along = (x - m) . m, m2 = |m|^2, mnorm >= |m|. A centroid whose value exceeds the threshold cannot be the serial result.
 */
int kmx_certificate_unmoved_threshold(uint32_t dim, float first, float tau, float x2, float along, float c2max, float m2, float mnorm,
                                      float* threshold);

/*
 * What the matrix cores do with a chain of accumulations (no counterpart in the reference; a diagnostic the tests use to
 * hold the hardware to the assumption the certificates make about it: at most one 2^-23 of the running magnitude per
 * accumulated product, however the instruction rounds or truncates inside). One wavefront computes
 *      d[i][j] = c[i][j] + sum_q a[i][q] b[j][q],   i, j < 32,  q < depth,
 * block by block in ascending q, one instruction per block, with the instructions, operand layout and order of the
 * sweeps: kind 0 = v_mfma_f32_32x32x2_f32 (depth = 2 blocks), kind 1 = v_mfma_f32_32x32x16_bf16 (depth = 16 blocks; the
 * values of a and b must be exactly representable in bf16, the low 16 bits of their words are dropped), kind 2 =
 * v_mfma_f32_16x16x4_f32 (depth = 4 blocks; the 32 x 32 result as four tiles of 16 x 16).
 * a: 32 x depth row-major; b: 32 x depth, the depth values of column j contiguous; c, d: 32 x 32 row-major. Device pointers.
 */
int kmx_probe_matrix_chain(int kind, const float* a, const float* b, const float* c, float* d, uint32_t blocks);

/* Message of the last failed call on this thread ("" if none). */
const char* kmx_last_error(void);

#ifdef __cplusplus
}
#endif

#endif
