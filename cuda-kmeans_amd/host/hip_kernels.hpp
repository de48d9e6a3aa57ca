/*
 * Kernel-runner boundary of the harness, host side: the same policy classes the reference declares in
 * experimental/k-means/k-means/headers/kernels.cuh (problem-instance structs :7-52, CudaExecParameters
 * :55-70, runFillZeros :74-75, DECLARE_ASSIGNMENT_KERNEL :81-93, DECLARE_UPDATE_KERNEL :96-105), each
 * with one static run(instance, exec). Here run() forwards to the C ABI of libkmx_hip.so
 * (include/kmx.h); no HIP header is needed on this side. Failures come back as error codes and are
 * rethrown as std::runtime_error, which is how the reference's runners report unsupported shapes
 * (kernels.cu:281-282,666,675,701) and how CUCH() reports device errors.
 *
 * F = float and F = double (the reference's --double) are built; the single-pass fused kernel is float-only and
 * reports that as an error for doubles.
 */
#ifndef KMX_HOST_HIP_KERNELS_HPP
#define KMX_HOST_HIP_KERNELS_HPP

#include "kmx.h"
#include "layouts.hpp"

#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>
#include <type_traits>

/* throws with the library's message when a kmx call fails */
inline void KMX_CHECK(int rc)
{
	if (rc != KMX_OK) throw std::runtime_error(std::string(kmx_last_error()));
}

template<typename F, typename IDX_T>
struct AssignmentProblemInstance {
	const F* data;
	const F* means;
	const IDX_T* lastAssignment;
	IDX_T* assignment; /* the result */
	IDX_T dim, k, n;

	AssignmentProblemInstance(const F* _data, const F* _means, const IDX_T* _lastAssignment, IDX_T* _assignment,
		std::size_t _dim, std::size_t _k, std::size_t _n)
		: data(_data), means(_means), lastAssignment(_lastAssignment), assignment(_assignment),
		dim((IDX_T)_dim), k((IDX_T)_k), n((IDX_T)_n) {}
};

template<typename F, typename IDX_T>
struct UpdateProblemInstance {
	const F* data;
	const IDX_T* assignment;
	F* means; /* the result; zeroed by the caller */
	IDX_T* clusterSizes; /* zeroed by the caller */
	IDX_T dim, k, n;

	UpdateProblemInstance(const F* _data, const IDX_T* _assignment, F* _means, IDX_T* _clusterSizes,
		std::size_t _dim, std::size_t _k, std::size_t _n)
		: data(_data), assignment(_assignment), means(_means), clusterSizes(_clusterSizes),
		dim((IDX_T)_dim), k((IDX_T)_k), n((IDX_T)_n) {}
};

/* = FusedProblemInstance (kernels.cuh:38-53) */
template<typename F, typename IDX_T>
struct FusedProblemInstance {
	const F* data;
	const F* meansIn;
	F* meansOut; /* the result; zeroed by the caller */
	IDX_T* clusterSizes; /* zeroed by the caller */
	IDX_T dim, k, n;

	FusedProblemInstance(const F* _data, const F* _meansIn, F* _meansOut, IDX_T* _clusterSizes,
		std::size_t _dim, std::size_t _k, std::size_t _n)
		: data(_data), meansIn(_meansIn), meansOut(_meansOut), clusterSizes(_clusterSizes),
		dim((IDX_T)_dim), k((IDX_T)_k), n((IDX_T)_n) {}
};

/* = CudaExecParameters; the field order is that of kmx_exec_params */
struct HipExecParameters {
	unsigned int blockSize;
	unsigned int blockCount;
	unsigned int sharedMemorySize;
	std::uint32_t privatizedCopies;
	std::uint32_t itemsPerThread;
	std::uint32_t regsCache;

	HipExecParameters(unsigned int _blockSize = 256, unsigned int _blockCount = 0, unsigned int _sharedMemorySize = 0,
		std::uint32_t _privatizedCopies = 1, std::uint32_t _itemsPerThread = 1, std::uint32_t _regsCache = 1)
		: blockSize(_blockSize), blockCount(_blockCount), sharedMemorySize(_sharedMemorySize),
		privatizedCopies(_privatizedCopies), itemsPerThread(_itemsPerThread), regsCache(_regsCache) {}
};
using CudaExecParameters = HipExecParameters; /* the reference's name */

static_assert(sizeof(HipExecParameters) == sizeof(kmx_exec_params), "HipExecParameters must mirror kmx_exec_params");

/* runFillZeros<F>(data, n): n 32-bit elements := 0 on the stream */
template<typename T>
void runFillZeros(T* data, std::size_t n)
{
	static_assert(sizeof(T) % 4 == 0, "element types are made of 32-bit words");
	KMX_CHECK(kmx_fill_zero_u32(data, n * (sizeof(T) / 4)));
}

namespace hip_detail {

/* the C ABI has one entry point per element type */
inline int assign_call(int variant, const float* data, int ld, std::size_t stride, const float* means, int lm, std::size_t strideMeans,
	const std::uint32_t* last, std::uint32_t* assignment, std::uint32_t dim, std::uint32_t k, std::uint32_t n, kmx_exec_params* exec)
{ return kmx_assign_f32(variant, data, ld, stride, means, lm, strideMeans, last, assignment, dim, k, n, exec); }
inline int assign_call(int variant, const double* data, int ld, std::size_t stride, const double* means, int lm, std::size_t strideMeans,
	const std::uint32_t* last, std::uint32_t* assignment, std::uint32_t dim, std::uint32_t k, std::uint32_t n, kmx_exec_params* exec)
{ return kmx_assign_f64(variant, data, ld, stride, means, lm, strideMeans, last, assignment, dim, k, n, exec); }

inline int update_call(int variant, const float* data, int ld, std::size_t stride, const std::uint32_t* assignment, float* means, int lm,
	std::size_t strideMeans, std::uint32_t* sizes, std::uint32_t dim, std::uint32_t k, std::uint32_t n, kmx_exec_params* exec)
{ return kmx_update_f32(variant, data, ld, stride, assignment, means, lm, strideMeans, sizes, dim, k, n, exec); }
inline int update_call(int variant, const double* data, int ld, std::size_t stride, const std::uint32_t* assignment, double* means, int lm,
	std::size_t strideMeans, std::uint32_t* sizes, std::uint32_t dim, std::uint32_t k, std::uint32_t n, kmx_exec_params* exec)
{ return kmx_update_f64(variant, data, ld, stride, assignment, means, lm, strideMeans, sizes, dim, k, n, exec); }

inline int fused_call(int variant, const float* data, int ld, std::size_t stride, const float* meansIn, float* meansOut, int lm,
	std::size_t strideMeans, std::uint32_t* sizes, std::uint32_t dim, std::uint32_t k, std::uint32_t n, kmx_exec_params* exec)
{ return kmx_fused_f32(variant, data, ld, stride, meansIn, meansOut, lm, strideMeans, sizes, dim, k, n, exec); }
inline int fused_call(int variant, const double* data, int ld, std::size_t stride, const double* meansIn, double* meansOut, int lm,
	std::size_t strideMeans, std::uint32_t* sizes, std::uint32_t dim, std::uint32_t k, std::uint32_t n, kmx_exec_params* exec)
{ return kmx_fused_f64(variant, data, ld, stride, meansIn, meansOut, lm, strideMeans, sizes, dim, k, n, exec); }

/* kmx_iteration_f32: the default pair of kernels in one call (floats); see HipKMeansAlgorithm */
inline int iteration_call(const float* data, int ld, std::size_t stride, const float* meansIn, float* meansOut, int lm, std::size_t strideMeans,
	std::uint32_t* assignment, std::uint32_t* sizes, std::uint32_t dim, std::uint32_t k, std::uint32_t n, kmx_exec_params* exec)
{ return kmx_iteration_f32(data, ld, stride, meansIn, meansOut, lm, strideMeans, assignment, sizes, dim, k, n, exec); }
inline int iteration_call(const double*, int, std::size_t, const double*, double*, int, std::size_t, std::uint32_t*, std::uint32_t*,
	std::uint32_t, std::uint32_t, std::uint32_t, kmx_exec_params*)
{ return KMX_ERR_UNSUPPORTED; } /* never reached: the driver takes the one call for floats only */

/* The points of a run are uploaded once and never change (cuda.hpp:54-64): the double-precision entry points are told so and
 * keep the float copy their ranking sweeps work on, instead of converting the points in every call. Floats need nothing. */
inline int prepare_points_call(const float*, int, std::size_t, std::uint32_t, std::uint32_t) { return KMX_OK; }
inline int prepare_points_call(const double* data, int ld, std::size_t stride, std::uint32_t dim, std::uint32_t n)
{ return kmx_prepare_points_f64(data, ld, stride, dim, n); }
inline int forget_points_call(const float*) { return KMX_OK; }
inline int forget_points_call(const double*) { return kmx_forget_points_f64(); }

template<typename F, class LAYOUT>
void preparePoints(const F* data, std::size_t n, std::size_t dim)
{
	KMX_CHECK(prepare_points_call(data, LAYOUT::ID, LAYOUT::precomputeConstants(n, dim), (std::uint32_t)dim, (std::uint32_t)n));
}

template<typename F>
void forgetPoints(const F* data)
{
	KMX_CHECK(forget_points_call(data));
}

template<typename F, typename IDX_T, class LAYOUT, class LAYOUT_MEANS>
void assign(int variant, const AssignmentProblemInstance<F, IDX_T>& in, HipExecParameters& exec)
{
	static_assert(sizeof(IDX_T) == 4, "built for 32-bit indices");
	KMX_CHECK(assign_call(variant,
		in.data, LAYOUT::ID, LAYOUT::precomputeConstants(in.n, in.dim),
		in.means, LAYOUT_MEANS::ID, LAYOUT_MEANS::precomputeConstants(in.k, in.dim),
		(const std::uint32_t*)in.lastAssignment, (std::uint32_t*)in.assignment,
		in.dim, in.k, in.n, reinterpret_cast<kmx_exec_params*>(&exec)));
}

template<typename F, typename IDX_T, class LAYOUT, class LAYOUT_MEANS>
void update(int variant, const UpdateProblemInstance<F, IDX_T>& in, HipExecParameters& exec)
{
	static_assert(sizeof(IDX_T) == 4, "built for 32-bit indices");
	KMX_CHECK(update_call(variant,
		in.data, LAYOUT::ID, LAYOUT::precomputeConstants(in.n, in.dim),
		(const std::uint32_t*)in.assignment,
		in.means, LAYOUT_MEANS::ID, LAYOUT_MEANS::precomputeConstants(in.k, in.dim),
		(std::uint32_t*)in.clusterSizes, in.dim, in.k, in.n, reinterpret_cast<kmx_exec_params*>(&exec)));
}

template<typename F, typename IDX_T, class LAYOUT, class LAYOUT_MEANS>
void fused(int variant, const FusedProblemInstance<F, IDX_T>& in, HipExecParameters& exec)
{
	static_assert(sizeof(IDX_T) == 4, "built for 32-bit indices");
	KMX_CHECK(fused_call(variant,
		in.data, LAYOUT::ID, LAYOUT::precomputeConstants(in.n, in.dim),
		in.meansIn, in.meansOut, LAYOUT_MEANS::ID, LAYOUT_MEANS::precomputeConstants(in.k, in.dim),
		(std::uint32_t*)in.clusterSizes, in.dim, in.k, in.n, reinterpret_cast<kmx_exec_params*>(&exec)));
}

/* assignment + update of one iteration in one call (kmx_iteration_f32) */
template<typename F, typename IDX_T, class LAYOUT, class LAYOUT_MEANS>
void iteration(const F* data, const F* meansIn, F* meansOut, IDX_T* assignment, IDX_T* sizes, std::size_t dim, std::size_t k, std::size_t n,
	HipExecParameters& exec)
{
	static_assert(sizeof(IDX_T) == 4, "built for 32-bit indices");
	KMX_CHECK(iteration_call(data, LAYOUT::ID, LAYOUT::precomputeConstants(n, dim), meansIn, meansOut, LAYOUT_MEANS::ID,
		LAYOUT_MEANS::precomputeConstants(k, dim), (std::uint32_t*)assignment, (std::uint32_t*)sizes,
		(std::uint32_t)dim, (std::uint32_t)k, (std::uint32_t)n, reinterpret_cast<kmx_exec_params*>(&exec)));
}

} // namespace hip_detail

#define KMX_DEFINE_ASSIGNMENT_KERNEL(NAME, VARIANT)\
template<typename F, typename IDX_T, class LAYOUT, class LAYOUT_MEANS, class METRIC>\
class NAME {\
public:\
	static void run(const AssignmentProblemInstance<F, IDX_T>& in, HipExecParameters& exec)\
	{ hip_detail::assign<F, IDX_T, LAYOUT, LAYOUT_MEANS>(VARIANT, in, exec); }\
};

KMX_DEFINE_ASSIGNMENT_KERNEL(BaseAssignmentKernel, KMX_ASSIGN_BASE)       /* kernels.cu:180-207 */
KMX_DEFINE_ASSIGNMENT_KERNEL(LdsFmaAssignmentKernel, KMX_ASSIGN_LDS_FMA)  /* role of CachedFixed / CachedRegs, kernels.cu:216-319,546-703 */
KMX_DEFINE_ASSIGNMENT_KERNEL(MfmaAssignmentKernel, KMX_ASSIGN_MFMA)       /* no counterpart: matrix-core path */
KMX_DEFINE_ASSIGNMENT_KERNEL(MfmaBf16AssignmentKernel, KMX_ASSIGN_MFMA_BF16X3) /* no counterpart: matrix-core path on split bf16 operands */
KMX_DEFINE_ASSIGNMENT_KERNEL(BestCachedAssignmentKernel, KMX_ASSIGN_BEST) /* kernels.cu:706-717 */

/* role of FusedCachedFixedKernel / FusedCachedRegsKernel (kernels.cu:883-1190): one call per iteration, no assignment buffer */
#define KMX_DEFINE_FUSED_KERNEL(NAME, VARIANT)\
template<typename F, typename IDX_T, class LAYOUT, class LAYOUT_MEANS, class METRIC>\
class NAME {\
public:\
	static void run(const FusedProblemInstance<F, IDX_T>& in, HipExecParameters& exec)\
	{ hip_detail::fused<F, IDX_T, LAYOUT, LAYOUT_MEANS>(VARIANT, in, exec); }\
};

KMX_DEFINE_FUSED_KERNEL(FusedTwoPassKernel, KMX_FUSED_TWO_PASS) /* assignment sweep + update behind one call, any shape */
KMX_DEFINE_FUSED_KERNEL(FusedOnePassKernel, KMX_FUSED_ONE_PASS) /* one kernel, a handful of centroids */
KMX_DEFINE_FUSED_KERNEL(FusedBestKernel, KMX_FUSED_BEST)        /* one pass where it applies */

/* EMUL (the reference's template argument, kernels.cuh:96-105): additions as compare-and-swap loops; built for the float
 * point and fine kernels (KMX_UPDATE_EMULATED_ATOMICS), ignored by the LDS kernels, which have no global fp32 atomics to emulate */
#define KMX_DEFINE_UPDATE_KERNEL(NAME, VARIANT, CAN_EMULATE, SELF_CLEARING)\
template<typename F, typename IDX_T, class LAYOUT, class LAYOUT_MEANS, int EMUL = false>\
class NAME {\
public:\
	/* false: the runner clears or overwrites its outputs itself, the driver may leave out the two runFillZeros calls */\
	static constexpr bool needsZeroedOutput = !(SELF_CLEARING == 2 || (SELF_CLEARING == 1 && std::is_same<F, float>::value));\
	static void run(const UpdateProblemInstance<F, IDX_T>& in, HipExecParameters& exec)\
	{\
		static_assert(!(EMUL && CAN_EMULATE) || std::is_same<F, float>::value, "emulated atomics are built for floats");\
		hip_detail::update<F, IDX_T, LAYOUT, LAYOUT_MEANS>((EMUL && CAN_EMULATE) ? (VARIANT | KMX_UPDATE_EMULATED_ATOMICS) : VARIANT, in, exec);\
	}\
};

/* SELF_CLEARING: 0 = the outputs must be zero on entry, 1 = not for floats, 2 = for neither element type */
KMX_DEFINE_UPDATE_KERNEL(UpdateAtomicPointKernel, KMX_UPDATE_ATOMIC_POINT, true, 0) /* kernels.cu:726-761 */
KMX_DEFINE_UPDATE_KERNEL(UpdateAtomicFineKernel, KMX_UPDATE_ATOMIC_FINE, true, 0)   /* kernels.cu:770-809 */
KMX_DEFINE_UPDATE_KERNEL(UpdateAtomicShmKernel, KMX_UPDATE_ATOMIC_SHM, false, 1)    /* kernels.cu:817-878 */
/* no kernel of the reference: the sums of SerialKMeansAlgorithm::updateMeans (serial.hpp:44-73) in its order, on the device */
KMX_DEFINE_UPDATE_KERNEL(UpdateSerialOrderKernel, KMX_UPDATE_SERIAL_ORDER, false, 2)

#endif
