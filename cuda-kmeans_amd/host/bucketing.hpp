/*
 * The update micro-benchmark ("bucketing"): sum vectors into k buckets selected by an index array, one independent
 * batch per iteration. Host-side counterpart of experimental/bucketing-cuda/bucketing-cuda/headers/
 * {interface.hpp, serial.hpp, cuda.hpp, kernels.cuh} of the reference: same algorithm interface, same serial
 * semantics (sums in vector order, fp32), the device kernels reached through kmx_bucket_sum_f32.
 */
#ifndef KMX_HOST_BUCKETING_HPP
#define KMX_HOST_BUCKETING_HPP

#include "hip_kernels.hpp"
#include "hip_kmeans.hpp"
#include "layouts.hpp"

#include <cstdint>
#include <vector>

/* = IBucketingAlgorithm (bucketing-cuda/headers/interface.hpp:8-41) */
template<typename F = float>
class IBucketingAlgorithm
{
protected:
	std::size_t mDim = 0, mK = 0, mN = 0, mIter = 1;
	std::vector<F> mResult;

public:
	virtual ~IBucketingAlgorithm() {}

	virtual void initialize(std::size_t dim, std::size_t k, std::size_t n, std::size_t iter,
		const std::vector<F>& /*data*/, const std::vector<std::uint32_t>& /*indices*/)
	{
		mDim = dim; mK = k; mN = n; mIter = iter;
	}

	virtual void run() = 0;

	/* iter x k x dim sums, unpadded AoS, whatever the working layout was */
	virtual const std::vector<F>& getResult() { return mResult; }

	virtual void cleanup() { mResult.clear(); }
};

namespace bucketing_detail {

/* working layout (possibly padded) -> dense [iter][k][dim] */
template<typename F, class LAYOUT>
void compact(std::vector<F>& out, const F* res, std::size_t iters, std::size_t k, std::size_t dim)
{
	const std::size_t stride = LAYOUT::precomputeConstants(k, dim), block = LAYOUT::size(k, dim);
	out.clear();
	out.reserve(iters * k * dim);
	for (std::size_t it = 0; it < iters; ++it)
		for (std::size_t b = 0; b < k; ++b)
			for (std::size_t d = 0; d < dim; ++d)
				out.push_back(LAYOUT::at(res + it * block, b, d, stride));
}

}

/* = SerialBucketingAlgorithm (bucketing-cuda/headers/serial.hpp:11-81): vectors in order, one add per coordinate */
template<typename F = float, class LAYOUT = AoSLayoutPolicy<>>
class SerialBucketingAlgorithm : public IBucketingAlgorithm<F>
{
	const F* mData = nullptr;
	const std::uint32_t* mIndices = nullptr;
	std::vector<F> mWork;
	bool mResultReady = false;

public:
	void initialize(std::size_t dim, std::size_t k, std::size_t n, std::size_t iter,
		const std::vector<F>& data, const std::vector<std::uint32_t>& indices) override
	{
		IBucketingAlgorithm<F>::initialize(dim, k, n, iter, data, indices);
		mData = data.data();
		mIndices = indices.data();
		mWork.assign(LAYOUT::size(k, dim) * iter, (F)0);
		mResultReady = false;
	}

	void run() override
	{
		const std::size_t strideData = LAYOUT::precomputeConstants(this->mN, this->mDim);
		const std::size_t strideRes = LAYOUT::precomputeConstants(this->mK, this->mDim);
		const std::size_t batchData = LAYOUT::size(this->mN, this->mDim), batchRes = LAYOUT::size(this->mK, this->mDim);
		for (std::size_t it = 0; it < this->mIter; ++it) {
			const F* data = mData + it * batchData;
			const std::uint32_t* indices = mIndices + it * this->mN;
			F* res = mWork.data() + it * batchRes;
			for (std::size_t i = 0; i < this->mN; ++i) {
				const std::uint32_t target = indices[i];
				for (std::size_t d = 0; d < this->mDim; ++d)
					LAYOUT::at(res, target, d, strideRes) += LAYOUT::at(data, i, d, strideData);
			}
		}
	}

	const std::vector<F>& getResult() override
	{
		if (!mResultReady) {
			bucketing_detail::compact<F, LAYOUT>(this->mResult, mWork.data(), this->mIter, this->mK, this->mDim);
			mResultReady = true;
		}
		return this->mResult;
	}
};

/* = ProblemInstance (bucketing-cuda/headers/kernels.cuh:7-22) */
template<typename F>
struct BucketingProblemInstance {
	const F* data;
	const std::uint32_t* indices;
	F* result;
	std::uint32_t dim, k, n;

	BucketingProblemInstance(const F* _data, const std::uint32_t* _indices, F* _result, std::size_t _dim, std::size_t _k, std::size_t _n)
		: data(_data), indices(_indices), result(_result), dim((std::uint32_t)_dim), k((std::uint32_t)_k), n((std::uint32_t)_n) {}
};

/* the C ABI has one entry point per element type (doubles: the atomic point, fine and shm kernels) */
inline int bucket_sum_call(int variant, const float* data, int layout, std::size_t stride, const std::uint32_t* indices, float* result,
	int layoutResult, std::size_t strideResult, std::uint32_t dim, std::uint32_t k, std::uint32_t n, kmx_exec_params* exec)
{ return kmx_bucket_sum_f32(variant, data, layout, stride, indices, result, layoutResult, strideResult, dim, k, n, exec); }
inline int bucket_sum_call(int variant, const double* data, int layout, std::size_t stride, const std::uint32_t* indices, double* result,
	int layoutResult, std::size_t strideResult, std::uint32_t dim, std::uint32_t k, std::uint32_t n, kmx_exec_params* exec)
{ return kmx_bucket_sum_f64(variant, data, layout, stride, indices, result, layoutResult, strideResult, dim, k, n, exec); }

/* kernel policy classes of the micro-benchmark (bucketing-cuda/headers/kernels.cuh:44-63): one static run() each */
#define KMX_DEFINE_BUCKETING_KERNEL(NAME, VARIANT, CAN_EMULATE)\
template<typename F, class LAYOUT, int EMUL = false>\
class NAME {\
public:\
	static void run(const BucketingProblemInstance<F>& in, HipExecParameters& exec)\
	{\
		/* EMUL: additions as compare-and-swap loops; kernels without global fp32 atomics ignore it, as in the reference */\
		KMX_CHECK(bucket_sum_call((EMUL && CAN_EMULATE) ? (VARIANT | KMX_UPDATE_EMULATED_ATOMICS) : VARIANT,\
			in.data, LAYOUT::ID, LAYOUT::precomputeConstants(in.n, in.dim), in.indices,\
			in.result, LAYOUT::ID, LAYOUT::precomputeConstants(in.k, in.dim),\
			in.dim, in.k, in.n, reinterpret_cast<kmx_exec_params*>(&exec)));\
	}\
};

KMX_DEFINE_BUCKETING_KERNEL(BaseKernel, KMX_UPDATE_BASE, false)                /* bucketing-cuda/kernels/kernels.cu:163-188 base */
KMX_DEFINE_BUCKETING_KERNEL(AtomicPointKernel, KMX_UPDATE_ATOMIC_POINT, true)  /* :195-226 atomic_point */
KMX_DEFINE_BUCKETING_KERNEL(AtomicWarpKernel, KMX_UPDATE_ATOMIC_WARP, true)    /* :234-266 atomic_warp, with 64-lane wavefronts */
KMX_DEFINE_BUCKETING_KERNEL(AtomicFineKernel, KMX_UPDATE_ATOMIC_FINE, true)    /* :275-307 atomic_fine */
KMX_DEFINE_BUCKETING_KERNEL(AtomicShmKernel, KMX_UPDATE_ATOMIC_SHM, false)     /* :317-372 atomic_shm: here the tuned LDS kernels */
KMX_DEFINE_BUCKETING_KERNEL(AtomicShm2Kernel, KMX_UPDATE_ATOMIC_SHM2, false)   /* :381-447 atomic_shm2: the whole block in LDS, sharedMemorySize / (k dim sizeof F) private copies */
KMX_DEFINE_BUCKETING_KERNEL(AtomicFakeKernel, KMX_UPDATE_FAKE, true)           /* :452-486 fake: constant 0.1 added atomically to bucket (i / dim) % k */
KMX_DEFINE_BUCKETING_KERNEL(AtomicShmFakeKernel, KMX_UPDATE_FAKE_SHM, false)   /* :495-550 fake_shm: the same with the first buckets cached in LDS */

/* = CudaBucketingAlgorithm (bucketing-cuda/headers/cuda.hpp:13-86): one buffer set per batch, one kernel call per batch */
template<typename F = float, class LAYOUT = AoSLayoutPolicy<>, class KERNEL = AtomicShmKernel<F, LAYOUT>>
class HipBucketingAlgorithm : public IBucketingAlgorithm<F>
{
	HipExecParameters mExecParams;
	std::vector<HipBuffer<F>> mDevData;
	std::vector<HipBuffer<std::uint32_t>> mDevIndices;
	std::vector<HipBuffer<F>> mDevResult;

public:
	explicit HipBucketingAlgorithm(const HipExecParameters& exec) : mExecParams(exec) {}

	void initialize(std::size_t dim, std::size_t k, std::size_t n, std::size_t iter,
		const std::vector<F>& data, const std::vector<std::uint32_t>& indices) override
	{
		IBucketingAlgorithm<F>::initialize(dim, k, n, iter, data, indices);
		this->mResult.clear();
		requireDevice();
		const std::size_t copies = mExecParams.privatizedCopies ? mExecParams.privatizedCopies : 1;
		const std::size_t dataSize = LAYOUT::size(n, dim), resSize = LAYOUT::size(k, dim);
		mDevData = std::vector<HipBuffer<F>>(iter);
		mDevIndices = std::vector<HipBuffer<std::uint32_t>>(iter);
		mDevResult = std::vector<HipBuffer<F>>(iter);
		for (std::size_t i = 0; i < iter; ++i) {
			mDevData[i].realloc(dataSize);
			mDevIndices[i].realloc(n);
			mDevResult[i].realloc(resSize * copies);
			KMX_CHECK(kmx_h2d(*mDevData[i], data.data() + i * dataSize, dataSize * sizeof(F)));
			KMX_CHECK(kmx_h2d(*mDevIndices[i], indices.data() + i * n, n * sizeof(std::uint32_t)));
			runFillZeros<F>(*mDevResult[i], resSize * copies);
		}
		KMX_CHECK(kmx_sync());
	}

	void run() override
	{
		for (std::size_t it = 0; it < this->mIter; ++it) {
			BucketingProblemInstance<F> instance(*mDevData[it], *mDevIndices[it], *mDevResult[it], this->mDim, this->mK, this->mN);
			KERNEL::run(instance, mExecParams);
		}
		KMX_CHECK(kmx_sync());
	}

	const std::vector<F>& getResult() override
	{
		if (this->mResult.empty()) {
			const std::size_t resSize = LAYOUT::size(this->mK, this->mDim);
			std::vector<F> all(resSize * this->mIter), batch;
			for (std::size_t it = 0; it < this->mIter; ++it) {
				mDevResult[it].read(batch, resSize);
				std::copy(batch.begin(), batch.end(), all.begin() + it * resSize);
			}
			bucketing_detail::compact<F, LAYOUT>(this->mResult, all.data(), this->mIter, this->mK, this->mDim);
		}
		return this->mResult;
	}

	void cleanup() override
	{
		IBucketingAlgorithm<F>::cleanup();
		mDevData.clear();
		mDevIndices.clear();
		mDevResult.clear();
	}
};

#endif
