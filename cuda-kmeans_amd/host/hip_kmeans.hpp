/*
 * Device-side algorithm objects of the harness: HipKMeansAlgorithm and HipAssignmentAlgorithm, the
 * counterparts of CudaKMeansAlgorithm / CudaAssignmentAlgorithm
 * (experimental/k-means/k-means/headers/cuda.hpp:15-112,237-299): ping-pong centroid and assignment
 * buffers, per iteration  assign -> zero(means[next]) -> zero(sizes) -> update (which ends with the
 * divide), one synchronisation after the loop, results fetched lazily.
 * HipBuffer plays the part of bpp::CudaBuffer (realloc / write / read / free / operator*), on top of
 * the C ABI.
 */
#ifndef KMX_HOST_HIP_KMEANS_HPP
#define KMX_HOST_HIP_KMEANS_HPP

#include "hip_kernels.hpp"
#include "kmeans_interface.hpp"
#include "layouts.hpp"
#include "metrics.hpp"

#include <cstdint>
#include <vector>

template<typename T>
class HipBuffer
{
	T* mPtr = nullptr;
	std::size_t mCount = 0;

public:
	HipBuffer() = default;
	HipBuffer(const HipBuffer&) = delete;
	HipBuffer& operator=(const HipBuffer&) = delete;
	~HipBuffer() { if (mPtr) kmx_free(mPtr); }

	void realloc(std::size_t count)
	{
		free();
		void* p = nullptr;
		KMX_CHECK(kmx_malloc(&p, count * sizeof(T)));
		mPtr = static_cast<T*>(p);
		mCount = count;
	}

	void free()
	{
		if (mPtr) KMX_CHECK(kmx_free(mPtr));
		mPtr = nullptr;
		mCount = 0;
	}

	std::size_t size() const { return mCount; }
	T* operator*() const { return mPtr; }

	/* host -> device; the copy is complete when write() returns */
	void write(const std::vector<T>& src)
	{
		if (src.size() > mCount) throw std::runtime_error("HipBuffer::write: source larger than the buffer");
		KMX_CHECK(kmx_h2d(mPtr, src.data(), src.size() * sizeof(T)));
		KMX_CHECK(kmx_sync());
	}

	/* device -> host (waits for the stream) */
	void read(std::vector<T>& dst, std::size_t count) const
	{
		dst.resize(count);
		KMX_CHECK(kmx_d2h(dst.data(), mPtr, count * sizeof(T)));
	}
};

inline void requireDevice()
{
	int devices = 0;
	KMX_CHECK(kmx_device_count(&devices));
	if (devices == 0) throw std::runtime_error("No HIP devices found!");
	KMX_CHECK(kmx_set_device(0));
}

template<typename F = float, typename IDX_T = std::uint32_t, class LAYOUT = AoSLayoutPolicy<>,
	class LAYOUT_MEANS = LAYOUT, class METRIC = EuclideanMetricPolicy<F, LAYOUT, LAYOUT_MEANS>,
	class ASGN_KERNEL = BaseAssignmentKernel<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC>,
	class UPDATE_KERNEL = UpdateAtomicShmKernel<F, IDX_T, LAYOUT, LAYOUT_MEANS, false>>
class HipKMeansAlgorithm : public IKMeansAlgorithm<F, IDX_T>
{
	HipExecParameters mExecParams;
	bool mResultReady = false;
	HipBuffer<F> mDevData;
	HipBuffer<F> mDevMeans[2];
	HipBuffer<IDX_T> mDevAssignment[2];
	HipBuffer<IDX_T> mDevClusterSizes;
	unsigned mLast = 0;
	/* split timing (optional): events around the assignment and the update of every iteration */
	bool mTimeSplit = false;
	bool mUseGraph = false;
	double mAssignMs = 0.0, mUpdateMs = 0.0;
	std::uint64_t mRechecked = 0;

	std::size_t meansSize() const { return LAYOUT_MEANS::size(this->mK, this->mDim); }

	/* The default pair of kernels on floats -- the selector's assignment and the tuned update -- is one library call
	 * (kmx_iteration_f32), which reads the points once where a single kernel can hold all centroids; the loop body of
	 * cuda.hpp:72-85 otherwise. With the timing split the two halves stay two calls: there is nothing to split in one kernel. */
	static constexpr bool kOneCall = std::is_same<F, float>::value
		&& std::is_same<ASGN_KERNEL, BestCachedAssignmentKernel<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC>>::value
		&& std::is_same<UPDATE_KERNEL, UpdateAtomicShmKernel<F, IDX_T, LAYOUT, LAYOUT_MEANS, false>>::value;

	void fetchResult()
	{
		if (mResultReady) return;
		mDevMeans[mLast].read(this->mMeans, meansSize());
		mDevAssignment[mLast].read(this->mAssignment, this->mN);
		mResultReady = true;
	}

public:
	/* useGraph: replay a recorded pair of iterations instead of launching every kernel (ignored with the timing split) */
	explicit HipKMeansAlgorithm(const HipExecParameters& exec, bool timeSplit = false, bool useGraph = false)
		: mExecParams(exec), mTimeSplit(timeSplit), mUseGraph(useGraph) {}

	void initialize(std::size_t dim, std::size_t k, std::size_t n, std::size_t iters,
		const std::vector<F>& data, const std::vector<F>& means) override
	{
		IKMeansAlgorithm<F, IDX_T>::initialize(dim, k, n, iters, data, means);
		mResultReady = false;
		requireDevice();
		const std::size_t copies = mExecParams.privatizedCopies ? mExecParams.privatizedCopies : 1;
		mDevData.realloc(LAYOUT::size(n, dim));
		mDevClusterSizes.realloc(k);
		for (auto& b : mDevMeans) b.realloc(meansSize() * copies);
		for (auto& b : mDevAssignment) b.realloc(n);
		mDevData.write(data);
		hip_detail::preparePoints<F, LAYOUT>(*mDevData, n, dim);
		mLast = 0;
		mDevMeans[mLast].write(means);
		runFillZeros<IDX_T>(*mDevAssignment[mLast], n);
		runFillZeros<IDX_T>(*mDevClusterSizes, k);
		KMX_CHECK(kmx_sync());
	}

private:
	/* one iteration, launched kernel by kernel, without the optional timing */
	void iterate()
	{
		const std::size_t copies = mExecParams.privatizedCopies ? mExecParams.privatizedCopies : 1;
		const unsigned next = (mLast + 1) % 2;
		if (kOneCall) {
			hip_detail::iteration<F, IDX_T, LAYOUT, LAYOUT_MEANS>(*mDevData, *mDevMeans[mLast], *mDevMeans[next], *mDevAssignment[next],
				*mDevClusterSizes, this->mDim, this->mK, this->mN, mExecParams);
			mLast = next;
			return;
		}
		AssignmentProblemInstance<F, IDX_T> assignment(*mDevData, *mDevMeans[mLast], *mDevAssignment[mLast],
			*mDevAssignment[next], this->mDim, this->mK, this->mN);
		ASGN_KERNEL::run(assignment, mExecParams);
		if (UPDATE_KERNEL::needsZeroedOutput) {
			runFillZeros<F>(*mDevMeans[next], meansSize() * copies);
			runFillZeros<IDX_T>(*mDevClusterSizes, this->mK);
		}
		UpdateProblemInstance<F, IDX_T> update(*mDevData, *mDevAssignment[next], *mDevMeans[next], *mDevClusterSizes,
			this->mDim, this->mK, this->mN);
		UPDATE_KERNEL::run(update, mExecParams);
		mLast = next;
	}

	/* the first iteration sizes the library's work space, then two ping-pong iterations are recorded once and replayed */
	void runRecorded()
	{
		iterate();
		const std::size_t pairs = (this->mIters - 1) / 2;
		void* graph = nullptr;
		KMX_CHECK(kmx_graph_begin());
		try {
			iterate();
			iterate();
		}
		catch (...) {
			kmx_graph_end(&graph);
			kmx_graph_destroy(graph);
			throw;
		}
		KMX_CHECK(kmx_graph_end(&graph));
		for (std::size_t i = 0; i < pairs; ++i) KMX_CHECK(kmx_graph_launch(graph));
		for (std::size_t done = 1 + 2 * pairs; done < this->mIters; ++done) iterate();
		KMX_CHECK(kmx_sync());
		KMX_CHECK(kmx_graph_destroy(graph));
	}

public:
	void run() override
	{
		if (mUseGraph && !mTimeSplit && this->mIters >= 3) { runRecorded(); return; }
		if (kOneCall && !mTimeSplit) {
			for (std::size_t iter = 0; iter < this->mIters; ++iter) iterate();
			KMX_CHECK(kmx_sync());
			return;
		}
		void* ev[3] = { nullptr, nullptr, nullptr };
		if (mTimeSplit) for (auto& e : ev) KMX_CHECK(kmx_event_create(&e));
		const std::size_t copies = mExecParams.privatizedCopies ? mExecParams.privatizedCopies : 1;
		for (std::size_t iter = 0; iter < this->mIters; ++iter) {
			const unsigned next = (mLast + 1) % 2;
			if (mTimeSplit) KMX_CHECK(kmx_event_record(ev[0]));
			AssignmentProblemInstance<F, IDX_T> assignment(*mDevData, *mDevMeans[mLast], *mDevAssignment[mLast],
				*mDevAssignment[next], this->mDim, this->mK, this->mN);
			ASGN_KERNEL::run(assignment, mExecParams);
			if (mTimeSplit) KMX_CHECK(kmx_event_record(ev[1]));

			if (UPDATE_KERNEL::needsZeroedOutput) {
				runFillZeros<F>(*mDevMeans[next], meansSize() * copies);
				runFillZeros<IDX_T>(*mDevClusterSizes, this->mK);
			}
			UpdateProblemInstance<F, IDX_T> update(*mDevData, *mDevAssignment[next], *mDevMeans[next], *mDevClusterSizes,
				this->mDim, this->mK, this->mN);
			UPDATE_KERNEL::run(update, mExecParams);
			if (mTimeSplit) {
				KMX_CHECK(kmx_event_record(ev[2]));
				float a = 0, u = 0;
				KMX_CHECK(kmx_event_elapsed_ms(ev[0], ev[1], &a));
				KMX_CHECK(kmx_event_elapsed_ms(ev[1], ev[2], &u));
				mAssignMs += a;
				mUpdateMs += u;
				std::uint64_t r = 0;
				KMX_CHECK(kmx_assign_last_rechecked(&r));
				mRechecked += r;
			}
			mLast = next;
		}
		KMX_CHECK(kmx_sync());
		for (auto e : ev) if (e) KMX_CHECK(kmx_event_destroy(e));
	}

	const std::vector<F>& getMeans() override { fetchResult(); return this->mMeans; }
	const std::vector<IDX_T>& getAssignment() override { fetchResult(); return this->mAssignment; }

	/* totals over the iterations of the last run(); meaningful only with timeSplit */
	double assignMs() const { return mAssignMs; }
	double updateMs() const { return mUpdateMs; }
	std::uint64_t recheckedPoints() const { return mRechecked; }

	void cleanup() override
	{
		IKMeansAlgorithm<F, IDX_T>::cleanup();
		hip_detail::forgetPoints<F>(*mDevData);
		mDevData.free();
		for (auto& b : mDevMeans) b.free();
		for (auto& b : mDevAssignment) b.free();
		mDevClusterSizes.free();
	}
};

/*
 * Counterpart of CudaFusedKMeansAlgorithm (cuda.hpp:116-233): no assignment buffers; every iteration zero-fills the
 * next centroid buffer and the counts and makes one FUSED kernel call. As in the reference, getAssignment() is not a
 * by-product of the iterations: it is computed afterwards against the FINAL centroids (the reference scans on the
 * host, cuda.hpp:199-221; here the device runs one more assignment pass, which returns the same indices).
 */
template<typename F = float, typename IDX_T = std::uint32_t, class LAYOUT = AoSLayoutPolicy<>,
	class LAYOUT_MEANS = LAYOUT, class METRIC = EuclideanMetricPolicy<F, LAYOUT, LAYOUT_MEANS>,
	class KERNEL = FusedBestKernel<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC>>
class HipFusedKMeansAlgorithm : public IKMeansAlgorithm<F, IDX_T>
{
	HipExecParameters mExecParams;
	bool mMeansReady = false, mAssignmentReady = false;
	HipBuffer<F> mDevData;
	HipBuffer<F> mDevMeans[2];
	HipBuffer<IDX_T> mDevClusterSizes;
	unsigned mLast = 0;

	std::size_t meansSize() const { return LAYOUT_MEANS::size(this->mK, this->mDim); }

public:
	explicit HipFusedKMeansAlgorithm(const HipExecParameters& exec) : mExecParams(exec) {}

	void initialize(std::size_t dim, std::size_t k, std::size_t n, std::size_t iters,
		const std::vector<F>& data, const std::vector<F>& means) override
	{
		IKMeansAlgorithm<F, IDX_T>::initialize(dim, k, n, iters, data, means);
		mMeansReady = mAssignmentReady = false;
		requireDevice();
		mDevData.realloc(LAYOUT::size(n, dim));
		mDevClusterSizes.realloc(k);
		for (auto& b : mDevMeans) b.realloc(meansSize());
		mDevData.write(data);
		hip_detail::preparePoints<F, LAYOUT>(*mDevData, n, dim);
		mLast = 0;
		mDevMeans[mLast].write(means);
		runFillZeros<IDX_T>(*mDevClusterSizes, k);
		KMX_CHECK(kmx_sync());
	}

	void run() override
	{
		for (std::size_t iter = 0; iter < this->mIters; ++iter) {
			const unsigned next = (mLast + 1) % 2;
			runFillZeros<F>(*mDevMeans[next], meansSize());
			runFillZeros<IDX_T>(*mDevClusterSizes, this->mK);
			FusedProblemInstance<F, IDX_T> fused(*mDevData, *mDevMeans[mLast], *mDevMeans[next], *mDevClusterSizes,
				this->mDim, this->mK, this->mN);
			KERNEL::run(fused, mExecParams);
			mLast = next;
		}
		KMX_CHECK(kmx_sync());
	}

	const std::vector<F>& getMeans() override
	{
		if (!mMeansReady) {
			mDevMeans[mLast].read(this->mMeans, meansSize());
			mMeansReady = true;
		}
		return this->mMeans;
	}

	const std::vector<IDX_T>& getAssignment() override
	{
		if (!mAssignmentReady) {
			HipBuffer<IDX_T> out;
			out.realloc(this->mN);
			AssignmentProblemInstance<F, IDX_T> assignment(*mDevData, *mDevMeans[mLast], nullptr, *out, this->mDim, this->mK, this->mN);
			BestCachedAssignmentKernel<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC>::run(assignment, mExecParams);
			out.read(this->mAssignment, this->mN);
			out.free();
			mAssignmentReady = true;
		}
		return this->mAssignment;
	}

	void cleanup() override
	{
		IKMeansAlgorithm<F, IDX_T>::cleanup();
		hip_detail::forgetPoints<F>(*mDevData);
		mDevData.free();
		for (auto& b : mDevMeans) b.free();
		mDevClusterSizes.free();
	}
};

template<typename F = float, typename IDX_T = std::uint32_t, class LAYOUT = AoSLayoutPolicy<>,
	class LAYOUT_MEANS = LAYOUT, class METRIC = EuclideanMetricPolicy<F, LAYOUT, LAYOUT_MEANS>,
	class KERNEL = BaseAssignmentKernel<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC>>
class HipAssignmentAlgorithm : public IAssignmentAlgorithm<F, IDX_T>
{
	HipExecParameters mExecParams;
	bool mResultReady = false;
	HipBuffer<F> mDevData;
	HipBuffer<F> mDevMeans;
	HipBuffer<IDX_T> mDevAssignment;

public:
	explicit HipAssignmentAlgorithm(const HipExecParameters& exec) : mExecParams(exec) {}

	void initialize(std::size_t dim, std::size_t k, std::size_t n, const std::vector<F>& data, const std::vector<F>& means) override
	{
		IAssignmentAlgorithm<F, IDX_T>::initialize(dim, k, n, data, means);
		mResultReady = false;
		requireDevice();
		mDevData.realloc(LAYOUT::size(n, dim));
		mDevMeans.realloc(LAYOUT_MEANS::size(k, dim));
		mDevAssignment.realloc(n);
		mDevData.write(data);
		mDevMeans.write(means);
		KMX_CHECK(kmx_sync());
	}

	void run() override
	{
		AssignmentProblemInstance<F, IDX_T> instance(*mDevData, *mDevMeans, nullptr, *mDevAssignment, this->mDim, this->mK, this->mN);
		KERNEL::run(instance, mExecParams);
		KMX_CHECK(kmx_sync());
	}

	const std::vector<IDX_T>& getAssignment() override
	{
		if (!mResultReady) {
			mDevAssignment.read(this->mAssignment, this->mN);
			mResultReady = true;
		}
		return this->mAssignment;
	}

	void cleanup() override
	{
		IAssignmentAlgorithm<F, IDX_T>::cleanup();
		mDevData.free();
		mDevMeans.free();
		mDevAssignment.free();
	}
};

#endif
