/*
 * Host (CPU) k-means: the `serial` algorithm of the command line and the yardstick of --verify.
 *
 * Semantics of the reference's SerialKMeansAlgorithm / SerialAssignmentAlgorithm
 * (experimental/k-means/k-means/headers/serial.hpp:12-149):
 *   assignment  nearest centroid by METRIC::distance, strict comparison starting at centroid 0, so the
 *               lowest index wins equal distances and a NaN distance never wins;
 *   update      zero, count, add the members in ascending point order, divide by (F)count; a cluster
 *               without members stays at the origin;
 *   run()       iters x (means become the previous means; assign against them; update).
 * The reference runs on one thread. `threads` > 1 (OpenMP) splits the points of the assignment and the
 * clusters of the update over threads; every sum keeps its ascending point order, so the results are
 * bit-identical to the single-threaded run.
 */
#ifndef KMX_HOST_SERIAL_KMEANS_HPP
#define KMX_HOST_SERIAL_KMEANS_HPP

#include "kmeans_interface.hpp"
#include "layouts.hpp"
#include "metrics.hpp"

#include <cstdint>
#include <vector>
#ifdef _OPENMP
#include <omp.h>
#endif

namespace serial_detail {

template<typename F, typename IDX_T, class LAYOUT, class LAYOUT_MEANS, class METRIC>
void assign(const F* data, const F* means, std::size_t dim, std::size_t k, std::size_t n, IDX_T* assignment, int threads)
{
	const auto strideData = LAYOUT::precomputeConstants(n, dim);
	const auto strideMeans = LAYOUT_MEANS::precomputeConstants(k, dim);
	(void)threads;
#ifdef _OPENMP
#pragma omp parallel for schedule(static) num_threads(threads) if (threads > 1)
#endif
	for (std::int64_t i = 0; i < (std::int64_t)n; ++i) {
		IDX_T nearest = 0;
		F best = METRIC::distance(data, (std::size_t)i, strideData, means, 0, strideMeans, dim);
		for (IDX_T m = 1; m < k; ++m) {
			const F dist = METRIC::distance(data, (std::size_t)i, strideData, means, m, strideMeans, dim);
			if (best > dist) {
				best = dist;
				nearest = m;
			}
		}
		assignment[i] = nearest;
	}
}

template<typename F, typename IDX_T, class LAYOUT, class LAYOUT_MEANS>
void update(const F* data, const IDX_T* assignment, std::size_t dim, std::size_t k, std::size_t n, F* means, IDX_T* sizes, int threads)
{
	const auto strideData = LAYOUT::precomputeConstants(n, dim);
	const auto strideMeans = LAYOUT_MEANS::precomputeConstants(k, dim);
	for (std::size_t c = 0; c < k; ++c) {
		sizes[c] = 0;
		for (std::size_t d = 0; d < dim; ++d) LAYOUT_MEANS::at(means, c, d, strideMeans) = F(0);
	}
	if (threads < 1) threads = 1;
	if ((std::size_t)threads > k) threads = (int)k;
#ifdef _OPENMP
#pragma omp parallel num_threads(threads) if (threads > 1)
#endif
	{
#ifdef _OPENMP
		const std::size_t t = (std::size_t)omp_get_thread_num(), T = (std::size_t)omp_get_num_threads();
#else
		const std::size_t t = 0, T = 1;
#endif
		for (std::size_t i = 0; i < n; ++i) {
			const std::size_t target = assignment[i];
			if (T > 1 && target % T != t) continue; /* a cluster belongs to one thread: ascending order is kept */
			++sizes[target];
			for (std::size_t d = 0; d < dim; ++d)
				LAYOUT_MEANS::at(means, target, d, strideMeans) += LAYOUT::at(data, i, d, strideData);
		}
	}
	for (std::size_t c = 0; c < k; ++c) {
		if (sizes[c] == 0) continue;
		const F divisor = (F)sizes[c];
		for (std::size_t d = 0; d < dim; ++d) LAYOUT_MEANS::at(means, c, d, strideMeans) /= divisor;
	}
}

} // namespace serial_detail

template<typename F = float, typename IDX_T = std::uint32_t, class LAYOUT = AoSLayoutPolicy<>,
	class LAYOUT_MEANS = LAYOUT, class METRIC = EuclideanMetricPolicy<F, LAYOUT, LAYOUT_MEANS>>
class SerialKMeansAlgorithm : public IKMeansAlgorithm<F, IDX_T>
{
	const F* mData = nullptr;
	std::vector<F> mPrevMeans;
	std::vector<IDX_T> mClusterSizes;
	int mThreads;

public:
	explicit SerialKMeansAlgorithm(int threads = 1) : mThreads(threads) {}

	void initialize(std::size_t dim, std::size_t k, std::size_t n, std::size_t iters,
		const std::vector<F>& data, const std::vector<F>& means) override
	{
		IKMeansAlgorithm<F, IDX_T>::initialize(dim, k, n, iters, data, means);
		mData = data.data();
		this->mMeans = means;
		mPrevMeans.assign(LAYOUT_MEANS::size(k, dim), F(0));
		mClusterSizes.assign(k, 0);
		this->mAssignment.assign(n, 0);
	}

	void run() override
	{
		for (std::size_t iter = 0; iter < this->mIters; ++iter) {
			this->mMeans.swap(mPrevMeans);
			serial_detail::assign<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC>(mData, mPrevMeans.data(), this->mDim, this->mK, this->mN,
				this->mAssignment.data(), mThreads);
			serial_detail::update<F, IDX_T, LAYOUT, LAYOUT_MEANS>(mData, this->mAssignment.data(), this->mDim, this->mK, this->mN,
				this->mMeans.data(), mClusterSizes.data(), mThreads);
		}
	}

	const std::vector<IDX_T>& getClusterSizes() const { return mClusterSizes; }

	void cleanup() override
	{
		IKMeansAlgorithm<F, IDX_T>::cleanup();
		mPrevMeans.clear();
		mClusterSizes.clear();
	}
};

template<typename F = float, typename IDX_T = std::uint32_t, class LAYOUT = AoSLayoutPolicy<>,
	class LAYOUT_MEANS = LAYOUT, class METRIC = EuclideanMetricPolicy<F, LAYOUT, LAYOUT_MEANS>>
class SerialAssignmentAlgorithm : public IAssignmentAlgorithm<F, IDX_T>
{
	const F* mData = nullptr;
	const F* mMeans = nullptr;
	int mThreads;

public:
	explicit SerialAssignmentAlgorithm(int threads = 1) : mThreads(threads) {}

	void initialize(std::size_t dim, std::size_t k, std::size_t n, const std::vector<F>& data, const std::vector<F>& means) override
	{
		IAssignmentAlgorithm<F, IDX_T>::initialize(dim, k, n, data, means);
		mData = data.data();
		mMeans = means.data();
	}

	void run() override
	{
		serial_detail::assign<F, IDX_T, LAYOUT, LAYOUT_MEANS, METRIC>(mData, mMeans, this->mDim, this->mK, this->mN,
			this->mAssignment.data(), mThreads);
	}
};

#endif
