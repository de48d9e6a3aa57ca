/*
 * Algorithm interfaces of the harness: what the command line selects by name and drives.
 * Same contract as the reference's IKMeansAlgorithm / IAssignmentAlgorithm
 * (experimental/k-means/k-means/headers/interface.hpp:7-84): initialize() receives the problem and may
 * move data to the device, run() performs the iterations, getMeans()/getAssignment() return the result
 * (fetched lazily by device implementations), cleanup() releases everything.
 */
#ifndef KMX_HOST_KMEANS_INTERFACE_HPP
#define KMX_HOST_KMEANS_INTERFACE_HPP

#include <cstddef>
#include <cstdint>
#include <vector>

template<typename F = float, typename IDX_T = std::uint32_t>
class IKMeansAlgorithm
{
protected:
	std::size_t mDim = 0, mK = 0, mN = 0, mIters = 1;
	std::vector<F> mMeans;
	std::vector<IDX_T> mAssignment;

public:
	virtual ~IKMeansAlgorithm() = default;

	/* iterations actually performed (an implementation may stop early) */
	std::size_t getIterations() const { return mIters; }

	virtual void initialize(std::size_t dim, std::size_t k, std::size_t n, std::size_t iters,
		const std::vector<F>& /*data*/, const std::vector<F>& /*means*/)
	{
		mDim = dim; mK = k; mN = n; mIters = iters;
	}

	virtual void run() = 0;

	/* centroids after the last update */
	virtual const std::vector<F>& getMeans() { return mMeans; }

	/* assignment computed in the last iteration (against the centroids before the last update) */
	virtual const std::vector<IDX_T>& getAssignment() { return mAssignment; }

	virtual void cleanup()
	{
		mMeans.clear();
		mAssignment.clear();
	}
};

template<typename F = float, typename IDX_T = std::uint32_t>
class IAssignmentAlgorithm
{
protected:
	std::size_t mDim = 0, mK = 0, mN = 0;
	std::vector<IDX_T> mAssignment;

public:
	virtual ~IAssignmentAlgorithm() = default;

	virtual void initialize(std::size_t dim, std::size_t k, std::size_t n,
		const std::vector<F>& /*data*/, const std::vector<F>& /*means*/)
	{
		mDim = dim; mK = k; mN = n;
		mAssignment.resize(n);
	}

	virtual void run() = 0;

	virtual const std::vector<IDX_T>& getAssignment() { return mAssignment; }

	virtual void cleanup() { mAssignment.clear(); }
};

#endif
