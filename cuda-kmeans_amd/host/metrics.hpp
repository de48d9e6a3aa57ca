/*
 * Distance policies (host side). Contract of the reference's metric_policies.hpp:14-64:
 * distance(data1, idx1, stride1, data2, idx2, stride2, dim). The arithmetic is the one every device
 * kernel must reproduce: difference, square and accumulate in F, ascending dimension, each operation
 * rounded on its own (build without floating-point contraction), then a correctly rounded sqrt.
 */
#ifndef KMX_HOST_METRICS_HPP
#define KMX_HOST_METRICS_HPP

#include "layouts.hpp"

#include <cmath>
#include <cstddef>

template<typename F = float, class LAYOUT1 = AoSLayoutPolicy<>, class LAYOUT2 = LAYOUT1>
class EuclideanSquaredMetricPolicy
{
public:
	static F distance(const F* data1, std::size_t idx1, typename LAYOUT1::precomputed_t stride1,
		const F* data2, std::size_t idx2, typename LAYOUT2::precomputed_t stride2, std::size_t dim)
	{
		F acc = F(0);
		for (std::size_t d = 0; d < dim; ++d) {
			const F diff = LAYOUT1::at(data1, idx1, d, stride1) - LAYOUT2::at(data2, idx2, d, stride2);
			const F sq = diff * diff;
			acc = acc + sq;
		}
		return acc;
	}
};

template<typename F = float, class LAYOUT1 = AoSLayoutPolicy<>, class LAYOUT2 = LAYOUT1>
class EuclideanMetricPolicy
{
public:
	static F distance(const F* data1, std::size_t idx1, typename LAYOUT1::precomputed_t stride1,
		const F* data2, std::size_t idx2, typename LAYOUT2::precomputed_t stride2, std::size_t dim)
	{
		return std::sqrt(EuclideanSquaredMetricPolicy<F, LAYOUT1, LAYOUT2>::distance(data1, idx1, stride1, data2, idx2, stride2, dim));
	}
};

#endif
