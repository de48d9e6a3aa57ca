/*
 * Data layout policies of the k-means harness (host side).
 *
 * Same contract as the reference's SoALayoutPolicy / AoSLayoutPolicy
 * (experimental/k-means/k-means/headers/layout_policies.hpp:14-60): `size(n, dims)` floats are needed for
 * n vectors, `precomputeConstants(n, dims)` is the stride, `at(data, idx, dim, stride)` addresses one
 * coordinate. ALIGN pads the stride to a multiple of ALIGN elements. `ID` is the kmx_layout value the
 * device boundary understands (include/kmx.h); the stride is what crosses it.
 */
#ifndef KMX_HOST_LAYOUTS_HPP
#define KMX_HOST_LAYOUTS_HPP

#include <cstddef>

namespace detail {
constexpr std::size_t pad_to(std::size_t v, std::size_t align) { return (v + align - 1) / align * align; }
}

/* structure of arrays: coordinate `dim` of all vectors is contiguous; stride = padded number of vectors */
template<int ALIGN = 32>
class SoALayoutPolicy
{
public:
	using precomputed_t = std::size_t;
	static constexpr int ID = 1; /* KMX_SOA */

	static std::size_t precomputeConstants(std::size_t n, std::size_t /*dims*/) { return detail::pad_to(n, ALIGN); }
	static std::size_t size(std::size_t n, std::size_t dims) { return precomputeConstants(n, dims) * dims; }

	template<typename F>
	static F& at(F* data, std::size_t idx, std::size_t dim, precomputed_t stride) { return data[dim * stride + idx]; }
};

/* array of structures: the coordinates of one vector are contiguous; stride = padded dimension */
template<int ALIGN = 1>
class AoSLayoutPolicy
{
public:
	using precomputed_t = std::size_t;
	static constexpr int ID = 0; /* KMX_AOS */

	static std::size_t precomputeConstants(std::size_t /*n*/, std::size_t dims) { return detail::pad_to(dims, ALIGN); }
	static std::size_t size(std::size_t n, std::size_t dims) { return precomputeConstants(n, dims) * n; }

	template<typename F>
	static F& at(F* data, std::size_t idx, std::size_t dim, precomputed_t stride) { return data[idx * stride + dim]; }
};

#endif
