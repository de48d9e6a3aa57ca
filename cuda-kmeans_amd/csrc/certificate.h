/*
 * The certification bounds of the ranking sweeps, in one place, callable from device code and from the host
 * (kmx_certificate_tau exposes them to the tests, which check them against an emulation of the split operands).
 *
 * A sweep ranks the centroids of a point by a[j] ~ A_j = |c_j|^2 - 2 c_j . x. It may decide the point without the
 * serial arithmetic (reference serial.hpp:21-35, metric_policies.hpp:23-28,40-44) only if the two smallest a[j] are
 * further apart than tau, where
 *      tau  >=  2 max_j |a[j] - A_j|  +  (serial margin),
 * the serial margin being the error of two serial sums plus what a correctly rounded sqrt can merge:
 * (2 d + 12) u' S with u' = 2^-23 and S = |x|^2 + max_j |c_j|^2.
 *
 * fp32 MFMA sweeps: |a[j] - A_j| <= (d + 2) u' (|c_j|^2 + 2 |x||c_j|) <= (d + 2) u' 2 S  ->  tau = (8 d + 24) u' S
 * (one u' per accumulation step allows for any rounding or truncation inside the matrix core).
 *
 * Sweeps on the vector ALU (a chain of d v_fma_f32 that starts from the fp32 norm; round to nearest, unit roundoff
 * u = u'/2): the norm carries at most 7 u |c_j|^2 (one product per lane, six levels of the wavefront sum), every fused
 * multiply-add rounds a running value of at most |c_j|^2 + 2 |c_j||x| <= 2 S once, so |a[j] - A_j| <= (2 d + 7) u S and
 * twice that plus the serial margin is (4 d + 19) u' S  ->  tau = (4 d + 24) u' S, about half the MFMA bound.
 *
 * Split-bf16 sweeps. Every operand v is hi + mid + rest with hi = bf16(v), mid = bf16(v - hi), both rounded to nearest:
 * a bf16 has 8 significant bits, so |mid| <= 2^-8 |v|, |rest| <= 2^-8 |mid| <= 2^-17 |v| (the worst case is
 * attained: v = 1 + odd * 2^-17). The sweep adds the products it keeps exactly (8 x 8 bits fit an fp32) and accumulates
 * them in fp32, so
 *      |a[j] - A_j|  <=  (accumulation)  +  |sum_i of the dropped products|.
 *   - three-product form (hi*hi + hi*mid + mid*hi per dimension, c' = -2 c, 3 d products and the norm):
 *        accumulation <= (3 d + 2) u' 2 S
 *        dropped = sum_i c'mid_i xmid_i + (c'hi_i + c'mid_i) xrest_i + c'rest_i x_i
 *                <= |c'mid| |xmid| + (|c'| + |c'rest|) |xrest| + |c'rest| |x|               (Cauchy-Schwarz)
 *        and elementwise |xrest_i| <= 2^-8 |xmid_i|, hence |xrest| <= 2^-8 |xmid|.
 *     The bound is evaluated with the norms of the parts at hand instead of their worst case 2^-15 |c'||x| (= 256 u' S,
 *     which would have to be doubled): |xmid| of the point from the operands the lane holds, max_j |c'mid_j| and
 *     max_j |c'rest_j| from the packing kernel. With random mantissas it comes to about a third of the worst case.
 *   - packed form (rows of at most 4 dimensions, all four hi/mid products kept, 4 d products and the norm):
 *        accumulation <= (4 d + 2) u' 2 S
 *        dropped = sum_i (c'hi_i + c'mid_i) xrest_i + c'rest_i x_i <= (|c'| + |c'rest|) |xrest| + |c'rest| |x|
 *     with |xrest| of the point computed when it is split.
 *     Both forms may work in a frame moved by a vector m (the middle of the centroids), on x' = fl(x - m) and
 *     c' = fl(c - m): distances do not depend on the frame, S becomes |x'|^2 + max_j |c'_j|^2, which is what makes tau
 *     small for data far from the origin, and the two roundings move a distance by at most 2 u (|x'| + |c'|)^2 <= 2 u' S,
 *     a difference of two distances by 4 u' S: 8 u' more in kd (part of the packed form's kd; the launcher adds it to
 *     the three-product form's when that sweep moves its frame).
 *   - one-product form (the first level of the two-level sweep: hi*hi only, d products and the norm):
 *        accumulation <= (d + 2) u' 2 S
 *        dropped = sum_i c'hi_i (x_i - xhi_i) + (c'_i - c'hi_i) x_i <= |c'hi| |xlo| + |c'lo| |x|
 *     with xlo = x - xhi, whose norm the lane computes when it splits the point (the subtraction is exact in fp32),
 *     |c'hi| <= (1 + 2^-8) |c'| and |c'lo| <= |c'mid| + |c'rest| from the packing kernel. The bound is about 2^-8 |c'||x|,
 *     two hundred times the three-product one: this level settles the points whose two nearest centroids are far apart
 *     (86 % at the headline configuration) with a third of the matrix work, the others are swept again with three products.
 * tau = kd S + TRUNC_FACTOR * (bound of the dropped products); kd = (12 d + 8 + 2 d + 12 + slack) u' and
 * (16 d + 8 + 2 d + 12 + 8 + slack) u'; TRUNC_FACTOR = 2 plus 1/16 for the fp32 roundings in the norms and square roots.
 * Values the bound does not cover (NaN, infinities, sums that overflow) make tau NaN or infinite, and the
 * comparison `second - first > tau` is then false: the point goes to the exact pass.
 */
#ifndef KMX_CERTIFICATE_H
#define KMX_CERTIFICATE_H

#if defined(__HIPCC__)
#define KMX_HD __host__ __device__ inline __attribute__((always_inline))
#else
#define KMX_HD inline
#endif

namespace kmx {

constexpr float CERT_UNIT = 1.1920929e-07f;   /* u' = 2^-23 */
constexpr float CERT_TRUNC_FACTOR = 2.0625f;
constexpr float CERT_BF16_UNIT = 0.00390625f; /* 2^-8: relative rounding error of a bf16 */

/* what the packing kernel knows about the centroids of a call: max |c_j|^2, max sum_i c'mid_i^2, max sum_i c'rest_i^2 (c' = -2 c) */
struct CentroidBounds {
	float c2max, mid2max, rest2max;
};

KMX_HD float cert_kd_fp32(unsigned dim) { return (8.0f * (float)dim + 24.0f) * CERT_UNIT; }
KMX_HD float cert_kd_fma(unsigned dim) { return (4.0f * (float)dim + 24.0f) * CERT_UNIT; }
KMX_HD float cert_kd_split(unsigned dim) { return (14.0f * (float)dim + 28.0f) * CERT_UNIT; }
KMX_HD float cert_kd_packed(unsigned dim) { return (18.0f * (float)dim + 36.0f) * CERT_UNIT; }
/* ranking values whose lowest `bits` mantissa bits are replaced (by the centroid's number): a value a moves by less than 2^bits
 * units in its last place, at most 2^bits u' |a|, and |a| = ||c'|^2 - 2 c'.x'| <= 2 |c'|^2 + |x'|^2 <= 2 S; a difference of two
 * values by twice that; the factor's slack covers the roundings inside a. */
KMX_HD float cert_kd_keyed(unsigned bits) { return 2.0f * CERT_TRUNC_FACTOR * (float)(1u << bits) * CERT_UNIT; }
KMX_HD float cert_kd_level1(unsigned dim) { return (6.0f * (float)dim + 28.0f) * CERT_UNIT; } /* 4 d + 8 accumulation, 2 d + 12 serial margin, slack */

/* The bound in the form the kernels evaluate per point: tau = kd (x2 + c2max) + a sqrt(xpart2) + b sqrt(x2), with
 * xpart2 = sum_i xmid_i^2 (three-product form) or sum_i xrest_i^2 (packed form); a and b depend on the centroids only. */
struct CertCoeffs {
	float c2max, a, b;
};

KMX_HD CertCoeffs cert_coeffs_split(const CentroidBounds& c)
{
	const float cnorm = 2.0f * __builtin_sqrtf(c.c2max); /* |c'| */
	const float cmid = __builtin_sqrtf(c.mid2max), crest = __builtin_sqrtf(c.rest2max);
	return CertCoeffs{ c.c2max, CERT_TRUNC_FACTOR * (cmid + (cnorm + crest) * CERT_BF16_UNIT), CERT_TRUNC_FACTOR * crest };
}

/* one-product form: tau = kd (x2 + c2max) + a sqrt(sum_i (x_i - xhi_i)^2) + b sqrt(x2) */
KMX_HD CertCoeffs cert_coeffs_level1(const CentroidBounds& c)
{
	const float cnorm = 2.0f * __builtin_sqrtf(c.c2max); /* |c'| */
	const float clo = __builtin_sqrtf(c.mid2max) + __builtin_sqrtf(c.rest2max); /* >= |c' - c'hi| */
	return CertCoeffs{ c.c2max, CERT_TRUNC_FACTOR * (cnorm * (1.0f + CERT_BF16_UNIT)), CERT_TRUNC_FACTOR * clo };
}

KMX_HD CertCoeffs cert_coeffs_packed(const CentroidBounds& c)
{
	const float cnorm = 2.0f * __builtin_sqrtf(c.c2max);
	const float crest = __builtin_sqrtf(c.rest2max);
	return CertCoeffs{ c.c2max, CERT_TRUNC_FACTOR * (cnorm + crest), CERT_TRUNC_FACTOR * crest };
}

/* a square root that is never below the true one: on the device the hardware's approximation (1 ulp) of an argument kept out
 * of the subnormal range, a millionth added, instead of the correctly rounded sequence of 18 instructions the kernels are
 * compiled with; NaN stays NaN */
KMX_HD float cert_sqrt_upper(float v)
{
#if defined(__HIP_DEVICE_COMPILE__)
	return __builtin_amdgcn_sqrtf(v < 1e-30f ? 1e-30f : v) * 1.000001f;
#else
	return __builtin_sqrtf(v);
#endif
}

KMX_HD float cert_tau(float kd, float x2, float xpart2, const CertCoeffs& c)
{
	return kd * (x2 + c.c2max) + (c.a * cert_sqrt_upper(xpart2) + c.b * cert_sqrt_upper(x2));
}

/*
 * The screening threshold of a sweep in a moved frame, taken back to the frame of the data for a kernel that evaluates
 * a_r[j] ~ A_j = |c_j|^2 - 2 c_j . x there, as a chain of fused multiply-adds. With x' = x - m, c' = c - m:
 *      A'_j = |c'_j|^2 - 2 c'_j . x' = A_j + sh,    sh = 2 x . m - |m|^2 = 2 x' . m + |m|^2      (the same for every j),
 * so a centroid can be the serial result only if A_j <= first' + tau' - sh (first' and tau' of the moved frame), and
 * the kernel may drop j only if a_r[j] exceeds that by more than its own error and the error of the computed sh:
 *   - the chain: (2 d + 7) u (|c_j|^2 + 2 |c_j||x|) <= (2 d + 7) u' Q with Q >= |x|^2 + max_j |c_j|^2 of the data as
 *     given; Q = (|x'| + |m|)^2 + (max_j |c'_j| + |m|)^2 from what the sweep has at hand;
 *   - sh: d products and sums, the rounding of x' = fl(x - m) against m (u |x'||m|) and of |m|^2:
 *     (d + 4) u' (|x'| + |m|)^2 <= (d + 4) u' Q;
 *   - the three roundings of first' + tau' - sh + slack: 2 u' Q.
 * Together (3 d + 13) u' Q, with d the padded length of the chains (up to 15 more than the row); the kernels add
 * (4 d + 40) u' Q. With m = 0 this is first + tau + (4 d + 40) u' S. (The three-product form also pays 8 u' S in kd
 * for the roundings of x' and c', as the packed form does.)
 */
KMX_HD float cert_kd_unmoved(unsigned dim) { return (4.0f * (float)dim + 40.0f) * CERT_UNIT; }
KMX_HD float cert_unmoved_threshold(float first, float tau, float x2, float along, float c2max, float m2, float mnorm, float kdu)
{
	const float sh = 2.0f * along + m2;
	const float xr = cert_sqrt_upper(x2) + mnorm, cr = cert_sqrt_upper(c2max) + mnorm;
	return (first + tau) - sh + kdu * ((xr * xr + cr * cr) * 1.00001f);
}

} // namespace kmx

#endif
