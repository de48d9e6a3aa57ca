"""Inputs aimed at the certificate of the ranking sweeps, on a real MI355X (-m gpu): every variant must return the serial
scan's index bit for bit where random data never probes the bound.

  * worst-case pairs (tests/test_certificate.py): every product the split-bf16 sweep drops has one sign for one kind of
    centroid and the other sign for its rival, on near-ties; a bound derived for 9-bit parts decides some of these
    points wrongly (shown on the CPU by test_certificate.py), so a sweep that certified too much would fail here;
  * a gap sweep: a million points, each next to the bisector of two centroids with a true gap log-uniform over
    [1e-9, 1e-3] (|ca|^2 + |cb|^2), coordinates shifted by 0, 1e2, 1e4 so that the magnitudes dwarf the gap.
"""
import numpy as np
import pytest

from test_certificate import U, accumulation_cases, exact_chain, near_ties, worst_case_inputs

pytestmark = pytest.mark.gpu

AOS = 0


def variants(km, dim):
    v = [km.ASSIGN_BEST, km.ASSIGN_MFMA_BF16X3, km.ASSIGN_MFMA, km.ASSIGN_BASE]
    return v + [km.ASSIGN_LDS_FMA] if dim <= 64 else v


def assign_all(km, data_buf, means, dim, k, n, variant):
    m = km.DeviceBuffer(means.nbytes); m.write(means)
    a = km.DeviceBuffer(4 * n)
    km.assign(variant, data_buf, AOS, dim, m, AOS, dim, a, dim, k, n)
    km.sync()
    out = a.read(np.uint32, n)
    rechecked = km.last_rechecked()
    m.free(); a.free()
    return out, rechecked


@pytest.mark.parametrize("dim", [2, 3, 4, 8, 16, 32, 64])
def test_worst_case_pairs_match_the_serial_scan(km, orc, gpu, dim):
    x, c = worst_case_inputs(dim, 64000)
    n, k = x.shape[0], c.shape[0]
    data, means = np.ascontiguousarray(x).ravel(), np.ascontiguousarray(c).ravel()
    want = orc.assign(data, means, dim, k, n, threads=0, fast=True)
    d = km.DeviceBuffer(data.nbytes); d.write(data)
    for v in variants(km, dim):
        got, rechecked = assign_all(km, d, means, dim, k, n, v)
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, "variant %d: %d of %d points differ from the serial scan (first %s), %d went to the exact pass" % (
            v, bad.size, n, bad[:5], rechecked)
    d.free()


@pytest.mark.parametrize("dim", [2, 3, 4])
def test_worst_case_pairs_in_the_moved_frame_of_the_packed_sweep(km, orc, gpu, dim):
    """From 128 centroids on the packed sweep works in a frame moved to the centroids' mean. 128 centroids in mirrored pairs
    have the mean 0 exactly, so the frame is the data's own and the worst-case signs of the dropped products survive."""
    x, c = worst_case_inputs(dim, 64000, mirrored=True, pairs=64)
    n, k = x.shape[0], c.shape[0]
    assert k == 128
    data, means = np.ascontiguousarray(x).ravel(), np.ascontiguousarray(c).ravel()
    want = orc.assign(data, means, dim, k, n, threads=0, fast=True)
    d = km.DeviceBuffer(data.nbytes); d.write(data)
    for v in (km.ASSIGN_BEST, km.ASSIGN_MFMA_BF16X3):
        got, rechecked = assign_all(km, d, means, dim, k, n, v)
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, "variant %d: %d of %d points differ from the serial scan (first %s), %d went to the exact pass" % (
            v, bad.size, n, bad[:5], rechecked)
    d.free()


def test_quoted_packed_example_of_a_wrong_decision(km, orc, gpu):
    """Two dimensions, x between c1 and c2 with a true gap below what the split drops: the ranking values differ by more
    than (18 d + 149) u' S in favour of c2 while the serial scan returns c1."""
    x = np.float32([1.0037002563476562, 1.0041122436523438])
    c1 = np.float32([1.0037307739257812, -1.0033798217773438])
    c2 = np.float32([-1.0037918090820312, 1.0016860961914062])
    n, k, dim = 4096, 512, 2
    rng = np.random.default_rng(2)
    means = (rng.normal(size=(k, dim)) * 40 + 100).astype(np.float32)      # far away
    means[7], means[300] = c2, c1
    data = np.tile(x, (n, 1)).astype(np.float32)
    data[1::2] += rng.integers(-3, 4, size=(n // 2, dim)).astype(np.float32) * np.float32(2.0 ** -17)
    want = orc.assign(data.ravel(), means.ravel(), dim, k, n, threads=0, fast=True)
    assert want[0] == 300
    d = km.DeviceBuffer(data.nbytes); d.write(data.ravel())
    for v in variants(km, dim):
        got, _ = assign_all(km, d, means.ravel(), dim, k, n, v)
        assert np.array_equal(got, want), "variant %d: %d mismatches" % (v, int((got != want).sum()))
    d.free()


@pytest.mark.parametrize("dim", [4, 32, 256])
@pytest.mark.parametrize("offset", [0.0, 1e2, 1e4])
def test_gap_sweep(km, orc, gpu, dim, offset):
    n, k, chunk = 1 << 20, 128, 1 << 16
    rng = np.random.default_rng(int(dim * 7 + offset))
    _, c = near_ties(dim, 1, k, rng, offset)
    data = np.empty((n, dim), np.float32)
    for first in range(0, n, chunk):                 # the generator works in float64: in pieces
        data[first:first + chunk], _ = near_ties(dim, chunk, k, rng, offset, centroids=c)
    means = np.ascontiguousarray(c).ravel()
    want = orc.assign(data.ravel(), means, dim, k, n, threads=0, fast=True)
    d = km.DeviceBuffer(data.nbytes); d.write(data.ravel())
    for v in variants(km, dim):
        got, rechecked = assign_all(km, d, means, dim, k, n, v)
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, "variant %d: %d of %d points differ (first %s), %d went to the exact pass" % (v, bad.size, n, bad[:5], rechecked)
    d.free()


@pytest.mark.parametrize("kind", [0, 1, 2])
def test_matrix_core_accumulation_stays_within_one_unit_per_step(km, gpu, kind):
    """The hardware assumption of the certificates (csrc/certificate.h: one u' of the running magnitude per accumulated
    product covers whatever the matrix core rounds or truncates), measured: chains of v_mfma_f32_32x32x2_f32 (kind 0),
    v_mfma_f32_32x32x16_bf16 (kind 1) and v_mfma_f32_16x16x4_f32 (kind 2) on products of exponents 2^0..2^-20 inside a block, cancelling pairs next to a term
    of 2^-20, a large accumulator with addends below its last place, up to 48 blocks. tests/test_certificate.py shows that
    an accumulator which truncates after every product fails half of this bound on the same operands."""
    worst = 0.0
    for name, (a, b, c) in accumulation_cases(kind).items():
        d = km.probe_matrix_chain(kind, a, b, c).astype(np.float64)
        exact, m = exact_chain(a, b, c)
        steps = a.shape[1]
        per_step = np.abs(d - exact) / (steps * U * m)
        assert per_step.max() <= 1.0, "%s: %.3f u' of the running magnitude per step" % (name, float(per_step.max()))
        worst = max(worst, float(per_step.max()))
    print("matrix cores, kind %d: at most %.4f u' of the running magnitude per accumulated product" % (kind, worst))


@pytest.mark.parametrize("dim", [16, 32, 64, 256])
def test_gap_sweep_with_coordinates_of_very_different_exponents(km, orc, gpu, dim):
    """Near-ties (true gaps log-uniform over 1e-9..1e-3 of |ca|^2 + |cb|^2, on both sides of every tau) between centroids
    whose coordinates span 2^0..2^-10 inside every block of 16 dimensions with alternating signs, so that the products of
    one matrix-core block span 2^0..2^-20 and partly cancel: every variant must return the serial scan's index."""
    n, k, chunk = 1 << 18, 128, 1 << 16
    rng = np.random.default_rng(dim)
    scale = (2.0 ** -(np.arange(dim) % 11)).astype(np.float32)
    sign = np.where(np.arange(dim) % 2 == 0, 1.0, -1.0).astype(np.float32)
    c = ((1.0 + rng.random(size=(k, dim))) * scale * sign * rng.choice([1.0, 1.0, 1.0, -1.0], size=(k, dim))).astype(np.float32)
    data = np.empty((n, dim), np.float32)
    for first in range(0, n, chunk):
        data[first:first + chunk], _ = near_ties(dim, chunk, k, rng, 0.0, centroids=c)
    means = np.ascontiguousarray(c).ravel()
    want = orc.assign(data.ravel(), means, dim, k, n, threads=0, fast=True)
    d = km.DeviceBuffer(data.nbytes); d.write(data.ravel())
    for v in variants(km, dim):
        got, rechecked = assign_all(km, d, means, dim, k, n, v)
        bad = np.nonzero(got != want)[0]
        assert bad.size == 0, "variant %d: %d of %d points differ (first %s), %d went to the exact pass" % (v, bad.size, n, bad[:5], rechecked)
    d.free()


@pytest.mark.parametrize("dim,k", [(16, 16), (32, 32), (8, 20), (4, 16), (24, 9), (16, 3)])
@pytest.mark.parametrize("offset", [0.0, 1e2, 1e4])
def test_gap_sweep_through_the_single_pass_iteration(km, orc, gpu, dim, k, offset):
    """The gap sweep (points next to bisectors, true gaps log-uniform over 1e-9..1e-3 on both sides of every tau) through
    kmx_iteration_f32 where it reads the points once: the ranking values of those kernels carry the centroid's number in
    their low bits (csrc/certificate.h: cert_kd_keyed), the rows of 8, 16 and 32 floats rank on v_mfma_f32_16x16x4_f32.
    The assignment is the serial scan's, the counts are exact."""
    n, chunk = 1 << 19, 1 << 16
    rng = np.random.default_rng(int(dim * 11 + k + offset))
    _, c = near_ties(dim, 1, k, rng, offset)
    data = np.empty((n, dim), np.float32)
    for first in range(0, n, chunk):
        data[first:first + chunk], _ = near_ties(dim, chunk, k, rng, offset, centroids=c)
    means = np.ascontiguousarray(c).ravel()
    want = orc.assign(data.ravel(), means, dim, k, n, threads=0, fast=True)
    d = km.DeviceBuffer(data.nbytes); d.write(data.ravel())
    m = km.DeviceBuffer(means.nbytes); m.write(means)
    out = km.DeviceBuffer(means.nbytes); a = km.DeviceBuffer(4 * n); sizes = km.DeviceBuffer(4 * k)
    km.iteration(d, 0, dim, m, out, 0, dim, a, sizes, dim, k, n)
    km.sync()
    assert km.last_iteration_passes() == 1
    got = a.read(np.uint32, n)
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, "%d of %d points differ (first %s)" % (bad.size, n, bad[:5])
    assert np.array_equal(sizes.read(np.uint32, k), np.bincount(want, minlength=k))
    for b in (d, m, out, a, sizes):
        b.free()
