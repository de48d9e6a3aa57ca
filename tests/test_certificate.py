"""The certification bound of the split-bf16 sweeps against an emulation of their arithmetic (CPU, no GPU).

The sweeps rank centroids with a[j] = |c_j|^2 + sum_i (kept products of the split operands) and decide a point without
the serial arithmetic when its two smallest a[j] differ by more than tau. The emulation here splits the operands
exactly as the kernels do (bf16, round to nearest even), adds the kept products without error (float64 holds them
exactly) and compares with the exact A_j = |c_j|^2 - 2 c_j . x: the difference is what the split drops. tau (from the
library's own function, kmx_certificate_tau) must cover twice that plus the accumulation allowance plus the serial
margin; and wherever the emulated ranking, disturbed by the full accumulation allowance, would certify a pair, the
serial oracle must agree with the decision.

The inputs are the worst cases of the split, which random data never reaches: coordinates 1 + odd * 2^-17 (both
remainders at their maximum) against centroids c and about -c, plus near-ties at every scale.
"""
import numpy as np
import pytest

U = 2.0 ** -23


def bf16_round(v):
    """float32 -> nearest bf16 (ties to even), returned as float32."""
    bits = np.asarray(v, np.float32).view(np.uint32).astype(np.uint64)
    bits = (bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000
    return bits.astype(np.uint32).view(np.float32)


def split(v):
    v = np.asarray(v, np.float32)
    hi = bf16_round(v)
    r = (v - hi).astype(np.float32)
    mid = bf16_round(r)
    rest = (r - mid).astype(np.float32)
    assert np.array_equal(hi.astype(np.float64) + mid.astype(np.float64) + rest.astype(np.float64), v.astype(np.float64))
    return hi, mid, rest


def test_split_remainders_reach_their_stated_worst_case():
    v = (1.0 + np.arange(1, 1 << 17, 2, dtype=np.float64) * 2.0 ** -17).astype(np.float32)
    hi, mid, rest = split(v)
    assert np.abs(mid / v).max() <= 2.0 ** -8 and np.abs(mid / v).max() > 0.99 * 2.0 ** -8
    assert np.abs(rest / v).max() <= 2.0 ** -17 and np.abs(rest / v).max() > 0.99 * 2.0 ** -17
    nz = mid != 0
    assert np.all(np.abs(rest[nz]) <= 2.0 ** -8 * np.abs(mid[nz]))


def adversarial(dim, n, k, rng):
    """Coordinates 1 + m * 2^-17 with odd m up to 511 (|mid| / |v| and |rest| / |v| next to their maxima), random signs.
    Centroids come in pairs (c, about -c) and half of the points are copies of a centroid: the products the split drops
    then all have one sign for c and the other for -c, so the two ranking values move apart by the sum of the bounds."""
    def worst(shape):
        return (1.0 + (2 * rng.integers(128, 256, size=shape) + 1) * 2.0 ** -17).astype(np.float32)
    c = worst((k, dim)) * rng.choice(np.float32([-1, 1]), size=(k, dim))
    c[1::2] = -c[0::2][: c[1::2].shape[0]] * (1 + rng.integers(-3, 4, size=c[1::2].shape) * np.float32(2.0 ** -12))
    x = worst((n, dim)) * rng.choice(np.float32([-1, 1]), size=(n, dim))
    x[: n // 2] = c[rng.integers(0, k, size=n // 2)]
    return x.astype(np.float32), c.astype(np.float32)


def worst_parts(rng, shape, mid_sign, rest_sign):
    """1 + m 2^-17 (m < 1024) whose split has a mid part of 0.8 to 1 times 2^-8 and a rest part of 2^-17, with the signs asked for.
    m = 4j + 1 rounds down to 8 bits (rest +), 4j + 3 rounds up (rest -); 1024 - m gives hi = 1 + 2^-7 and a negative mid."""
    j = rng.integers(100, 127, size=shape)
    pos_mid, plus_rest = mid_sign > 0, rest_sign > 0
    m = np.where(pos_mid, np.where(plus_rest, 4 * j + 1, 4 * j + 3), 1024 - np.where(plus_rest, 4 * j + 3, 4 * j + 1))
    return 1.0 + m * 2.0 ** -17


def worst_case_pairs(dim, pairs, per_pair, rng, shared_mid_signs, mirrored=False):
    """Near-ties on which every product the split drops has one sign for one centroid and the other sign for its rival.
    All centroids of even index agree in sign with the points on half of the coordinates, those of odd index on the other
    half, so a point is about equally far from both kinds; the signs of the mid and rest parts are chosen per coordinate
    so that, for the even kind, c'mid xmid, c'hi xrest and c'rest xhi are all positive, and all negative for the odd kind.
    The ranking values of the two kinds then move apart by twice the worst case of the dropped products (2 * 2^-15 S for
    three products, 2 * 2^-16 S for the packed form) while the true gaps straddle zero."""
    sx = rng.choice([-1.0, 1.0], size=(1, dim))
    match = np.ones((1, dim))
    match[0, rng.permutation(dim)[: dim // 2]] = -1           # +1: the point has the sign of the even kind there
    mid_sign = rng.choice([-1.0, 1.0], size=(1, dim) if shared_mid_signs else (pairs, dim)) * np.ones((pairs, dim))
    c = np.empty((2 * pairs, dim))
    c[0::2] = sx * match * worst_parts(rng, (pairs, dim), match * mid_sign, match * np.ones((pairs, dim)))
    c[1::2] = -sx * match * worst_parts(rng, (pairs, dim), match * mid_sign, match * np.ones((pairs, dim)))
    if mirrored:   # the odd kind the exact negatives of the even kind: every product changes sign, and the centroids' mean is 0
        c[1::2] = -c[0::2]
    pid = np.repeat(np.arange(pairs), per_pair)
    x = sx * worst_parts(rng, (pairs * per_pair, dim), mid_sign[pid], match * np.ones((pairs * per_pair, dim)))
    return x.astype(np.float32), c.astype(np.float32)


# (dim, pairs, shared_mid_signs): shapes at which the inputs defeat a certificate derived for 9-bit parts
WORST_CASE_SHAPES = [(2, 32, False), (3, 32, False), (4, 32, False), (8, 4, True), (16, 2, True), (32, 1, True), (64, 1, True)]


def worst_case_inputs(dim, n=64000, mirrored=False, pairs=None):
    default_pairs, shared = next((p, s) for d, p, s in WORST_CASE_SHAPES if d == dim)
    pairs = pairs or default_pairs
    return worst_case_pairs(dim, pairs, n // pairs, np.random.default_rng(dim), shared, mirrored)


def near_ties(dim, n, k, rng, offset, centroids=None):
    """Points close to the bisector of two centroids, true gap log-uniform over six decades, coordinates shifted by offset."""
    c = centroids if centroids is not None else rng.normal(size=(k, dim)).astype(np.float32) * np.float32(3) + np.float32(offset)
    a, b = rng.integers(0, k, size=n), rng.integers(0, k, size=n)
    b = np.where(a == b, (b + 1) % k, b)
    ca, cb = c[a].astype(np.float64), c[b].astype(np.float64)
    gap = 10.0 ** rng.uniform(-9, -3, size=n) * rng.choice([-1.0, 1.0], size=n)
    s = (ca ** 2).sum(1) + (cb ** 2).sum(1)
    direction = cb - ca
    length = np.maximum(np.sqrt((direction ** 2).sum(1)), 1e-30)
    t = gap * s / (2 * length)
    x = (ca + cb) / 2 + direction / length[:, None] * t[:, None]
    return x.astype(np.float32), c


def emulate(x, c, packed):
    """The ranking values of the sweep without accumulation error, the exact ones, and the norms the certificate uses."""
    xh, xm, xr = (p.astype(np.float64) for p in split(x))
    cp = (np.float32(-2) * c).astype(np.float32)
    ch, cm, cr = (p.astype(np.float64) for p in split(cp))
    c2 = (c.astype(np.float32) ** 2).sum(1, dtype=np.float32).astype(np.float64)          # the packing kernel's fp32 norm
    kept = ch @ xh.T + ch @ xm.T + cm @ xh.T
    if packed:
        kept = kept + cm @ xm.T
    a = c2[:, None] + kept                                                                  # [k, n]
    exact = (c.astype(np.float64) ** 2).sum(1)[:, None] + cp.astype(np.float64) @ x.astype(np.float64).T
    norms = dict(x2=(x.astype(np.float32) ** 2).sum(1, dtype=np.float32), xmid2=(xm ** 2).sum(1), xrest2=(xr ** 2).sum(1),
                 c2max=float(c2.max()), cmid2max=float((cm ** 2).sum(1).max()), crest2max=float((cr ** 2).sum(1).max()))
    return a, exact, norms


def serial_distances(x, c):
    """sqrt(sum (x - c)^2) with every operation rounded to fp32 in ascending dimension (metric_policies.hpp:23-28,40-44)."""
    n, dim = x.shape
    out = np.zeros((c.shape[0], n), np.float32)
    for j in range(c.shape[0]):
        s = np.zeros(n, np.float32)
        for q in range(dim):
            diff = (x[:, q] - c[j, q]).astype(np.float32)
            s = (s + (diff * diff).astype(np.float32)).astype(np.float32)
        out[j] = np.sqrt(s, dtype=np.float32)
    return out


CASES = [(2, True), (3, True), (4, True), (2, False), (4, False), (8, False), (16, False), (32, False), (64, False), (256, False)]


@pytest.mark.parametrize("dim,packed", CASES)
@pytest.mark.parametrize("kind", ["adversarial", "pairs", "ties0", "ties100", "ties10000"])
def test_tau_covers_the_split_and_the_serial_margin(km, dim, packed, kind):
    rng = np.random.default_rng(dim * 31 + packed)
    n, k = (4096, 16) if dim <= 64 else (1024, 8)
    if kind == "adversarial":
        x, c = adversarial(dim, n, k, rng)
    elif kind == "pairs":
        if dim > 64:
            pytest.skip("the construction is used up to 64 dimensions")
        x, c = worst_case_inputs(dim, 8192)
        n = x.shape[0]
    else:
        x, c = near_ties(dim, n, k, rng, float(kind[4:]))
    a, exact, nm = emulate(x, c, packed)
    form = 2 if packed else 1
    xpart = nm["xrest2"] if packed else nm["xmid2"]
    tau = np.array([km.certificate_tau(form, dim, float(nm["x2"][i]), float(xpart[i]), nm["c2max"], nm["cmid2max"], nm["crest2max"])
                    for i in range(n)], np.float64)
    s_all = nm["x2"].astype(np.float64) + nm["c2max"]
    products = 4 * dim if packed else 3 * dim
    accumulation = (products + 2) * U * 2 * s_all          # allowance for the fp32 accumulation in the matrix core
    margin = (2 * dim + 12) * U * s_all                    # two serial sums and the sqrt collision
    dropped = np.abs(a - exact).max(0)
    assert np.all(2 * dropped + 2 * accumulation + margin <= tau), \
        "tau misses %d of %d points (worst ratio %.3f)" % (int((2 * dropped + 2 * accumulation + margin > tau).sum()), n,
                                                          float(((2 * dropped + 2 * accumulation + margin) / tau).max()))
    # decisions: a pair (winner j1, other j2) that could be certified under the full accumulation allowance must be a strict serial win
    dist = serial_distances(x, c)
    j1 = a.argmin(0)
    certified = (a - a[j1, np.arange(n)][None, :]) + 2 * accumulation[None, :] > tau[None, :]
    certified[j1, np.arange(n)] = False
    wrong = certified & ~(dist[j1, np.arange(n)][None, :] < dist)
    assert not wrong.any(), "%d certified pairs contradict the serial comparison" % int(wrong.sum())


@pytest.mark.parametrize("dim", [17, 20, 32])
@pytest.mark.parametrize("kind", ["adversarial", "pairs", "ties0", "ties100", "ties10000"])
def test_tau_of_the_first_level_covers_one_product_per_dimension(km, dim, kind):
    """The first level of the two-level sweep keeps hi * hi only: a1[j] = |c_j|^2 + sum_i c'hi_i xhi_i. Its tau (form 4, with
    sum_i (x_i - xhi_i)^2 of the point) must cover twice what that drops plus the accumulation allowance of d products
    plus the serial margin, and every pair it would certify must be a strict win of the serial comparison."""
    rng = np.random.default_rng(dim * 17)
    n, k = 4096, 16
    if kind == "adversarial":
        x, c = adversarial(dim, n, k, rng)
    elif kind == "pairs":
        if dim != 32:
            pytest.skip("the construction exists for 32 dimensions")
        x, c = worst_case_inputs(dim, 8192)
        n = x.shape[0]
    else:
        x, c = near_ties(dim, n, k, rng, float(kind[4:]))
    xh = split(x)[0]
    cp = (np.float32(-2) * c).astype(np.float32)
    ch, cm, cr = (p.astype(np.float64) for p in split(cp))
    c2 = (c.astype(np.float32) ** 2).sum(1, dtype=np.float32).astype(np.float64)
    a1 = c2[:, None] + ch @ xh.astype(np.float64).T
    exact = (c.astype(np.float64) ** 2).sum(1)[:, None] + cp.astype(np.float64) @ x.astype(np.float64).T
    xlo = (x - xh).astype(np.float32)                                   # exact in fp32, as in the kernel
    x2 = (x.astype(np.float32) ** 2).sum(1, dtype=np.float32)
    xlo2 = (xlo ** 2).sum(1, dtype=np.float32)
    c2max, cmid2max, crest2max = float(c2.max()), float((cm ** 2).sum(1).max()), float((cr ** 2).sum(1).max())
    tau = np.array([km.certificate_tau(4, dim, float(x2[i]), float(xlo2[i]), c2max, cmid2max, crest2max) for i in range(n)], np.float64)
    s_all = x2.astype(np.float64) + c2max
    accumulation = (dim + 2) * U * 2 * s_all
    margin = (2 * dim + 12) * U * s_all
    dropped = np.abs(a1 - exact).max(0)
    need = 2 * dropped + 2 * accumulation + margin
    assert np.all(need <= tau), "tau misses %d of %d points (worst ratio %.3f)" % (int((need > tau).sum()), n, float((need / tau).max()))
    # the bound is not slack by orders of magnitude either: on the adversarial mantissas it is within 8x of what is dropped
    if kind == "adversarial":
        assert float((tau / np.maximum(need, 1e-30)).min()) < 8.0
    dist = serial_distances(x, c)
    j1 = a1.argmin(0)
    certified = (a1 - a1[j1, np.arange(n)][None, :]) + 2 * accumulation[None, :] > tau[None, :]
    certified[j1, np.arange(n)] = False
    wrong = certified & ~(dist[j1, np.arange(n)][None, :] < dist)
    assert not wrong.any(), "%d certified pairs contradict the serial comparison" % int(wrong.sum())


@pytest.mark.parametrize("dim", [2, 4, 8, 16, 32, 64])
@pytest.mark.parametrize("kind", ["adversarial", "ties0", "ties100", "ties10000"])
def test_tau_of_the_vector_alu_sweeps_covers_a_chain_of_fused_multiply_adds(km, dim, kind):
    """KMX_ASSIGN_LDS_FMA and the single-pass fused kernel rank by a[j] = fma(c'_d, x_d, ... fma(c'_1, x_1, |c_j|^2)) in fp32,
    round to nearest (form 3 of kmx_certificate_tau: (4 d + 24) u' S). The chain is emulated with exact products and one
    rounding per step; twice its distance from the exact value plus the serial margin stays below tau, and what tau
    certifies is a strict serial win."""
    rng = np.random.default_rng(dim * 13 + len(kind))
    n, k = 4096, 16
    x, c = adversarial(dim, n, k, rng) if kind == "adversarial" else near_ties(dim, n, k, rng, float(kind[4:]))
    cp = (np.float32(-2) * c).astype(np.float32)
    c2 = np.zeros(k, np.float32)
    for q in range(dim):
        c2 = (c2 + (c[:, q] * c[:, q]).astype(np.float32)).astype(np.float32)      # any fp32 sum of the squares: at most d roundings
    a = np.repeat(c2[:, None], n, 1)
    for q in range(dim):
        a = (cp[:, q].astype(np.float64)[:, None] * x[:, q].astype(np.float64)[None, :] + a.astype(np.float64)).astype(np.float32)
    exact = (c.astype(np.float64) ** 2).sum(1)[:, None] + cp.astype(np.float64) @ x.astype(np.float64).T
    x2 = (x.astype(np.float32) ** 2).sum(1, dtype=np.float32)
    c2max = float(c2.max())
    tau = np.array([km.certificate_tau(3, dim, float(x2[i]), 0.0, c2max, 0.0, 0.0) for i in range(n)], np.float64)
    assert tau[0] == pytest.approx((4 * dim + 24) * U * (float(x2[0]) + c2max), rel=1e-6)
    s_all = x2.astype(np.float64) + c2max
    margin = (2 * dim + 12) * U * s_all
    off = np.abs(a.astype(np.float64) - exact).max(0)
    assert np.all(off <= (2 * dim + 7) * (U / 2) * s_all)          # the bound of the chain itself
    assert np.all(2 * off + margin <= tau)
    dist = serial_distances(x, c)
    j1 = a.argmin(0)
    certified = (a.astype(np.float64) - a[j1, np.arange(n)].astype(np.float64)[None, :]) > tau[None, :]
    certified[j1, np.arange(n)] = False
    wrong = certified & ~(dist[j1, np.arange(n)][None, :] < dist)
    assert not wrong.any(), "%d certified pairs contradict the serial comparison" % int(wrong.sum())


@pytest.mark.parametrize("dim", [4, 16, 32])
@pytest.mark.parametrize("k", [16, 32])
@pytest.mark.parametrize("kind", ["adversarial", "ties0", "ties100"])
def test_tau_of_the_single_pass_kernels_pays_for_the_centroid_number_in_the_low_bits(km, dim, k, kind):
    """The single-pass iteration kernels replace the lowest 4 (k <= 16) or 5 bits of every ranking value by the centroid's
    number and track minima of the result (forms 5 and 6 of kmx_certificate_tau). The chain is emulated as for form 3, the
    bits are replaced as the kernels do, and twice the distance of the keyed values from the exact ones plus the serial
    margin must stay below tau; what tau certifies on the keyed values is a strict serial win, and the centroid read back
    from the low bits of the minimum is the centroid of that value."""
    bits = 4 if k <= 16 else 5
    rng = np.random.default_rng(dim * 19 + k + len(kind))
    n = 4096
    x, c = adversarial(dim, n, k, rng) if kind == "adversarial" else near_ties(dim, n, k, rng, float(kind[4:]))
    cp = (np.float32(-2) * c).astype(np.float32)
    c2 = np.zeros(k, np.float32)
    for q in range(dim):
        c2 = (c2 + (c[:, q] * c[:, q]).astype(np.float32)).astype(np.float32)
    a = np.repeat(c2[:, None], n, 1)
    for q in range(dim):
        a = (cp[:, q].astype(np.float64)[:, None] * x[:, q].astype(np.float64)[None, :] + a.astype(np.float64)).astype(np.float32)
    mask = np.uint32((1 << bits) - 1)
    keyed = ((a.view(np.uint32) & ~mask) | np.arange(k, dtype=np.uint32)[:, None]).view(np.float32)
    exact = (c.astype(np.float64) ** 2).sum(1)[:, None] + cp.astype(np.float64) @ x.astype(np.float64).T
    x2 = (x.astype(np.float32) ** 2).sum(1, dtype=np.float32)
    c2max = float(c2.max())
    s_all = x2.astype(np.float64) + c2max
    tau5 = np.array([km.certificate_tau(5, dim, float(x2[i]), float(bits), c2max, 0.0, 0.0) for i in range(n)], np.float64)
    tau6 = np.array([km.certificate_tau(6, dim, float(x2[i]), float(bits), c2max, 0.0, 0.0) for i in range(n)], np.float64)
    tau3 = np.array([km.certificate_tau(3, dim, float(x2[i]), 0.0, c2max, 0.0, 0.0) for i in range(n)], np.float64)
    assert np.all(tau6 >= tau5) and np.all(tau5 > tau3)
    assert tau5[0] == pytest.approx(tau3[0] + 4.125 * (1 << bits) * U * s_all[0], rel=1e-5)
    moved = np.abs(keyed.astype(np.float64) - a.astype(np.float64))
    assert np.all(moved.max(0) <= 2.0625 * (1 << bits) * U * s_all)            # one value's share of the allowance
    assert moved.max() > 0.25 * (1 << bits) * U * np.abs(a).max() * 0.5            # and the bits do move the values
    margin = (2 * dim + 12) * U * s_all
    off = np.abs(keyed.astype(np.float64) - exact).max(0)
    assert np.all(2 * off + margin <= tau5)
    dist = serial_distances(x, c)
    j1 = keyed.argmin(0)
    assert np.array_equal(keyed[j1, np.arange(n)].view(np.uint32) & mask, j1.astype(np.uint32))
    certified = (keyed.astype(np.float64) - keyed[j1, np.arange(n)].astype(np.float64)[None, :]) > tau5[None, :]
    certified[j1, np.arange(n)] = False
    wrong = certified & ~(dist[j1, np.arange(n)][None, :] < dist)
    assert not wrong.any(), "%d certified pairs contradict the serial comparison" % int(wrong.sum())
    if dim == 4 and kind == "adversarial":
        # teeth: with few dimensions the replaced bits take the values out of the bound of the chain itself
        assert np.any(off > (2 * dim + 7) * (U / 2) * s_all)
    with pytest.raises(Exception):
        km.certificate_tau(5, dim, 1.0, 3.0, 1.0, 0.0, 0.0)


@pytest.mark.parametrize("dim", [2, 3, 4])
@pytest.mark.parametrize("kind", ["ties0", "ties100", "ties10000", "uniform", "mirrored pairs"])
def test_tau_in_a_moved_frame_covers_the_distances_of_the_data(km, dim, kind):
    """Packed rows are swept as fl(x - m), fl(c - m) with m near the middle of the centroids. The ranking values of that
    frame, against the exact ones of the unrounded differences (distances do not depend on the frame): the frame's tau,
    from the frame's norms, covers what the split drops and the two roundings; what it certifies is a strict serial win on
    the data as given."""
    rng = np.random.default_rng(dim * 17 + len(kind))
    n, k = 4096, 160
    if kind == "uniform":
        x, c = rng.random((n, dim)).astype(np.float32), rng.random((k, dim)).astype(np.float32)
    elif kind == "mirrored pairs":
        x, c = worst_case_inputs(dim, 8192, mirrored=True, pairs=80)
        n = x.shape[0]
    else:
        x, c = near_ties(dim, n, k, rng, float(kind[4:]))
    m = (c.sum(0, dtype=np.float32) / np.float32(c.shape[0])).astype(np.float32)
    if kind == "mirrored pairs":
        assert not m.any()
    xs, cs = (x - m).astype(np.float32), (c - m).astype(np.float32)
    a, _, nm = emulate(xs, cs, True)
    xd, cd = x.astype(np.float64) - m.astype(np.float64), c.astype(np.float64) - m.astype(np.float64)
    exact = (cd ** 2).sum(1)[:, None] - 2 * cd @ xd.T
    tau = np.array([km.certificate_tau(2, dim, float(nm["x2"][i]), float(nm["xrest2"][i]), nm["c2max"], nm["cmid2max"], nm["crest2max"])
                    for i in range(n)], np.float64)
    s_all = nm["x2"].astype(np.float64) + nm["c2max"]
    accumulation = (4 * dim + 2) * U * 2 * s_all
    margin = (2 * dim + 12) * U * s_all
    off = np.abs(a - exact).max(0)
    assert np.all(2 * off + 2 * accumulation + margin <= tau), "worst ratio %.3f" % float(((2 * off + 2 * accumulation + margin) / tau).max())
    dist = serial_distances(x, c)
    j1 = a.argmin(0)
    certified = (a - a[j1, np.arange(n)][None, :]) + 2 * accumulation[None, :] > tau[None, :]
    certified[j1, np.arange(n)] = False
    wrong = certified & ~(dist[j1, np.arange(n)][None, :] < dist)
    assert not wrong.any(), "%d certified pairs contradict the serial comparison" % int(wrong.sum())
    if kind in ("ties100", "ties10000"):   # the point of the frame: tau follows the spread of the data, not its distance from the origin
        _, _, nm0 = emulate(x, c, True)
        tau0 = np.array([km.certificate_tau(2, dim, float(nm0["x2"][i]), float(nm0["xrest2"][i]), nm0["c2max"], nm0["cmid2max"],
                                            nm0["crest2max"]) for i in range(n)])
        assert np.median(tau) < np.median(tau0) / 50   # (the points with the largest gaps lie far from the centroids in any frame)


@pytest.mark.parametrize("dim,packed,old_units", [(2, True, 18 * 2 + 149), (8, False, 14 * 8 + 224), (16, False, 14 * 16 + 224)])
def test_the_worst_case_inputs_defeat_a_bound_that_assumes_nine_bit_parts(dim, packed, old_units):
    """The inputs have teeth: a bound derived from |mid| <= 2^-9 |v|, |rest| <= 2^-18 |v| (one bit too optimistic for a
    bf16) does not cover what the split drops on them."""
    rng = np.random.default_rng(5)
    x, c = adversarial(dim, 8192, 16, rng)
    a, exact, nm = emulate(x, c, packed)
    s_all = nm["x2"].astype(np.float64) + nm["c2max"]
    products = 4 * dim if packed else 3 * dim
    needed = 2 * np.abs(a - exact).max(0) + 2 * (products + 2) * U * 2 * s_all + (2 * dim + 12) * U * s_all
    assert (needed > old_units * U * s_all).any()


def decisions(x, c, packed, tau):
    """(points the ranking would decide, decided points whose serial result is another centroid)"""
    a, _, _ = emulate(x, c, packed)
    n = x.shape[0]
    order = np.argsort(a, 0, kind="stable")
    j1, j2 = order[0], order[1]
    gap = a[j2, np.arange(n)] - a[j1, np.arange(n)]
    serial = serial_distances(x, c).argmin(0)              # the first minimum: the serial scan's tie-break
    decided = gap > tau
    return int(decided.sum()), int((decided & (serial != j1)).sum())


@pytest.mark.parametrize("dim,packed,old_units", [(2, True, 18 * 2 + 149), (4, True, 18 * 4 + 149), (8, False, 14 * 8 + 224),
                                                  (16, False, 14 * 16 + 224)])
def test_worst_case_pairs_are_decided_wrongly_by_the_nine_bit_bound_and_never_by_tau(km, dim, packed, old_units):
    """The inputs of the GPU regression test (tests/test_gpu_certificate.py): even without any accumulation error a
    certificate of (14 d + 224) u' S, or (18 d + 149) u' S for packed rows, decides some of them against the serial scan;
    the library's tau decides none wrongly."""
    x, c = worst_case_inputs(dim, 64000)
    _, _, nm = emulate(x, c, packed)
    s_all = nm["x2"].astype(np.float64) + nm["c2max"]
    _, wrong_old = decisions(x, c, packed, old_units * U * s_all)
    assert wrong_old > 0
    xpart = nm["xrest2"] if packed else nm["xmid2"]
    tau = np.array([km.certificate_tau(2 if packed else 1, dim, float(nm["x2"][i]), float(xpart[i]), nm["c2max"], nm["cmid2max"],
                                       nm["crest2max"]) for i in range(x.shape[0])])
    decided, wrong = decisions(x, c, packed, tau)
    assert wrong == 0


def test_fp32_form_and_argument_errors(km):
    assert km.certificate_tau(0, 32, 3.0, 0.0, 5.0, 0.0, 0.0) == pytest.approx((8 * 32 + 24) * U * 8.0, rel=1e-6)
    with pytest.raises(km.KmxError):
        km.certificate_tau(7, 32, 1.0, 1.0, 1.0, 1.0, 1.0)
    assert not np.isfinite(km.certificate_tau(1, 8, float("inf"), 1.0, 1.0, 1.0, 1.0))
    assert np.isnan(km.certificate_tau(1, 8, float("nan"), 1.0, 1.0, 1.0, 1.0))


@pytest.mark.parametrize("dim", [5, 16, 32, 100, 256])
@pytest.mark.parametrize("offset", [0.0, 50.0, 3000.0, -1.0e5])
def test_threshold_taken_back_to_the_frame_of_the_data(km, dim, offset):
    """kmx_certificate_unmoved_threshold. A sweep in the frame moved by m knows its best moved ranking value
    A'_j = |c_j - m|^2 - 2 (c_j - m).(x - m); the kernels of the exact pass evaluate a_r[j] = fma(-2, chain of fused
    multiply-adds over x . c_j, |c_j|^2) on the data as given, in fp32. Here everything the kernels compute in fp32
    is emulated in fp32, in their order (x - m and its projection on m, |m|^2, the chain), and the exact values in
    float64. With first = the exact A'_j of a centroid and tau = 0 the threshold must not fall below that centroid's
    own a_r[j] (it would be dropped although it attains `first`), nor exceed it by more than twice the allowance."""
    rng = np.random.default_rng(dim + int(abs(offset)))
    n, k = 200, 32
    c = (rng.uniform(-10, 10, (k, dim)) + offset).astype(np.float32)
    x = (c[rng.integers(0, k, n)] + rng.normal(size=(n, dim)) * (1 + rng.integers(0, 2, (n, 1)) * 20)).astype(np.float32)
    m = c[:16].mean(axis=0).astype(np.float32)
    xs = (x - m).astype(np.float32)                      # what the sweep splits
    cs = (c - m).astype(np.float32)
    def chain32(a, b, start=np.float32(0)):
        acc = np.full(a.shape[:-1], start, np.float32)
        for i in range(a.shape[-1]):                     # one rounding per fused multiply-add
            acc = (acc.astype(np.float64) + a[..., i].astype(np.float64) * b[..., i].astype(np.float64)).astype(np.float32)
        return acc
    x2 = chain32(xs, xs)
    along = chain32(xs, np.broadcast_to(m, xs.shape))
    m2 = chain32(m[None, :], m[None, :])[0]
    mnorm = np.float32(np.sqrt(np.float64(m2)) * 1.0001)
    c2max = np.float32((cs.astype(np.float64) ** 2).sum(axis=1).max() * (1 + 1e-6))
    x64, c64, m64 = x.astype(np.float64), c.astype(np.float64), m.astype(np.float64)
    S = (x64 ** 2).sum(axis=1) + (c64 ** 2).sum(axis=1).max()
    worst_low, worst_high = np.inf, 0.0
    for j in range(k):
        moved = ((c64[j] - m64) ** 2).sum() - 2.0 * ((x64 - m64) * (c64[j] - m64)).sum(axis=1)          # A'_j, exact
        c2 = chain32(c[j][None, :], c[j][None, :])[0]
        a_r = (np.float64(c2) - 2.0 * chain32(x, np.broadcast_to(c[j], x.shape)).astype(np.float64)).astype(np.float32)
        thr = np.array([km.certificate_unmoved_threshold(dim, float(np.float32(moved[i])), 0.0, float(x2[i]), float(along[i]),
                                                         float(c2max), float(m2), float(mnorm)) for i in range(n)])
        gap = thr - a_r.astype(np.float64)
        worst_low = min(worst_low, float((gap / S).min()))
        worst_high = max(worst_high, float((gap / S).max()))
    allowance = (4 * dim + 40) * U
    assert worst_low >= 0.0, "threshold below the centroid's own value by %.3g S" % -worst_low
    # Q, the bound of |x|^2 + max |c|^2 that the threshold uses, exceeds S by at most the triangle inequality's factor of 4
    assert worst_high <= 4.0 * 2.0 * allowance, "threshold %.3g S above the value: more than twice the allowance" % worst_high


# ---------------------------------------------------------------- the accumulation inside the matrix cores
#
# The certificates allow one u' = 2^-23 of the running magnitude per accumulated product "for any rounding or truncation
# inside the matrix core" (csrc/certificate.h). The running magnitude is bounded by M = |c| + sum_q |a_q b_q| (which
# |c_j|^2 + 2 |c_j||x| of the derivation bounds in turn, by Cauchy-Schwarz), so the assumption reads
#       |d - (c + sum_q a_q b_q)|  <=  steps * u' * M        for a chain of `steps` products.
# The operand sets below are chosen so that an accumulator that merely truncates after every product -- the worst the
# assumption admits -- uses most of that allowance: they fail a bound of half a u' per step under that model (shown here, on
# the CPU), and tests/test_gpu_certificate.py holds the hardware's own results on the same operands to the full bound.

def accumulation_cases(kind):
    """Operand sets for kmx_probe_matrix_chain: name -> (a[32, depth], b[32, depth], c[32, 32]) in float32.
    kind 1: a and b hold bf16 values (products exact in fp32); kinds 0 and 2: full fp32 mantissas."""
    rng = np.random.default_rng(1234 + kind)
    block = {0: 2, 1: 16, 2: 4}[kind]
    quant = bf16_round if kind == 1 else (lambda v: np.asarray(v, np.float32))
    cases = {}

    def mant(shape):   # mantissas in [1, 2) with all their bits in use
        return 1.0 + rng.integers(0, 1 << 23, size=shape) * 2.0 ** -23

    for blocks in (1, 3, 12, 48):
        depth = blocks * block
        # products of very different exponents inside one block: 2^0 ... 2^-20
        ea, eb = rng.integers(0, 11, size=(32, depth)), rng.integers(0, 11, size=(32, depth))
        a = quant(mant((32, depth)) * 2.0 ** -ea * rng.choice([-1.0, 1.0], size=(32, depth)))
        b = quant(mant((32, depth)) * 2.0 ** -eb * rng.choice([-1.0, 1.0], size=(32, depth)))
        cases["wide_exponents_%d" % blocks] = (a, b, (rng.normal(size=(32, 32)) * 0.5).astype(np.float32))
        # cancelling pairs next to a small term: +A, -A, +eps, ... ; the accumulator starts small as well
        a = quant(mant((32, depth)))
        b = quant(mant((32, depth)))
        a[:, 1::2] = -a[:, 0::2][:, : a[:, 1::2].shape[1]]
        b[:, 1::2] = b[:, 0::2][:, : b[:, 1::2].shape[1]]
        last = depth - 1 if depth % 2 else depth - 2
        a[:, last:] = quant(mant((32, depth - last)) * 2.0 ** -20)        # the terms that must survive the cancellation
        b[:, last:] = quant(mant((32, depth - last)))
        cases["cancelling_pairs_%d" % blocks] = (a, b, (rng.normal(size=(32, 32)) * 2.0 ** -18).astype(np.float32))
        # a large accumulator and products just below its unit in the last place, all of one sign: what truncation loses most of
        c = ((1.0 + rng.integers(0, 1 << 22, size=(32, 32)) * 2.0 ** -23) * 1024.0).astype(np.float32)   # ulp(c) = 2^-13
        a = quant((1.0 + rng.integers(0, 4, size=(32, depth)) * 2.0 ** -7) * 2.0 ** -7)
        b = quant(np.full((32, depth), 0.96875 * 2.0 ** -6))             # a_q b_q in (0.96, 0.995) ulp(c)
        cases["small_addends_%d" % blocks] = (a, b, c)
    return cases


def exact_chain(a, b, c):
    """c + a b^T in float64 (every product of two fp32 values is exact there) and M = |c| + sum_q |a_q b_q|."""
    a64, b64, c64 = a.astype(np.float64), b.astype(np.float64), c.astype(np.float64)
    return c64 + a64 @ b64.T, np.abs(c64) + np.abs(a64) @ np.abs(b64).T


def chopped_chain(a, b, c):
    """The worst accumulator the assumption admits: fp32, one product at a time, every sum truncated towards zero."""
    s = c.astype(np.float32).copy()
    for q in range(a.shape[1]):
        v = s.astype(np.float64) + np.outer(a[:, q].astype(np.float64), b[:, q].astype(np.float64))
        r = v.astype(np.float32)
        over = np.abs(r.astype(np.float64)) > np.abs(v)
        r[over] = np.nextafter(r[over], np.float32(0))
        s = r
    return s


@pytest.mark.parametrize("kind", [0, 1, 2])
def test_accumulation_cases_use_the_allowance_of_one_unit_per_step(kind):
    """A truncating accumulator stays within steps * u' * M on every operand set and exceeds half of that on some:
    the operands have teeth against a bound of half a u' per step."""
    beyond_half = 0
    for name, (a, b, c) in accumulation_cases(kind).items():
        exact, m = exact_chain(a, b, c)
        err = np.abs(chopped_chain(a, b, c).astype(np.float64) - exact)
        steps = a.shape[1]
        assert np.all(err <= steps * U * m), name
        beyond_half += int((err > 0.5 * steps * U * m).sum())
    assert beyond_half > 1000, "only %d results of the truncating model exceed half a unit per step" % beyond_half
