"""A seeded walk over shapes, layouts and kinds of data that no hand-picked list covers: every assignment variant against the
serial oracle (bit for bit) and the tuned update against float64 means of the same assignment, through the C ABI (-m gpu)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

DIMS = [1, 2, 3, 4, 5, 7, 8, 12, 16, 20, 24, 31, 32, 33, 40, 48, 64, 65, 100, 128, 200, 256]
KS = [1, 2, 5, 16, 31, 64, 100, 128, 200, 256, 320, 512, 700, 1024, 1500, 2048, 4096]
NS = [1, 63, 1000, 4097, 20000, 65536]


def flat(rows, layout):
    return np.ascontiguousarray(rows if layout == 0 else rows.T).ravel()


@pytest.mark.parametrize("seed", [11, 12, 13, 14])
def test_random_shapes_match_the_oracle(km, orc, gpu, seed):
    rng = np.random.default_rng(seed)
    for case in range(12):
        dim, k, n = int(rng.choice(DIMS)), int(rng.choice(KS)), int(rng.choice(NS))
        if dim * k > 300000:
            k = max(1, 300000 // dim)
        if n * k * dim > 2e9:
            n = max(1, int(2e9 // (k * dim)))
        layout, layout_means = int(rng.integers(0, 2)), int(rng.integers(0, 2))
        kind = str(rng.choice(["gauss", "offset", "grid", "clustered"]))
        rows = rng.normal(size=(n, dim)).astype(np.float32)
        if kind == "offset":
            rows = (rows + np.float32(rng.choice([10, 1000, 30000]))).astype(np.float32)
        elif kind == "grid":
            rows = (np.round(rows * 2) / 2).astype(np.float32)
        elif kind == "clustered":
            centres = rng.uniform(-10, 10, size=(max(1, k // 2), dim)).astype(np.float32)
            rows = (centres[rng.integers(0, centres.shape[0], n)] + rows * np.float32(0.5)).astype(np.float32)
        means = rows[rng.integers(0, n, k)].copy() if rng.random() < 0.7 else rng.normal(size=(k, dim)).astype(np.float32)
        what = "seed %d case %d: dim %d, k %d, n %d, layouts %d/%d, %s" % (seed, case, dim, k, n, layout, layout_means, kind)
        want = orc.assign(flat(rows, 0), flat(means, 0), dim, k, n, threads=0, fast=True)
        d = km.DeviceBuffer(4 * n * dim); d.write(flat(rows, layout))
        m = km.DeviceBuffer(4 * k * dim); m.write(flat(means, layout_means))
        a = km.DeviceBuffer(4 * n)
        stride, stride_means = km.layout_stride(layout, n, dim), km.layout_stride(layout_means, k, dim)
        variants = [km.ASSIGN_BEST, km.ASSIGN_MFMA_BF16X3, km.ASSIGN_MFMA] + ([km.ASSIGN_LDS_FMA] if dim <= 64 else [])
        for v in variants:
            km.assign(v, d, layout, stride, m, layout_means, stride_means, a, dim, k, n)
            km.sync()
            got = a.read(np.uint32, n)
            assert np.array_equal(got, want), "%s, variant %d: %d mismatches" % (what, v, int((got != want).sum()))
        out = km.DeviceBuffer(4 * k * dim); sizes = km.DeviceBuffer(4 * k)
        a.write(want)
        km.update(km.UPDATE_ATOMIC_SHM, d, layout, stride, a, out, layout_means, stride_means, sizes, dim, k, n)
        km.sync()
        gm = out.read(np.float32, k * dim)
        gm = gm.reshape(k, dim) if layout_means == 0 else gm.reshape(dim, k).T
        counts = np.bincount(want, minlength=k)
        assert np.array_equal(sizes.read(np.uint32, k), counts), what
        sums = np.zeros((k, dim)); np.add.at(sums, want, rows.astype(np.float64))
        truth = np.where(counts[:, None] > 0, sums / np.maximum(counts, 1)[:, None], 0.0)
        scale = max(float(np.sqrt(np.mean(truth ** 2))), 1e-30)
        assert float(np.abs(gm - truth).max()) / scale < 1e-4, what
        for b in (d, m, a, out, sizes):
            b.free()


@pytest.mark.parametrize("seed", [21, 22, 23])
def test_random_shapes_of_the_single_pass_iteration(km, orc, gpu, seed):
    """kmx_iteration_f32 where it reads the points once (k <= 32, dim <= 32): both kernels behind it (rows of 8, 16, 32 floats
    rank on the matrix cores, the other widths lane per point), every layout, rows with padding between them (16-byte pieces
    or single words, by the stride), point counts around the batch of 256: the serial scan's assignment bit for bit, exact
    counts, centroids against float64 means of that assignment."""
    rng = np.random.default_rng(seed)
    for case in range(16):
        dim, k = int(rng.integers(1, 33)), int(rng.integers(1, 33))
        n = int(rng.choice([1, 63, 255, 256, 257, 1000, 4097, 70001]))
        layout, layout_means = int(rng.integers(0, 2)), int(rng.integers(0, 2))
        pad = int(rng.choice([0, 0, 1, 4])) if layout == 0 else int(rng.choice([0, 0, 3]))
        kind = str(rng.choice(["gauss", "offset", "grid", "clustered"]))
        rows = rng.normal(size=(n, dim)).astype(np.float32)
        if kind == "offset":
            rows = (rows + np.float32(rng.choice([10, 1000, 30000]))).astype(np.float32)
        elif kind == "grid":
            rows = (np.round(rows * 2) / 2).astype(np.float32)
        elif kind == "clustered":
            centres = rng.uniform(-10, 10, size=(max(1, k // 2), dim)).astype(np.float32)
            rows = (centres[rng.integers(0, centres.shape[0], n)] + rows * np.float32(0.5)).astype(np.float32)
        means = rows[rng.integers(0, n, k)].copy() if rng.random() < 0.7 else rng.normal(size=(k, dim)).astype(np.float32)
        what = "seed %d case %d: dim %d, k %d, n %d, layouts %d/%d, padding %d, %s" % (seed, case, dim, k, n, layout, layout_means, pad, kind)
        want = orc.assign(flat(rows, 0), flat(means, 0), dim, k, n, threads=0, fast=True)
        if layout == 0:    # AoS: `pad` words of leftovers behind every row
            stride = dim + pad
            padded = np.full((n, stride), np.float32(np.nan)); padded[:, :dim] = rows
        else:              # SoA: `pad` words of leftovers behind every coordinate's run of n values
            stride = n + pad
            padded = np.full((dim, stride), np.float32(np.nan)); padded[:, :n] = rows.T
        d = km.DeviceBuffer(padded.nbytes); d.write(padded.astype(np.float32).ravel())
        m = km.DeviceBuffer(4 * k * dim); m.write(flat(means, layout_means))
        out = km.DeviceBuffer(4 * k * dim); out.write(np.full(k * dim, 0x7FC54321, np.uint32))
        a = km.DeviceBuffer(4 * n); a.write(np.full(n, 0xFFFFFFF1, np.uint32))
        sizes = km.DeviceBuffer(4 * k); sizes.write(np.full(k, 0xDEADBEEF, np.uint32))
        km.iteration(d, layout, stride, m, out, layout_means, km.layout_stride(layout_means, k, dim), a, sizes, dim, k, n)
        km.sync()
        assert km.last_iteration_passes() == 1, what
        got = a.read(np.uint32, n)
        assert np.array_equal(got, want), "%s: %d mismatches" % (what, int((got != want).sum()))
        counts = np.bincount(want, minlength=k)
        assert np.array_equal(sizes.read(np.uint32, k), counts), what
        gm = out.read(np.float32, k * dim)
        gm = gm.reshape(k, dim) if layout_means == 0 else gm.reshape(dim, k).T
        sums = np.zeros((k, dim)); np.add.at(sums, want, rows.astype(np.float64))
        truth = np.where(counts[:, None] > 0, sums / np.maximum(counts, 1)[:, None], 0.0)
        scale = max(float(np.sqrt(np.mean(truth ** 2))), 1e-30)
        assert float(np.abs(gm - truth).max()) / scale < 1e-4, what
        for b in (d, m, out, a, sizes):
            b.free()
