"""kmx_update_f32_noalloc (the entry point that allocates nothing) against kmx_update_f32, through the C ABI on a real
MI355X: same counts bit for bit, same centroids within the update's tolerance, on two calls in a row of which the
second has the smaller input (the scratch array keeps the first call's contents), and a refusal by name when the
partial sums do not fit the static array."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

AOS, SOA = 0, 1
CENTROID_RTOL = 1e-4


def run_update(km, fn, variant, d, a, dim, k, n, layout, layout_means, dirty_word):
    msize = km.layout_size(layout_means, k, dim)
    m = km.DeviceBuffer(4 * msize); s = km.DeviceBuffer(4 * k)
    if variant == km.UPDATE_ATOMIC_SHM:     # no precondition on the outputs: hand over leftovers
        m.write(np.full(msize, dirty_word, np.uint32)); s.write(np.full(k, 0xDEADBEEF, np.uint32))
    else:
        m.zero(); s.zero()
    fn(variant, d, layout, km.layout_stride(layout, n, dim), a, m, layout_means, km.layout_stride(layout_means, k, dim), s, dim, k, n)
    km.sync()
    out = m.read(np.float32, msize), s.read(np.uint32, k)
    m.free(); s.free()
    return out


def rel_err(got, want):
    scale = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
    return float(np.abs(got.astype(np.float64) - want).max() / max(scale, 1e-30))


# (dim, k, first n, second n): the sorted path (partial sums in the scratch array) and the private-copies path (no scratch)
CASES = [(32, 1024, 300000, 70000), (4, 4096, 500000, 4099), (256, 300, 60000, 999), (8, 64, 100000, 5000), (16, 16, 200000, 777)]


@pytest.mark.parametrize("dim,k,n1,n2", CASES)
@pytest.mark.parametrize("layout,layout_means", [(AOS, AOS), (AOS, SOA), (SOA, AOS)])
def test_noalloc_update_equals_update(km, orc, gpu, dim, k, n1, n2, layout, layout_means):
    rng = np.random.default_rng(dim * 1000 + k)
    for n in (n1, n2):                                   # two calls in a row, the second smaller
        pts = rng.normal(size=(n, dim)).astype(np.float32) * np.float32(3)
        asg = rng.integers(0, k, size=n).astype(np.uint32)
        asg[asg == 1] = 0                                # an empty cluster
        data = np.ascontiguousarray(pts if layout == AOS else pts.T).ravel()
        d = km.DeviceBuffer(data.nbytes); d.write(data)
        a = km.DeviceBuffer(4 * n); a.write(asg)
        for variant in (km.UPDATE_ATOMIC_SHM, km.UPDATE_ATOMIC_FINE):
            want_m, want_s = run_update(km, km.update, variant, d, a, dim, k, n, layout, layout_means, 0x7FC12345)
            got_m, got_s = run_update(km, km.update_noalloc, variant, d, a, dim, k, n, layout, layout_means, 0x7FC54321)
            assert np.array_equal(got_s, want_s), (variant, n)
            assert rel_err(got_m, want_m) < CENTROID_RTOL, (variant, n)
        om, osz = orc.update(data, asg, dim, k, n, layout, layout_means, threads=0)
        assert np.array_equal(got_s, osz) and rel_err(got_m, om) < CENTROID_RTOL
        d.free(); a.free()


def device_memory_in_use():
    """Bytes of device memory in use, asked of the HIP runtime this process has loaded (hipMemGetInfo)."""
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")
    free, total = ctypes.c_size_t(0), ctypes.c_size_t(0)
    assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
    return total.value - free.value


def test_noalloc_update_allocates_nothing_and_records(km, orc, gpu):
    """After the device has been set up (kmx_set_device looks up the scratch array), calls of the entry point leave the
    device's memory in use unchanged -- under a graph recording too, whose replays give the eager call's result."""
    dim, k, n = 32, 1024, 200000
    rng = np.random.default_rng(3)
    pts = rng.normal(size=(n, dim)).astype(np.float32)
    asg = rng.integers(0, k, size=n).astype(np.uint32)
    d = km.DeviceBuffer(pts.nbytes); d.write(pts.ravel())
    a = km.DeviceBuffer(4 * n); a.write(asg)
    m = km.DeviceBuffer(4 * k * dim); s = km.DeviceBuffer(4 * k)
    km.sync()
    before = device_memory_in_use()
    km.update_noalloc(km.UPDATE_ATOMIC_SHM, d, AOS, dim, a, m, AOS, dim, s, dim, k, n)
    km.sync()
    assert device_memory_in_use() == before
    want_m, want_s = m.read(np.float32, k * dim), s.read(np.uint32, k)
    om, osz = orc.update(pts.ravel(), asg, dim, k, n, threads=0)
    assert np.array_equal(want_s, osz) and rel_err(want_m, om) < CENTROID_RTOL
    with km.Graph() as g:
        km.update_noalloc(km.UPDATE_ATOMIC_SHM, d, AOS, dim, a, m, AOS, dim, s, dim, k, n)
    for _ in range(3):
        m.write(np.full(k * dim, 0x7FC00001, np.uint32)); s.write(np.full(k, 7, np.uint32))   # eager work between the replays
        g.launch()
        km.sync()
        assert np.array_equal(s.read(np.uint32, k), want_s)
        assert rel_err(m.read(np.float32, k * dim), want_m) < 1e-5   # (the order of the additions inside a cluster varies from run to run)
    g.destroy()   # (the runtime keeps memory of its own for a graph: nothing to compare after this point)
    for b in (d, a, m, s):
        b.free()


def test_noalloc_update_refuses_what_does_not_fit(km, gpu):
    dim, k, n = 64, 16384, 1 << 20                       # 32 chunks x 2 slices... x 16384 x 65 words: beyond 64 MiB
    d = km.DeviceBuffer(4 * n * dim); d.zero()
    a = km.DeviceBuffer(4 * n); a.zero()
    m = km.DeviceBuffer(4 * k * dim); s = km.DeviceBuffer(4 * k)
    with pytest.raises(km.KmxError, match="scratch memory"):
        km.update_noalloc(km.UPDATE_ATOMIC_SHM, d, AOS, dim, a, m, AOS, dim, s, dim, k, n)
    km.update(km.UPDATE_ATOMIC_SHM, d, AOS, dim, a, m, AOS, dim, s, dim, k, n)     # the allocating entry point takes it
    km.sync()
    assert s.read(np.uint32, k)[0] == n
    for b in (d, a, m, s):
        b.free()
