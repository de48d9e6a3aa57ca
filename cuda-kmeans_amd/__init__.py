"""Python plumbing over the kmx C ABI (include/kmx.h) -- used by the tests and by bench.py.

The product is the HIP library (csrc/libkmx_hip.so) and the C++ host harness (host/); this module
only binds the same C entry points with ctypes so that pytest and the benchmark can drive them. It
mirrors the reference's algorithm objects (CudaKMeansAlgorithm / CudaAssignmentAlgorithm,
experimental/k-means/k-means/headers/cuda.hpp:15-112,237-299): initialize / run / getMeans /
getAssignment / cleanup with the same meaning. There is no CPU fallback: without the built
library, or without a GPU, the calls raise.

The directory name contains a hyphen, so import it with importlib.import_module("cuda-kmeans_amd").
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
HIP_LIB_PATH = os.path.join(_HERE, "csrc", "libkmx_hip.so")
HOST_LIB_PATH = os.path.join(_HERE, "host", "libkmx_host.so")

AOS, SOA = 0, 1
ASSIGN_BASE, ASSIGN_LDS_FMA, ASSIGN_MFMA, ASSIGN_BEST, ASSIGN_MFMA_BF16X3 = 0, 1, 2, 3, 4
FUSED_TWO_PASS, FUSED_ONE_PASS, FUSED_BEST = 0, 1, 2
UPDATE_ATOMIC_POINT, UPDATE_ATOMIC_FINE, UPDATE_ATOMIC_SHM, UPDATE_BASE, UPDATE_ATOMIC_WARP = 0, 1, 2, 3, 4
UPDATE_ATOMIC_SHM2, UPDATE_FAKE, UPDATE_FAKE_SHM = 5, 6, 7  # the remaining kernels of the update micro-benchmark
UPDATE_SERIAL_ORDER = 8  # the sums of the serial loop (ascending point number inside a cluster), bit for bit, in O(n dim)
UPDATE_EMULATED_ATOMICS = 0x100  # flag for the point, fine and wavefront variants: compare-and-swap loops

KMX_OK, KMX_ERR_INVALID_ARGUMENT, KMX_ERR_UNSUPPORTED, KMX_ERR_DEVICE, KMX_ERR_NO_DEVICE = 0, 1, 2, 3, 4

# every symbol include/kmx.h declares (checked by the CPU test-suite against the built library)
ABI_SYMBOLS = [
    "kmx_device_count", "kmx_set_device", "kmx_device_props", "kmx_malloc", "kmx_free", "kmx_h2d", "kmx_d2h",
    "kmx_d2d", "kmx_sync", "kmx_set_stream", "kmx_shutdown", "kmx_fill_zero_u32", "kmx_assign_f32",
    "kmx_assign_last_rechecked", "kmx_assign_last_variant", "kmx_update_f32", "kmx_bucket_sum_f32", "kmx_fused_f32", "kmx_assign_f64", "kmx_update_f64", "kmx_fused_f64", "kmx_bucket_sum_f64", "kmx_set_queued_rows_limit",
    "kmx_graph_begin", "kmx_graph_end", "kmx_graph_launch", "kmx_graph_destroy", "kmx_event_create", "kmx_event_destroy", "kmx_event_record",
    "kmx_event_elapsed_ms", "kmx_set_profiling", "kmx_last_kernel_ms", "kmx_last_error", "kmx_certificate_tau", "kmx_certificate_unmoved_threshold",
    "kmx_update_f32_noalloc", "kmx_reserve_f32", "kmx_prepare_points_f64", "kmx_forget_points_f64", "kmx_probe_matrix_chain", "kmx_set_two_level_sweep", "kmx_iteration_f32", "kmx_iteration_last_passes",
]


class KmxError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("kmx error %d: %s" % (code, message))
        self.code = code


class ExecParams(ctypes.Structure):
    """= kmx_exec_params = CudaExecParameters (kernels.cuh:55-70)."""
    _fields_ = [("block_size", ctypes.c_uint32), ("block_count", ctypes.c_uint32),
                ("shared_mem_bytes", ctypes.c_uint32), ("privatized_copies", ctypes.c_uint32),
                ("items_per_thread", ctypes.c_uint32), ("regs_cache", ctypes.c_uint32)]

    def __init__(self, block_size=256, block_count=0, shared_mem_bytes=0, privatized_copies=1, items_per_thread=1,
                 regs_cache=1):
        super().__init__(block_size, block_count, shared_mem_bytes, privatized_copies, items_per_thread, regs_cache)


class Props(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char * 128), ("arch", ctypes.c_char * 64), ("compute_units", ctypes.c_uint32),
                ("wavefront_size", ctypes.c_uint32), ("max_threads_per_block", ctypes.c_uint32),
                ("lds_bytes_per_block", ctypes.c_uint32), ("clock_khz", ctypes.c_uint32),
                ("global_mem_bytes", ctypes.c_uint64)]


class DatasetSpec(ctypes.Structure):
    """= kmx_dataset_spec (host/datagen.h)."""
    _fields_ = [("seed", ctypes.c_uint64), ("n", ctypes.c_uint64), ("dim", ctypes.c_uint32), ("k", ctypes.c_uint32),
                ("iterations", ctypes.c_uint32), ("kind", ctypes.c_uint32), ("weights", ctypes.c_uint32),
                ("centres", ctypes.c_uint32), ("lo", ctypes.c_double), ("hi", ctypes.c_double),
                ("centre_sigma", ctypes.c_double), ("sigma", ctypes.c_double)]


def build(force=True):
    """Compile the HIP library for gfx950 and the host library (always recompiles when force)."""
    flag = ["-B"] if force else []
    subprocess.check_call(["make", "-j8"] + flag + ["-C", os.path.join(_HERE, "csrc")])
    subprocess.check_call(["make"] + flag + ["-C", os.path.join(_HERE, "host")])


_hip = None
_host = None


def hip_lib():
    """The HIP library; raises if it has not been built (no fallback)."""
    global _hip
    if _hip is None:
        if not os.path.exists(HIP_LIB_PATH):
            raise RuntimeError("libkmx_hip.so is not built (run __graft_entry__.build()); there is no CPU fallback")
        lib = ctypes.CDLL(HIP_LIB_PATH)
        vp, sz, u32 = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_uint32
        lib.kmx_last_error.restype = ctypes.c_char_p
        lib.kmx_device_count.argtypes = [ctypes.POINTER(ctypes.c_int)]
        lib.kmx_set_device.argtypes = [ctypes.c_int]
        lib.kmx_device_props.argtypes = [ctypes.POINTER(Props)]
        lib.kmx_malloc.argtypes = [ctypes.POINTER(vp), sz]
        lib.kmx_free.argtypes = [vp]
        lib.kmx_h2d.argtypes = [vp, vp, sz]
        lib.kmx_d2h.argtypes = [vp, vp, sz]
        lib.kmx_d2d.argtypes = [vp, vp, sz]
        lib.kmx_sync.argtypes = []
        lib.kmx_set_stream.argtypes = [vp]
        lib.kmx_shutdown.argtypes = []
        lib.kmx_fill_zero_u32.argtypes = [vp, sz]
        lib.kmx_assign_f32.argtypes = [ctypes.c_int, vp, ctypes.c_int, sz, vp, ctypes.c_int, sz, vp, vp, u32, u32, u32,
                                       ctypes.POINTER(ExecParams)]
        lib.kmx_assign_last_rechecked.argtypes = [ctypes.POINTER(ctypes.c_uint64)]
        lib.kmx_assign_last_variant.argtypes = [ctypes.POINTER(ctypes.c_int)]
        lib.kmx_update_f32.argtypes = [ctypes.c_int, vp, ctypes.c_int, sz, vp, vp, ctypes.c_int, sz, vp, u32, u32, u32,
                                       ctypes.POINTER(ExecParams)]
        lib.kmx_update_f32_noalloc.argtypes = lib.kmx_update_f32.argtypes
        lib.kmx_reserve_f32.argtypes = [ctypes.c_int] * 4 + [u32] * 3
        lib.kmx_prepare_points_f64.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t, u32, u32]
        lib.kmx_forget_points_f64.argtypes = []
        lib.kmx_bucket_sum_f32.argtypes = [ctypes.c_int, vp, ctypes.c_int, sz, vp, vp, ctypes.c_int, sz, u32, u32, u32,
                                           ctypes.POINTER(ExecParams)]
        lib.kmx_fused_f32.argtypes = [ctypes.c_int, vp, ctypes.c_int, sz, vp, vp, ctypes.c_int, sz, vp, u32, u32, u32,
                                      ctypes.POINTER(ExecParams)]
        lib.kmx_assign_f64.argtypes = lib.kmx_assign_f32.argtypes
        lib.kmx_update_f64.argtypes = lib.kmx_update_f32.argtypes
        lib.kmx_fused_f64.argtypes = lib.kmx_fused_f32.argtypes
        lib.kmx_bucket_sum_f64.argtypes = lib.kmx_bucket_sum_f32.argtypes
        lib.kmx_certificate_tau.argtypes = [ctypes.c_int, u32] + [ctypes.c_float] * 5 + [ctypes.POINTER(ctypes.c_float)]
        lib.kmx_certificate_unmoved_threshold.argtypes = [u32] + [ctypes.c_float] * 7 + [ctypes.POINTER(ctypes.c_float)]
        lib.kmx_graph_begin.argtypes = []
        lib.kmx_graph_end.argtypes = [ctypes.POINTER(vp)]
        lib.kmx_graph_launch.argtypes = [vp]
        lib.kmx_graph_destroy.argtypes = [vp]
        lib.kmx_event_create.argtypes = [ctypes.POINTER(vp)]
        lib.kmx_event_destroy.argtypes = [vp]
        lib.kmx_event_record.argtypes = [vp]
        lib.kmx_event_elapsed_ms.argtypes = [vp, vp, ctypes.POINTER(ctypes.c_float)]
        lib.kmx_set_profiling.argtypes = [ctypes.c_int]
        lib.kmx_set_queued_rows_limit.argtypes = [ctypes.c_size_t]
        lib.kmx_last_kernel_ms.argtypes = [ctypes.c_int, ctypes.POINTER(ctypes.c_float)]
        lib.kmx_probe_matrix_chain.argtypes = [ctypes.c_int, vp, vp, vp, vp, u32]
        lib.kmx_set_two_level_sweep.argtypes = [ctypes.c_int]
        lib.kmx_iteration_f32.argtypes = [vp, ctypes.c_int, sz, vp, vp, ctypes.c_int, sz, vp, vp, u32, u32, u32, ctypes.POINTER(ExecParams)]
        lib.kmx_iteration_last_passes.argtypes = [ctypes.POINTER(ctypes.c_int)]
        _hip = lib
    return _hip


def host_lib():
    global _host
    if _host is None:
        if not os.path.exists(HOST_LIB_PATH):
            raise RuntimeError("libkmx_host.so is not built (run __graft_entry__.build())")
        lib = ctypes.CDLL(HOST_LIB_PATH)
        lib.kmx_gen_baseline_config.argtypes = [ctypes.c_int, ctypes.POINTER(DatasetSpec)]
        lib.kmx_gen_points.argtypes = [ctypes.POINTER(DatasetSpec), ctypes.c_uint64, ctypes.c_uint64, ctypes.c_int,
                                       ctypes.c_size_t, ctypes.c_void_p, ctypes.c_int]
        lib.kmx_gen_first_k_means.argtypes = [ctypes.POINTER(DatasetSpec), ctypes.c_int, ctypes.c_size_t, ctypes.c_void_p]
        lib.kmx_fnv1a64.argtypes = [ctypes.c_void_p, ctypes.c_size_t]
        lib.kmx_fnv1a64.restype = ctypes.c_uint64
        _host = lib
    return _host


def check(rc):
    if rc != 0:
        raise KmxError(rc, hip_lib().kmx_last_error().decode())


# ---------------------------------------------------------------- data sets (host side) ----------

def layout_size(layout, count, dim):
    """LAYOUT::size with ALIGN = 1 (layout_policies.hpp:27-30,51-54)."""
    return count * dim


def layout_stride(layout, count, dim):
    """LAYOUT::precomputeConstants with ALIGN = 1 (layout_policies.hpp:32-35,56-59)."""
    return dim if layout == AOS else count


def baseline_config(config_id):
    spec = DatasetSpec()
    if host_lib().kmx_gen_baseline_config(config_id, ctypes.byref(spec)) != 0:
        raise ValueError("unknown benchmark configuration %r" % (config_id,))
    return spec


def generate_points(spec, count=None, first=0, layout=AOS, threads=0):
    """Points [first, first+count) of the data set described by spec, as a flat float32 array."""
    count = int(spec.n) if count is None else int(count)
    out = np.empty(layout_size(layout, count, spec.dim), dtype=np.float32)
    rc = host_lib().kmx_gen_points(ctypes.byref(spec), first, count, layout, layout_stride(layout, count, spec.dim),
                                   out.ctypes.data, threads)
    if rc != 0:
        raise ValueError("kmx_gen_points rejected its arguments")
    return out


def first_k_means(spec, layout_means=AOS):
    """Initial centroids = the first k points of the data set."""
    out = np.empty(layout_size(layout_means, spec.k, spec.dim), dtype=np.float32)
    rc = host_lib().kmx_gen_first_k_means(ctypes.byref(spec), layout_means, layout_stride(layout_means, spec.k, spec.dim),
                                          out.ctypes.data)
    if rc != 0:
        raise ValueError("kmx_gen_first_k_means rejected its arguments")
    return out


def widen_points(values):
    """float32 values as doubles that use the whole double mantissa: v * (1 + j * 2^-30) with j = (position % 7) - 3,
    in IEEE double arithmetic (the same bits everywhere). Inputs of the double-precision tests and fixtures."""
    v = np.ascontiguousarray(values, dtype=np.float32).astype(np.float64)
    j = (np.arange(v.size, dtype=np.int64) % 7 - 3).astype(np.float64).reshape(v.shape)
    return v * (1.0 + j * 2.0 ** -30)


def fnv1a64(array):
    a = np.ascontiguousarray(array)
    return int(host_lib().kmx_fnv1a64(a.ctypes.data, a.nbytes))


# ---------------------------------------------------------------- device plumbing ----------------

def device_count():
    c = ctypes.c_int(0)
    check(hip_lib().kmx_device_count(ctypes.byref(c)))
    return c.value


def device_props():
    p = Props()
    check(hip_lib().kmx_device_props(ctypes.byref(p)))
    return p


def sync():
    check(hip_lib().kmx_sync())


class DeviceBuffer:
    """Owned device allocation (the role of bpp::CudaBuffer in cuda.hpp:25-28)."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        self._ptr = ctypes.c_void_p(None)
        check(hip_lib().kmx_malloc(ctypes.byref(self._ptr), self.nbytes))

    @property
    def ptr(self):
        return self._ptr

    def write(self, array):
        a = np.ascontiguousarray(array)
        assert a.nbytes <= self.nbytes
        check(hip_lib().kmx_h2d(self._ptr, a.ctypes.data, a.nbytes))
        check(hip_lib().kmx_sync())  # the numpy buffer may go away right after the call

    def read(self, dtype, count):
        out = np.empty(count, dtype=dtype)
        assert out.nbytes <= self.nbytes
        check(hip_lib().kmx_d2h(out.ctypes.data, self._ptr, out.nbytes))
        return out

    def zero(self):
        check(hip_lib().kmx_fill_zero_u32(self._ptr, self.nbytes // 4))

    def free(self):
        if self._ptr:
            check(hip_lib().kmx_free(self._ptr))
            self._ptr = ctypes.c_void_p(None)

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Event:
    def __init__(self):
        self._e = ctypes.c_void_p(None)
        check(hip_lib().kmx_event_create(ctypes.byref(self._e)))

    def record(self):
        check(hip_lib().kmx_event_record(self._e))

    def elapsed_ms(self, stop):
        ms = ctypes.c_float(0)
        check(hip_lib().kmx_event_elapsed_ms(self._e, stop._e, ctypes.byref(ms)))
        return ms.value

    def __del__(self):
        try:
            if self._e:
                hip_lib().kmx_event_destroy(self._e)
        except Exception:
            pass


def _is_double(dtype):
    dtype = np.dtype(dtype)
    if dtype not in (np.dtype(np.float32), np.dtype(np.float64)):
        raise ValueError("element type must be float32 or float64")
    return dtype == np.dtype(np.float64)


def assign(variant, data_buf, layout, stride, means_buf, layout_means, stride_means, assignment_buf, dim, k, n,
           exec_params=None, dtype=np.float32):
    """ASGN_KERNEL::run (kernels.cuh:81-93) through kmx_assign_f32 / kmx_assign_f64; enqueues and returns."""
    ex = exec_params if exec_params is not None else ExecParams()
    fn = hip_lib().kmx_assign_f64 if _is_double(dtype) else hip_lib().kmx_assign_f32
    check(fn(variant, data_buf.ptr, layout, stride, means_buf.ptr, layout_means, stride_means,
                                   None, assignment_buf.ptr, dim, k, n, ctypes.byref(ex)))
    return ex


def update(variant, data_buf, layout, stride, assignment_buf, means_buf, layout_means, stride_means, sizes_buf, dim, k,
           n, exec_params=None, dtype=np.float32):
    """UPDATE_KERNEL::run (kernels.cuh:96-105) through kmx_update_f32 / kmx_update_f64; enqueues and returns."""
    ex = exec_params if exec_params is not None else ExecParams()
    fn = hip_lib().kmx_update_f64 if _is_double(dtype) else hip_lib().kmx_update_f32
    check(fn(variant, data_buf.ptr, layout, stride, assignment_buf.ptr, means_buf.ptr,
                                   layout_means, stride_means, sizes_buf.ptr, dim, k, n, ctypes.byref(ex)))
    return ex


NOALLOC_SCRATCH_BYTES = 64 << 20  # KMX_UPDATE_NOALLOC_SCRATCH_BYTES


def update_noalloc(variant, data_buf, layout, stride, assignment_buf, means_buf, layout_means, stride_means, sizes_buf, dim, k,
                   n, exec_params=None):
    """kmx_update_f32_noalloc: kmx_update_f32 with its scratch memory in the library's static device array."""
    ex = exec_params if exec_params is not None else ExecParams()
    check(hip_lib().kmx_update_f32_noalloc(variant, data_buf.ptr, layout, stride, assignment_buf.ptr, means_buf.ptr,
                                           layout_means, stride_means, sizes_buf.ptr, dim, k, n, ctypes.byref(ex)))
    return ex


def bucket_sum(variant, data_buf, layout, stride, indices_buf, result_buf, layout_result, stride_result, dim, k, n,
               exec_params=None, dtype=np.float32):
    """KERNEL::run of the update micro-benchmark (bucketing-cuda/headers/kernels.cuh:44-63) through kmx_bucket_sum_f32 / _f64."""
    ex = exec_params if exec_params is not None else ExecParams()
    fn = hip_lib().kmx_bucket_sum_f64 if _is_double(dtype) else hip_lib().kmx_bucket_sum_f32
    check(fn(variant, data_buf.ptr, layout, stride, indices_buf.ptr, result_buf.ptr,
                                       layout_result, stride_result, dim, k, n, ctypes.byref(ex)))
    return ex


def fused(variant, data_buf, layout, stride, means_in_buf, means_out_buf, layout_means, stride_means, sizes_buf, dim, k,
          n, exec_params=None, dtype=np.float32):
    """FUSED_KERNEL::run (kernels.cuh:107-116) through kmx_fused_f32 / kmx_fused_f64; enqueues and returns."""
    ex = exec_params if exec_params is not None else ExecParams()
    fn = hip_lib().kmx_fused_f64 if _is_double(dtype) else hip_lib().kmx_fused_f32
    check(fn(variant, data_buf.ptr, layout, stride, means_in_buf.ptr, means_out_buf.ptr,
                                  layout_means, stride_means, sizes_buf.ptr, dim, k, n, ctypes.byref(ex)))
    return ex


def iteration(data_buf, layout, stride, means_in_buf, means_out_buf, layout_means, stride_means, assignment_buf, sizes_buf,
              dim, k, n, exec_params=None):
    """kmx_iteration_f32: assignment (selector) and update (tuned) of one Lloyd iteration in one call; enqueues and returns."""
    ex = exec_params if exec_params is not None else ExecParams()
    check(hip_lib().kmx_iteration_f32(data_buf.ptr, layout, stride, means_in_buf.ptr, means_out_buf.ptr, layout_means, stride_means,
                                      assignment_buf.ptr, sizes_buf.ptr, dim, k, n, ctypes.byref(ex)))
    return ex


def last_iteration_passes():
    """Passes over the points the last kmx_iteration_f32 call made (1: the single-pass kernel, 2: assignment, then update)."""
    p = ctypes.c_int(0)
    check(hip_lib().kmx_iteration_last_passes(ctypes.byref(p)))
    return p.value


class Graph:
    """A recording of library calls (kmx_graph_begin .. kmx_graph_end) that can be launched as one unit."""

    def __init__(self):
        self._g = ctypes.c_void_p()

    def __enter__(self):
        check(hip_lib().kmx_graph_begin())
        return self

    def __exit__(self, exc_type, exc, tb):
        rc = hip_lib().kmx_graph_end(ctypes.byref(self._g))
        if exc_type is None:
            check(rc)
        elif rc == 0:
            self.destroy()   # a recording that ended in an exception is not kept
        return False

    def launch(self):
        check(hip_lib().kmx_graph_launch(self._g))

    def destroy(self):
        if self._g:
            check(hip_lib().kmx_graph_destroy(self._g))
            self._g = ctypes.c_void_p()


def certificate_unmoved_threshold(dim, first, tau, x2, along, c2max, m2, mnorm):
    """The threshold a sweep in a moved frame hands to the exact-pass kernels that evaluate in the frame of the data
    (kmx_certificate_unmoved_threshold; host function, no device needed)."""
    out = ctypes.c_float()
    check(hip_lib().kmx_certificate_unmoved_threshold(dim, first, tau, x2, along, c2max, m2, mnorm, ctypes.byref(out)))
    return float(out.value)


def certificate_tau(form, dim, x2, xpart2, c2max, cmid2max, crest2max):
    """The certification bound the kernels use (kmx_certificate_tau; host function, no device needed)."""
    out = ctypes.c_float()
    check(hip_lib().kmx_certificate_tau(form, dim, x2, xpart2, c2max, cmid2max, crest2max, ctypes.byref(out)))
    return out.value


def probe_matrix_chain(kind, a, b, c):
    """kmx_probe_matrix_chain on host arrays: a (32, depth), b (32, depth: row j = column j of B), c (32, 32), all
    float32; returns d = c + a b^T as the matrix cores accumulate it, block by block (kind 0: fp32 32x32x2, 1: bf16
    operands 32x32x16, 2: fp32 16x16x4)."""
    a, b, c = (np.ascontiguousarray(v, dtype=np.float32) for v in (a, b, c))
    depth = a.shape[1]
    block = {0: 2, 1: 16, 2: 4}[kind]
    assert a.shape == (32, depth) and b.shape == (32, depth) and c.shape == (32, 32) and depth % block == 0
    bufs = [DeviceBuffer(v.nbytes) for v in (a, b, c, c)]
    try:
        for buf, v in zip(bufs, (a, b, c)):
            buf.write(v)
        check(hip_lib().kmx_probe_matrix_chain(kind, bufs[0].ptr, bufs[1].ptr, bufs[2].ptr, bufs[3].ptr, depth // block))
        sync()
        return bufs[3].read(np.float32, 32 * 32).reshape(32, 32)
    finally:
        for buf in bufs:
            buf.free()


def reserve(assign_variant, update_variant, layout, layout_means, dim, k, n):
    """kmx_reserve_f32: sizes the work space so that assignment / update calls of this shape allocate nothing."""
    check(hip_lib().kmx_reserve_f32(assign_variant, update_variant, layout, layout_means, dim, k, n))


def set_queued_rows_limit(nbytes):
    """Bound of the block of copied rows the exact pass keeps for SoA points (kmx_set_queued_rows_limit)."""
    check(hip_lib().kmx_set_queued_rows_limit(ctypes.c_size_t(nbytes)))


def set_two_level_sweep(mode):
    """kmx_set_two_level_sweep: 0 = one level always, 1 = two levels where they pay (default), 2 = wherever the kernels allow."""
    check(hip_lib().kmx_set_two_level_sweep(mode))


def set_profiling(enabled):
    check(hip_lib().kmx_set_profiling(1 if enabled else 0))


def last_kernel_ms(which):
    """Duration of the dominant kernel of the last assignment (0) / update (1) call made under set_profiling(True)."""
    ms = ctypes.c_float(0)
    check(hip_lib().kmx_last_kernel_ms(which, ctypes.byref(ms)))
    return ms.value


def last_assign_variant():
    """The concrete variant the last assignment call ran (what ASSIGN_BEST selected)."""
    v = ctypes.c_int(-1)
    check(hip_lib().kmx_assign_last_variant(ctypes.byref(v)))
    return v.value


def last_rechecked():
    c = ctypes.c_uint64(0)
    check(hip_lib().kmx_assign_last_rechecked(ctypes.byref(c)))
    return c.value


# ---------------------------------------------------------------- algorithm objects --------------

class HipKMeansAlgorithm:
    """Mirror of CudaKMeansAlgorithm (cuda.hpp:15-112): ping-pong means/assignment buffers, per iteration
    assign -> zero(means[next]) -> zero(sizes) -> update(+divide), one sync at the end of run()."""

    def __init__(self, assign_variant=ASSIGN_BEST, update_variant=UPDATE_ATOMIC_SHM, exec_params=None,
                 layout=AOS, layout_means=AOS, dtype=np.float32):
        self.dtype = np.dtype(dtype)  # float32, or float64 for the reference's --double instantiation
        self.item = self.dtype.itemsize
        self.assign_variant = assign_variant
        self.update_variant = update_variant
        self.exec = exec_params if exec_params is not None else ExecParams()
        self.layout, self.layout_means = layout, layout_means
        self.rechecked = []  # filled by run(collect_rechecked=True)
        self._bufs = []

    def initialize(self, dim, k, n, iters, data, means):
        if device_count() == 0:
            raise KmxError(KMX_ERR_NO_DEVICE, "No HIP devices found!")
        check(hip_lib().kmx_set_device(0))
        self.dim, self.k, self.n, self.iters = int(dim), int(k), int(n), int(iters)
        self.stride = layout_stride(self.layout, self.n, self.dim)
        self.stride_means = layout_stride(self.layout_means, self.k, self.dim)
        self.means_size = layout_size(self.layout_means, self.k, self.dim)
        copies = max(1, self.exec.privatized_copies)
        self.cu_data = DeviceBuffer(self.item * layout_size(self.layout, self.n, self.dim))
        self.cu_sizes = DeviceBuffer(4 * self.k)
        self.cu_means = [DeviceBuffer(self.item * self.means_size * copies) for _ in range(2)]
        self.cu_assignment = [DeviceBuffer(4 * self.n) for _ in range(2)]
        self._bufs = [self.cu_data, self.cu_sizes] + self.cu_means + self.cu_assignment
        self.cu_data.write(data)
        if _is_double(self.dtype):   # the points never change after the upload (cuda.hpp:54-64): their float copy is made once
            check(hip_lib().kmx_prepare_points_f64(self.cu_data.ptr, self.layout, self.stride, self.dim, self.n))
        self.reset(means)

    def reset(self, means):
        """Back to the state right after initialize() (initial centroids, zeroed assignment)."""
        self.last = 0
        self.cu_means[0].write(means)
        self.cu_assignment[0].zero()
        self.cu_sizes.zero()
        sync()

    def iteration(self):
        nxt = (self.last + 1) % 2
        assign(self.assign_variant, self.cu_data, self.layout, self.stride, self.cu_means[self.last], self.layout_means,
               self.stride_means, self.cu_assignment[nxt], self.dim, self.k, self.n, self.exec, self.dtype)
        return nxt

    def update_step(self, nxt):
        # the tuned float update clears or overwrites its outputs itself (kmx_update_f32, KMX_UPDATE_ATOMIC_SHM)
        self_clearing = (self.update_variant == UPDATE_ATOMIC_SHM and np.dtype(self.dtype) == np.float32) or \
            self.update_variant == UPDATE_SERIAL_ORDER
        if not self_clearing:
            self.cu_means[nxt].zero()
            self.cu_sizes.zero()
        update(self.update_variant, self.cu_data, self.layout, self.stride, self.cu_assignment[nxt], self.cu_means[nxt],
               self.layout_means, self.stride_means, self.cu_sizes, self.dim, self.k, self.n, self.exec, self.dtype)
        self.last = nxt

    def one_call(self):
        """The default pair of kernels on floats goes through kmx_iteration_f32, which reads the points once where it can."""
        return self.assign_variant == ASSIGN_BEST and self.update_variant == UPDATE_ATOMIC_SHM and self.dtype == np.dtype(np.float32)

    def step(self):
        """One whole iteration: one kmx_iteration_f32 call for the default pair of kernels, else assignment, then update."""
        if not self.one_call():
            self.update_step(self.iteration())
            return
        nxt = (self.last + 1) % 2
        iteration(self.cu_data, self.layout, self.stride, self.cu_means[self.last], self.cu_means[nxt], self.layout_means,
                  self.stride_means, self.cu_assignment[nxt], self.cu_sizes, self.dim, self.k, self.n, self.exec)
        self.last = nxt

    def run(self, iters=None, collect_rechecked=False, use_graph=False):
        """All iterations, one sync at the end. use_graph: the first iteration runs call by call (it sizes the work
        space), then two ping-pong iterations are recorded once and replayed; an odd one out runs call by call."""
        todo = self.iters if iters is None else iters
        if use_graph and not collect_rechecked and todo >= 3:
            self.step()
            pairs = (todo - 1) // 2
            with Graph() as g:
                for _ in range(2):
                    self.step()
            for _ in range(pairs):
                g.launch()
            todo -= 1 + 2 * pairs
            for _ in range(todo):
                self.step()
            sync()
            g.destroy()
            return
        for _ in range(todo):
            if collect_rechecked:
                nxt = self.iteration()
                self.rechecked.append(last_rechecked())
                self.update_step(nxt)
            else:
                self.step()
        sync()

    def getMeans(self):
        return self.cu_means[self.last].read(self.dtype, self.means_size)

    def getAssignment(self):
        return self.cu_assignment[self.last].read(np.uint32, self.n)

    def getClusterSizes(self):
        return self.cu_sizes.read(np.uint32, self.k)

    def cleanup(self):
        if _is_double(self.dtype):
            check(hip_lib().kmx_forget_points_f64())
        for b in self._bufs:
            b.free()
        self._bufs = []


class HipFusedKMeansAlgorithm:
    """Mirror of CudaFusedKMeansAlgorithm (cuda.hpp:116-233): no assignment buffers; per iteration
    zero(means[next]) -> zero(sizes) -> fused(means[last] -> means[next]); getAssignment() is computed afterwards
    against the FINAL centroids (the reference does that on the host, cuda.hpp:199-221; here one more device pass)."""

    def __init__(self, variant=FUSED_BEST, exec_params=None, layout=AOS, layout_means=AOS, dtype=np.float32):
        self.dtype = np.dtype(dtype)
        self.item = self.dtype.itemsize
        self.variant = variant
        self.exec = exec_params if exec_params is not None else ExecParams()
        self.layout, self.layout_means = layout, layout_means
        self._bufs = []

    def initialize(self, dim, k, n, iters, data, means):
        if device_count() == 0:
            raise KmxError(KMX_ERR_NO_DEVICE, "No HIP devices found!")
        check(hip_lib().kmx_set_device(0))
        self.dim, self.k, self.n, self.iters = int(dim), int(k), int(n), int(iters)
        self.stride = layout_stride(self.layout, self.n, self.dim)
        self.stride_means = layout_stride(self.layout_means, self.k, self.dim)
        self.means_size = layout_size(self.layout_means, self.k, self.dim)
        self.cu_data = DeviceBuffer(self.item * layout_size(self.layout, self.n, self.dim))
        self.cu_sizes = DeviceBuffer(4 * self.k)
        self.cu_means = [DeviceBuffer(self.item * self.means_size) for _ in range(2)]
        self._bufs = [self.cu_data, self.cu_sizes] + self.cu_means
        self.cu_data.write(data)
        if _is_double(self.dtype):   # see HipKMeansAlgorithm.initialize
            check(hip_lib().kmx_prepare_points_f64(self.cu_data.ptr, self.layout, self.stride, self.dim, self.n))
        self.last = 0
        self.cu_means[0].write(means)
        self.cu_sizes.zero()
        sync()

    def reset(self, means):
        """Back to the state right after initialize() (initial centroids)."""
        self.last = 0
        self.cu_means[0].write(means)
        self.cu_sizes.zero()
        sync()

    def iteration(self):
        nxt = (self.last + 1) % 2
        self.cu_means[nxt].zero()
        self.cu_sizes.zero()
        fused(self.variant, self.cu_data, self.layout, self.stride, self.cu_means[self.last], self.cu_means[nxt],
              self.layout_means, self.stride_means, self.cu_sizes, self.dim, self.k, self.n, self.exec, self.dtype)
        self.last = nxt

    def run(self, iters=None):
        for _ in range(self.iters if iters is None else iters):
            self.iteration()
        sync()

    def getMeans(self):
        return self.cu_means[self.last].read(self.dtype, self.means_size)

    def getClusterSizes(self):
        return self.cu_sizes.read(np.uint32, self.k)

    def getAssignment(self):
        out = DeviceBuffer(4 * max(self.n, 1))
        try:
            assign(ASSIGN_BEST, self.cu_data, self.layout, self.stride, self.cu_means[self.last], self.layout_means,
                   self.stride_means, out, self.dim, self.k, self.n, self.exec, self.dtype)
            sync()
            return out.read(np.uint32, self.n)
        finally:
            out.free()

    def cleanup(self):
        if _is_double(self.dtype):
            check(hip_lib().kmx_forget_points_f64())
        for b in self._bufs:
            b.free()
        self._bufs = []


class HipAssignmentAlgorithm:
    """Mirror of CudaAssignmentAlgorithm (cuda.hpp:237-299): one assignment pass."""

    def __init__(self, variant=ASSIGN_BEST, exec_params=None, layout=AOS, layout_means=AOS, dtype=np.float32):
        self.dtype = np.dtype(dtype)
        self.item = self.dtype.itemsize
        self.variant = variant
        self.exec = exec_params if exec_params is not None else ExecParams()
        self.layout, self.layout_means = layout, layout_means
        self._bufs = []

    def initialize(self, dim, k, n, data, means):
        if device_count() == 0:
            raise KmxError(KMX_ERR_NO_DEVICE, "No HIP devices found!")
        check(hip_lib().kmx_set_device(0))
        self.dim, self.k, self.n = int(dim), int(k), int(n)
        self.cu_data = DeviceBuffer(self.item * layout_size(self.layout, self.n, self.dim))
        self.cu_means = DeviceBuffer(self.item * layout_size(self.layout_means, self.k, self.dim))
        self.cu_assignment = DeviceBuffer(4 * max(self.n, 1))
        self._bufs = [self.cu_data, self.cu_means, self.cu_assignment]
        self.cu_data.write(data)
        self.cu_means.write(means)
        sync()

    def run(self):
        assign(self.variant, self.cu_data, self.layout, layout_stride(self.layout, self.n, self.dim), self.cu_means,
               self.layout_means, layout_stride(self.layout_means, self.k, self.dim), self.cu_assignment, self.dim,
               self.k, self.n, self.exec, self.dtype)
        sync()

    def getAssignment(self):
        return self.cu_assignment.read(np.uint32, self.n)

    def cleanup(self):
        for b in self._bufs:
            b.free()
        self._bufs = []
