"""TEST INFRASTRUCTURE ONLY -- ctypes bindings for the CPU oracle (oracle/liboracle.so) and, where
it was built, the reference's own serial k-means (oracle/_ref/libref_serial.so).

Only tests, the smoke check and the benchmark's cpu_baseline leg may import this module.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_f32p = ctypes.POINTER(ctypes.c_float)
_u32p = ctypes.POINTER(ctypes.c_uint32)
_f64p = ctypes.POINTER(ctypes.c_double)

AOS, SOA = 0, 1


def layout_size(layout, count, dim):
    """Number of floats of a (count x dim) array; ALIGN = 1 (layout_policies.hpp:27-30,51-54)."""
    return count * dim


def layout_stride(layout, count, dim):
    """precomputeConstants (layout_policies.hpp:32-35,56-59)."""
    return dim if layout == AOS else count


def _ptr(a, typ):
    return a.ctypes.data_as(typ) if a is not None else None


def build(force=False):
    """Compile liboracle.so (and oracle/_ref when the reference tree is present)."""
    subprocess.check_call(["make", "-B" if force else "-s", "-C", _HERE, "all"], stdout=subprocess.DEVNULL)


_oracle = None
_ref = None


def oracle_lib():
    global _oracle
    if _oracle is None:
        path = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            build()
        lib = ctypes.CDLL(path)
        sig = [_f32p, ctypes.c_int, ctypes.c_size_t, _f32p, ctypes.c_int, ctypes.c_size_t,
               ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, _u32p, _f32p, _f32p, ctypes.c_int]
        lib.oracle_assign.argtypes = sig
        lib.oracle_assign.restype = None
        lib.oracle_assign_fast.argtypes = sig
        lib.oracle_assign_fast.restype = None
        lib.oracle_update.argtypes = [_f32p, ctypes.c_int, ctypes.c_size_t, _u32p, _f32p, ctypes.c_int, ctypes.c_size_t,
                                      _u32p, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_int]
        lib.oracle_update.restype = None
        lib.oracle_kmeans.argtypes = [_f32p, ctypes.c_int, ctypes.c_size_t, _f32p, ctypes.c_int, ctypes.c_size_t,
                                      ctypes.c_size_t, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32,
                                      _u32p, _u32p, ctypes.c_int, ctypes.c_int]
        lib.oracle_kmeans.restype = None
        lib.oracle_assign_f64.argtypes = [_f64p, ctypes.c_int, ctypes.c_size_t, _f64p, ctypes.c_int, ctypes.c_size_t,
                                          ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, _u32p, _f64p, _f64p, ctypes.c_int]
        lib.oracle_assign_f64.restype = None
        lib.oracle_update_f64.argtypes = [_f64p, ctypes.c_int, ctypes.c_size_t, _u32p, _f64p, ctypes.c_int, ctypes.c_size_t,
                                          _u32p, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_int]
        lib.oracle_update_f64.restype = None
        lib.oracle_kmeans_f64.argtypes = [_f64p, ctypes.c_int, ctypes.c_size_t, _f64p, ctypes.c_int, ctypes.c_size_t,
                                          ctypes.c_size_t, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32,
                                          _u32p, _u32p, ctypes.c_int]
        lib.oracle_kmeans_f64.restype = None
        _oracle = lib
    return _oracle


def ref_lib():
    """The reference's own serial implementation, or None where it was not built."""
    global _ref
    if _ref is None:
        path = os.path.join(_HERE, "_ref", "libref_serial.so")
        if not os.path.exists(path):
            return None
        lib = ctypes.CDLL(path)
        lib.ref_serial_kmeans.argtypes = [_f32p, ctypes.c_int, _f32p, ctypes.c_int, ctypes.c_size_t, ctypes.c_size_t,
                                          ctypes.c_size_t, ctypes.c_size_t, _f32p, _u32p]
        lib.ref_serial_kmeans.restype = ctypes.c_int
        lib.ref_serial_assign.argtypes = [_f32p, ctypes.c_int, _f32p, ctypes.c_int, ctypes.c_size_t, ctypes.c_size_t,
                                          ctypes.c_size_t, _u32p]
        lib.ref_serial_assign.restype = ctypes.c_int
        if hasattr(lib, "ref_serial_kmeans_f64"):
            lib.ref_serial_kmeans_f64.argtypes = [_f64p, ctypes.c_int, _f64p, ctypes.c_int, ctypes.c_size_t, ctypes.c_size_t,
                                                  ctypes.c_size_t, ctypes.c_size_t, _f64p, _u32p]
            lib.ref_serial_kmeans_f64.restype = ctypes.c_int
            lib.ref_serial_assign_f64.argtypes = [_f64p, ctypes.c_int, _f64p, ctypes.c_int, ctypes.c_size_t, ctypes.c_size_t,
                                                  ctypes.c_size_t, _u32p]
            lib.ref_serial_assign_f64.restype = ctypes.c_int
        _ref = lib
    return _ref


def _check(data, means, layout, layout_means, dim, k, n, dtype=np.float32):
    assert data.dtype == dtype and means.dtype == dtype
    assert data.flags.c_contiguous and means.flags.c_contiguous
    assert data.size >= layout_size(layout, n, dim) and means.size >= layout_size(layout_means, k, dim)


def assign(data, means, dim, k, n, layout=AOS, layout_means=AOS, threads=1, fast=False, detail=False):
    """Oracle assignment. Returns assignment, or (assignment, best_dist, second_dist) with detail=True."""
    _check(data, means, layout, layout_means, dim, k, n)
    lib = oracle_lib()
    asg = np.empty(n, dtype=np.uint32)
    best = np.empty(n, dtype=np.float32) if detail else None
    second = np.empty(n, dtype=np.float32) if detail else None
    fn = lib.oracle_assign_fast if fast else lib.oracle_assign
    fn(_ptr(data, _f32p), layout, layout_stride(layout, n, dim), _ptr(means, _f32p), layout_means,
       layout_stride(layout_means, k, dim), dim, k, n, _ptr(asg, _u32p), _ptr(best, _f32p), _ptr(second, _f32p), threads)
    return (asg, best, second) if detail else asg


def update(data, assignment, dim, k, n, layout=AOS, layout_means=AOS, threads=1):
    """Oracle update. Returns (means, cluster_sizes)."""
    assert assignment.dtype == np.uint32 and assignment.size >= n
    means = np.zeros(layout_size(layout_means, k, dim), dtype=np.float32)
    sizes = np.zeros(k, dtype=np.uint32)
    oracle_lib().oracle_update(_ptr(data, _f32p), layout, layout_stride(layout, n, dim), _ptr(assignment, _u32p),
                               _ptr(means, _f32p), layout_means, layout_stride(layout_means, k, dim), _ptr(sizes, _u32p),
                               dim, k, n, threads)
    return means, sizes


def kmeans(data, means, dim, k, n, iters, layout=AOS, layout_means=AOS, threads=1, fast=False):
    """Oracle Lloyd iterations. Returns (means, assignment, cluster_sizes)."""
    _check(data, means, layout, layout_means, dim, k, n)
    m = means.copy()
    asg = np.zeros(n, dtype=np.uint32)
    sizes = np.zeros(k, dtype=np.uint32)
    oracle_lib().oracle_kmeans(_ptr(data, _f32p), layout, layout_stride(layout, n, dim), _ptr(m, _f32p), layout_means,
                               layout_stride(layout_means, k, dim), m.size, dim, k, n, iters, _ptr(asg, _u32p),
                               _ptr(sizes, _u32p), threads, 1 if fast else 0)
    return m, asg, sizes


def ref_kmeans(data, means, dim, k, n, iters, layout=AOS, layout_means=AOS):
    """The reference's SerialKMeansAlgorithm (only where oracle/_ref was built). Returns (means, assignment)."""
    lib = ref_lib()
    if lib is None:
        raise RuntimeError("oracle/_ref/libref_serial.so is not built")
    _check(data, means, layout, layout_means, dim, k, n)
    m = np.empty(layout_size(layout_means, k, dim), dtype=np.float32)
    asg = np.empty(n, dtype=np.uint32)
    rc = lib.ref_serial_kmeans(_ptr(data, _f32p), layout, _ptr(means, _f32p), layout_means, dim, k, n, iters,
                               _ptr(m, _f32p), _ptr(asg, _u32p))
    assert rc == 0
    return m, asg


def ref_assign(data, means, dim, k, n, layout=AOS, layout_means=AOS):
    """The reference's SerialAssignmentAlgorithm (only where oracle/_ref was built)."""
    lib = ref_lib()
    if lib is None:
        raise RuntimeError("oracle/_ref/libref_serial.so is not built")
    _check(data, means, layout, layout_means, dim, k, n)
    asg = np.empty(n, dtype=np.uint32)
    rc = lib.ref_serial_assign(_ptr(data, _f32p), layout, _ptr(means, _f32p), layout_means, dim, k, n, _ptr(asg, _u32p))
    assert rc == 0
    return asg


# ---- F = double (the reference's --double instantiation) ----

def assign_f64(data, means, dim, k, n, layout=AOS, layout_means=AOS, threads=1, detail=False):
    """Oracle assignment on doubles. Returns assignment, or (assignment, best_dist, second_dist) with detail=True."""
    _check(data, means, layout, layout_means, dim, k, n, np.float64)
    asg = np.empty(n, dtype=np.uint32)
    best = np.empty(n, dtype=np.float64) if detail else None
    second = np.empty(n, dtype=np.float64) if detail else None
    oracle_lib().oracle_assign_f64(_ptr(data, _f64p), layout, layout_stride(layout, n, dim), _ptr(means, _f64p), layout_means,
                                   layout_stride(layout_means, k, dim), dim, k, n, _ptr(asg, _u32p), _ptr(best, _f64p),
                                   _ptr(second, _f64p), threads)
    return (asg, best, second) if detail else asg


def update_f64(data, assignment, dim, k, n, layout=AOS, layout_means=AOS, threads=1):
    """Oracle update on doubles. Returns (means, cluster_sizes)."""
    assert data.dtype == np.float64 and assignment.dtype == np.uint32 and assignment.size >= n
    means = np.zeros(layout_size(layout_means, k, dim), dtype=np.float64)
    sizes = np.zeros(k, dtype=np.uint32)
    oracle_lib().oracle_update_f64(_ptr(data, _f64p), layout, layout_stride(layout, n, dim), _ptr(assignment, _u32p),
                                   _ptr(means, _f64p), layout_means, layout_stride(layout_means, k, dim), _ptr(sizes, _u32p),
                                   dim, k, n, threads)
    return means, sizes


def kmeans_f64(data, means, dim, k, n, iters, layout=AOS, layout_means=AOS, threads=1):
    """Oracle Lloyd iterations on doubles. Returns (means, assignment, cluster_sizes)."""
    _check(data, means, layout, layout_means, dim, k, n, np.float64)
    m = means.copy()
    asg = np.zeros(n, dtype=np.uint32)
    sizes = np.zeros(k, dtype=np.uint32)
    oracle_lib().oracle_kmeans_f64(_ptr(data, _f64p), layout, layout_stride(layout, n, dim), _ptr(m, _f64p), layout_means,
                                   layout_stride(layout_means, k, dim), m.size, dim, k, n, iters, _ptr(asg, _u32p),
                                   _ptr(sizes, _u32p), threads)
    return m, asg, sizes


def ref_kmeans_f64(data, means, dim, k, n, iters, layout=AOS, layout_means=AOS):
    """The reference's SerialKMeansAlgorithm<double, ...> (only where oracle/_ref was built). Returns (means, assignment)."""
    lib = ref_lib()
    if lib is None or not hasattr(lib, "ref_serial_kmeans_f64"):
        raise RuntimeError("oracle/_ref/libref_serial.so is not built")
    _check(data, means, layout, layout_means, dim, k, n, np.float64)
    m = np.empty(layout_size(layout_means, k, dim), dtype=np.float64)
    asg = np.empty(n, dtype=np.uint32)
    rc = lib.ref_serial_kmeans_f64(_ptr(data, _f64p), layout, _ptr(means, _f64p), layout_means, dim, k, n, iters,
                                   _ptr(m, _f64p), _ptr(asg, _u32p))
    assert rc == 0
    return m, asg


def ref_assign_f64(data, means, dim, k, n, layout=AOS, layout_means=AOS):
    """The reference's SerialAssignmentAlgorithm<double, ...> (only where oracle/_ref was built)."""
    lib = ref_lib()
    if lib is None or not hasattr(lib, "ref_serial_assign_f64"):
        raise RuntimeError("oracle/_ref/libref_serial.so is not built")
    _check(data, means, layout, layout_means, dim, k, n, np.float64)
    asg = np.empty(n, dtype=np.uint32)
    rc = lib.ref_serial_assign_f64(_ptr(data, _f64p), layout, _ptr(means, _f64p), layout_means, dim, k, n, _ptr(asg, _u32p))
    assert rc == 0
    return asg
