"""ORACLE -- test infrastructure: ctypes access to oracle/_build/liboracle.so (configs.c)
and, where it was built, oracle/_ref/libxkcp_ref.so (the reference's own SHA3-256)."""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "_build", "liboracle.so")
LIB_OMP = os.path.join(HERE, "_build", "liboracle_omp.so")
REF_SHA3 = os.path.join(HERE, "_ref", "libxkcp_ref.so")

_lib = None


def build():
    subprocess.run(["make", "-C", HERE], check=True, stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            build()
        L = C.CDLL(LIB)
        p, i64 = C.c_void_p, C.c_int64
        L.oracle_dotp_f32.restype = C.c_float
        L.oracle_dotp_f32.argtypes = [p, p, i64]
        L.oracle_fold_sum_i32.argtypes = [p, i64, i64, C.c_int32, p]
        L.oracle_scanl1_i64.argtypes = [p, i64, p]
        L.oracle_scanl1_f32.argtypes = [p, i64, p]
        L.oracle_scanl_i32.argtypes = [p, i64, C.c_int32, p]
        L.oracle_foldseg_i32.argtypes = [p, p, i64, C.c_int32, p]
        L.oracle_histogram_i32.argtypes = [p, i64, p, i64]
        L.oracle_jacobi_f32.argtypes = [p, p, i64, i64]
        L.oracle_jacobi_iter_f32.restype = C.c_int
        L.oracle_jacobi_iter_f32.argtypes = [p, p, i64, i64, C.c_int]
        _lib = L
    return _lib


def _c(a, dt):
    a = np.ascontiguousarray(a, dt)
    return a, a.ctypes.data


def dotp_f32(xs, ys):
    xs, px = _c(xs, np.float32)
    ys, py = _c(ys, np.float32)
    return np.float32(lib().oracle_dotp_f32(px, py, min(xs.size, ys.size)))


def fold_sum_i32(m, z):
    m, pm = _c(m, np.int32)
    rows = int(np.prod(m.shape[:-1], dtype=np.int64))
    out = np.empty(m.shape[:-1], np.int32)
    lib().oracle_fold_sum_i32(pm, rows, m.shape[-1], z, out.ctypes.data)
    return out


def scanl1_i64(x):
    x, px = _c(x, np.int64)
    out = np.empty_like(x)
    lib().oracle_scanl1_i64(px, x.size, out.ctypes.data)
    return out


def scanl1_f32(x):
    x, px = _c(x, np.float32)
    out = np.empty_like(x)
    lib().oracle_scanl1_f32(px, x.size, out.ctypes.data)
    return out


def foldseg_i32(vals, lengths, z=0):
    """foldSeg (+) z vals lengths = foldSeg' .. (scanl (+) 0 lengths)  (Prelude.hs:710-717)."""
    vals, pv = _c(vals, np.int32)
    lengths, pl = _c(lengths, np.int32)
    offs = np.empty(lengths.size + 1, np.int32)
    lib().oracle_scanl_i32(pl, lengths.size, 0, offs.ctypes.data)
    out = np.empty(lengths.size, np.int32)
    lib().oracle_foldseg_i32(pv, offs.ctypes.data, lengths.size, z, out.ctypes.data)
    return out


def histogram_i32(keys, nbins):
    keys, pk = _c(keys, np.int32)
    out = np.empty(nbins, np.int32)
    lib().oracle_histogram_i32(pk, keys.size, out.ctypes.data, nbins)
    return out


def jacobi_f32(grid, iters=1):
    a = np.array(grid, np.float32, copy=True, order="C")
    b = np.empty_like(a)
    h, w = a.shape
    where = lib().oracle_jacobi_iter_f32(a.ctypes.data, b.ctypes.data, h, w, iters)
    return b if where else a


# ---- the same loops over all host cores (configs_omp.c): a timing baseline, not the checker ----

_omp = None


def omp():
    global _omp
    if _omp is None:
        if not os.path.exists(LIB_OMP):
            build()
        L = C.CDLL(LIB_OMP)
        p, i64 = C.c_void_p, C.c_int64
        L.oracle_omp_threads.restype = C.c_int
        L.oracle_omp_dotp_f32.restype = C.c_float
        L.oracle_omp_dotp_f32.argtypes = [p, p, i64]
        L.oracle_omp_scanl1_i64.argtypes = [p, i64, p]
        L.oracle_omp_scanl1_f32.argtypes = [p, i64, p]
        L.oracle_omp_foldseg_i32.argtypes = [p, p, i64, C.c_int32, p]
        L.oracle_omp_histogram_i32.argtypes = [p, i64, p, i64]
        L.oracle_omp_jacobi_iter_f32.restype = C.c_int
        L.oracle_omp_jacobi_iter_f32.argtypes = [p, p, i64, i64, C.c_int]
        _omp = L
    return _omp


def omp_threads():
    return int(omp().oracle_omp_threads())


def omp_dotp_f32(xs, ys):
    xs, px = _c(xs, np.float32)
    ys, py = _c(ys, np.float32)
    return np.float32(omp().oracle_omp_dotp_f32(px, py, min(xs.size, ys.size)))


def omp_scanl1(x):
    x = np.ascontiguousarray(x)
    out = np.empty_like(x)
    fn = omp().oracle_omp_scanl1_i64 if x.dtype == np.int64 else omp().oracle_omp_scanl1_f32
    assert x.dtype in (np.int64, np.float32)
    fn(x.ctypes.data, x.size, out.ctypes.data)
    return out


def offsets_i32(lengths):
    """scanl (+) 0 of the segment lengths (sequential: 2^20 entries)"""
    lengths, pl = _c(lengths, np.int32)
    offs = np.empty(lengths.size + 1, np.int32)
    lib().oracle_scanl_i32(pl, lengths.size, 0, offs.ctypes.data)
    return offs


def omp_foldseg_i32(vals, offs, z=0):
    vals, pv = _c(vals, np.int32)
    offs, po = _c(offs, np.int32)
    out = np.empty(offs.size - 1, np.int32)
    omp().oracle_omp_foldseg_i32(pv, po, offs.size - 1, z, out.ctypes.data)
    return out


def seq_foldseg_offsets_i32(vals, offs, z=0):
    vals, pv = _c(vals, np.int32)
    offs, po = _c(offs, np.int32)
    out = np.empty(offs.size - 1, np.int32)
    lib().oracle_foldseg_i32(pv, po, offs.size - 1, z, out.ctypes.data)
    return out


def omp_histogram_i32(keys, nbins):
    keys, pk = _c(keys, np.int32)
    out = np.empty(nbins, np.int32)
    omp().oracle_omp_histogram_i32(pk, keys.size, out.ctypes.data, nbins)
    return out


def omp_jacobi_f32(grid, iters=1):
    a = np.array(grid, np.float32, copy=True, order="C")
    b = np.empty_like(a)
    h, w = a.shape
    where = omp().oracle_omp_jacobi_iter_f32(a.ctypes.data, b.ctypes.data, h, w, iters)
    return b if where else a


def ref_sha3_256(data: bytes):
    """Digest by the reference's own cbits/xkcp build, or None where that was not built."""
    if not os.path.exists(REF_SHA3):
        return None
    L = C.CDLL(REF_SHA3)
    L.SHA3_256.argtypes = [C.c_char_p, C.c_char_p, C.c_size_t]
    out = C.create_string_buffer(32)
    L.SHA3_256(out, data, len(data))
    return out.raw
