"""Loader for the CPU oracle (``oracle/liboracle.so``) and, where it was built,
the reference's own compiled ``core_ops.cpp`` (``oracle/_ref``).

Checker only: imported by the tests, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py``; never by the product.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
LIB = os.path.join(ORACLE_DIR, "liboracle.so")
REF_LIB = os.path.join(ORACLE_DIR, "_ref", "libref_coreops.so")

TOL = {np.dtype(np.float32): 1e-5, np.dtype(np.float64): 1e-12}

_u32, _u64, _vp = ctypes.c_uint32, ctypes.c_uint64, ctypes.c_void_p
_lib = None
_ref = None


def _p(a):
    return a.ctypes.data_as(_vp)


def load(path: str = LIB):
    global _lib
    if _lib is not None and path == LIB:
        return _lib
    if not os.path.exists(path):
        target = os.path.basename(path)
        subprocess.run(["make", "-C", ORACLE_DIR, target], check=True, capture_output=True)
    lib = ctypes.CDLL(path)
    for name in ("oracle_sddmm_f64", "oracle_sddmm_f32", "oracle_sddmm_scale_f64"):
        fn = getattr(lib, name)
        fn.restype = ctypes.c_int
        fn.argtypes = [_u32, _u32, _u32, _vp, _vp, _u64, _vp, _vp, _vp, _vp]
    for name in ("oracle_spmm_f64", "oracle_spmm_f32", "oracle_spmm_scale_f64"):
        fn = getattr(lib, name)
        fn.restype = ctypes.c_int
        fn.argtypes = [_u32, _u32, _u32, _vp, _u64, _vp, _vp, _vp, _vp]
    if path == LIB:
        _lib = lib
    return lib


def have_ref() -> bool:
    return os.path.exists(REF_LIB)


def load_ref():
    """The reference's own core_ops.cpp behind C entry points (fp64 only)."""
    global _ref
    if _ref is None:
        lib = ctypes.CDLL(REF_LIB)
        lib.ref_sddmm_f64.restype = ctypes.c_int
        lib.ref_sddmm_f64.argtypes = [_u32, _u32, _u32, _vp, _vp, _u64, _vp, _vp, _vp, _vp]
        lib.ref_spmm_f64.restype = ctypes.c_int
        lib.ref_spmm_f64.argtypes = [_u32, _u32, _u32, _vp, _u64, _vp, _vp, _vp, _vp]
        lib.ref_localize_indices.restype = ctypes.c_int
        lib.ref_localize_indices.argtypes = [_u64, _vp, _vp, _vp, _vp, _vp, _vp]
        _ref = lib
    return _ref


def _prep(ii, jj):
    return (np.ascontiguousarray(ii, dtype=np.uint32), np.ascontiguousarray(jj, dtype=np.uint32))


def _suffix(dtype):
    return "f64" if np.dtype(dtype) == np.float64 else "f32"


def sddmm(A, B, ii, jj, svv, lib=None) -> np.ndarray:
    """C.vv of the reference's sddmm (src/core_ops.cpp:5-22), same real type as A."""
    lib = lib or load()
    A, B, svv = (np.ascontiguousarray(x) for x in (A, B, svv))
    assert A.dtype == B.dtype == svv.dtype and A.shape[1] == B.shape[1]
    ii, jj = _prep(ii, jj)
    out = np.empty(ii.size, dtype=A.dtype)
    fn = getattr(lib, "oracle_sddmm_" + _suffix(A.dtype))
    rc = fn(A.shape[0], B.shape[0], A.shape[1], _p(A), _p(B), ii.size, _p(ii), _p(jj), _p(svv),
            _p(out))
    if rc != 0:
        raise IndexError("oracle sddmm: index out of range")
    return out


def spmm(X, ii, jj, avv, Y, lib=None) -> np.ndarray:
    """Y after the reference's spmm (src/core_ops.cpp:24-35); Y is copied, not modified."""
    lib = lib or load()
    X, avv = np.ascontiguousarray(X), np.ascontiguousarray(avv)
    Y = np.array(Y, copy=True, order="C")
    assert X.dtype == Y.dtype == avv.dtype and X.shape[1] == Y.shape[1]
    ii, jj = _prep(ii, jj)
    fn = getattr(lib, "oracle_spmm_" + _suffix(X.dtype))
    rc = fn(X.shape[0], Y.shape[0], X.shape[1], _p(X), ii.size, _p(ii), _p(jj), _p(avv), _p(Y))
    if rc != 0:
        raise IndexError("oracle spmm: index out of range")
    return Y


def sddmm_scale(A, B, ii, jj, svv) -> np.ndarray:
    """|S.vv[e]| * sum_j |A[r,j] B[c,j]| in double: the magnitude each result is judged against."""
    lib = load()
    A, B, svv = (np.ascontiguousarray(x, dtype=np.float64) for x in (A, B, svv))
    ii, jj = _prep(ii, jj)
    out = np.empty(ii.size, dtype=np.float64)
    rc = lib.oracle_sddmm_scale_f64(A.shape[0], B.shape[0], A.shape[1], _p(A), _p(B), ii.size,
                                    _p(ii), _p(jj), _p(svv), _p(out))
    assert rc == 0
    return out


def spmm_scale(X, ii, jj, avv, Y0) -> np.ndarray:
    """|Y0| + sum_e |a_e X[c_e,:]| in double."""
    lib = load()
    X, avv = (np.ascontiguousarray(x, dtype=np.float64) for x in (X, avv))
    S = np.abs(np.asarray(Y0, dtype=np.float64)).copy(order="C")
    ii, jj = _prep(ii, jj)
    rc = lib.oracle_spmm_scale_f64(X.shape[0], S.shape[0], X.shape[1], _p(X), ii.size, _p(ii),
                                   _p(jj), _p(avv), _p(S))
    assert rc == 0
    return S


def rel_err(got, ref, scale) -> float:
    """max |got - ref| / max(scale, |ref|); entries whose scale is 0 must match exactly."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    den = np.maximum(np.asarray(scale, dtype=np.float64), np.abs(ref))
    diff = np.abs(got - ref)
    if not np.all(np.isfinite(got)):
        return float("inf")
    zero = den == 0
    if np.any(diff[zero] != 0):
        return float("inf")
    if np.all(zero):
        return 0.0
    return float(np.max(diff[~zero] / den[~zero]))


def sddmm_rel_err(A, B, ii, jj, svv, got) -> float:
    """Error of `got` against the oracle run in the same real type."""
    ref = sddmm(A, B, ii, jj, svv)
    return rel_err(got, ref, sddmm_scale(A, B, ii, jj, svv))


def spmm_rel_err(X, ii, jj, avv, Y0, got) -> float:
    ref = spmm(X, ii, jj, avv, Y0)
    return rel_err(got, ref, spmm_scale(X, ii, jj, avv, Y0))


def sddmm_rel_err_exact(A, B, ii, jj, svv, got) -> float:
    """Error of `got` against the fp64 oracle on the same (exactly converted) inputs."""
    ref = sddmm(*(np.asarray(x, dtype=np.float64) for x in (A, B)), ii, jj,
                np.asarray(svv, dtype=np.float64))
    return rel_err(got, ref, sddmm_scale(A, B, ii, jj, svv))


def spmm_rel_err_exact(X, ii, jj, avv, Y0, got) -> float:
    ref = spmm(np.asarray(X, dtype=np.float64), ii, jj, np.asarray(avv, dtype=np.float64),
               np.asarray(Y0, dtype=np.float64))
    return rel_err(got, ref, spmm_scale(X, ii, jj, avv, Y0))
