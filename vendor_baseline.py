"""The vendor's sparse library on the same operands, for bench.py: rocSPARSE's
generic SpMM (CSR x row-major dense, every CSR algorithm it offers) and SDDMM
(dense x dense sampled by a CSR pattern), timed next to this library's kernels.

A measurement aid, not a dependency: nothing in the library or its tests uses
it, and bench.py leaves the object out when rocSPARSE cannot be loaded.
rocSPARSE's SDDMM computes alpha * (A B^T) on the pattern without the
element-wise scale by S.vv that SpKernels::sddmm applies (src/core_ops.cpp:18):
one multiply per entry less, the same memory traffic.
"""
import ctypes
import time

import numpy as np

# rocsparse-types.h
_OP_NONE, _BASE_ZERO, _I32 = 111, 0, 2
_F32, _F64 = 151, 152
_ROW, _COL = 0, 1
_STAGE_SIZE, _STAGE_PRE, _STAGE_RUN = 1, 2, 3
SPMM_ALGS = {"default": 0, "csr": 1, "csr_row_split": 4, "csr_nnz_split": 5, "csr_merge_path": 9}


class VendorError(RuntimeError):
    pass


def _load():
    # every call used here returns an int status, ctypes' default result type
    return ctypes.CDLL("librocsparse.so"), ctypes.CDLL("libamdhip64.so")


def _ok(status, what):
    if status != 0:
        raise VendorError(f"{what} returned {status}")


def time_rocsparse(ctx, w, dtype, dA, dB, dY, reps=10):
    """Times rocSPARSE on workload `w` with this context's resident panels dA (m x K),
    dB (n x K) and dY (m x K); w must be sorted by row.  Returns a dict of
    microseconds per call.  dY is overwritten."""
    from spcomm3d_amd import device

    rs, hip = _load()
    p = ctypes.c_void_p
    i64 = ctypes.c_int64
    real = np.dtype(np.float64 if device.dtype_code(dtype) == device.capi.F64 else np.float32)
    dt = _F64 if real == np.float64 else _F32
    m, n, k, nnz = w.nrows, w.ncols, w.k, w.nnz
    if np.any(np.diff(w.ii.astype(np.int64)) < 0):
        raise VendorError("the CSR view needs a pattern sorted by row")
    rowptr = np.zeros(m + 1, dtype=np.int64)
    np.add.at(rowptr, w.ii.astype(np.int64) + 1, 1)
    rowptr = np.cumsum(rowptr).astype(np.int32)

    def words(a):  # 32-bit words in a device buffer of this library
        v = ctx.vals(a.size, np.float32)
        v.upload(np.ascontiguousarray(a).view(np.float32))
        return v

    d_rp, d_ci = words(rowptr), words(w.jj.astype(np.int32))
    d_val = ctx.vals(nnz, real)
    d_val.upload(w.values(real))
    ctx.sync()

    handle, S, X, Y, A, Bt = p(), p(), p(), p(), p(), p()
    out = {"library": "rocSPARSE", "reps": reps, "spmm_us": {}, "note":
           "generic API, CSR int32, row-major dense; SDDMM without the scale by S.vv"}
    held = [d_rp, d_ci, d_val]
    try:
        _ok(rs.rocsparse_create_handle(ctypes.byref(handle)), "rocsparse_create_handle")
        _ok(rs.rocsparse_create_csr_descr(ctypes.byref(S), i64(m), i64(n), i64(nnz),
                                          p(d_rp.device_ptr()), p(d_ci.device_ptr()),
                                          p(d_val.device_ptr()), _I32, _I32, _BASE_ZERO, dt),
            "rocsparse_create_csr_descr")
        for desc, rows, cols, ld, buf, order in ((X, n, k, k, dB, _ROW), (Y, m, k, k, dY, _ROW),
                                                 (A, m, k, k, dA, _ROW), (Bt, k, n, k, dB, _COL)):
            _ok(rs.rocsparse_create_dnmat_descr(ctypes.byref(desc), i64(rows), i64(cols), i64(ld),
                                                p(buf.device_ptr()), dt, order),
                "rocsparse_create_dnmat_descr")
        one = (ctypes.c_double if dt == _F64 else ctypes.c_float)(1.0)
        zero = (ctypes.c_double if dt == _F64 else ctypes.c_float)(0.0)

        def timed(call):
            for _ in range(2):
                _ok(call(), "warm-up")
            _ok(hip.hipDeviceSynchronize(), "hipDeviceSynchronize")
            t0 = time.perf_counter()
            for _ in range(reps):
                _ok(call(), "timed call")
            _ok(hip.hipDeviceSynchronize(), "hipDeviceSynchronize")
            return 1e6 * (time.perf_counter() - t0) / reps

        for name, alg in SPMM_ALGS.items():
            size = ctypes.c_size_t(0)

            def spmm(stage, buf):
                return rs.rocsparse_spmm(handle, _OP_NONE, _OP_NONE, ctypes.byref(one), S, X,
                                         ctypes.byref(one), Y, dt, alg, stage, ctypes.byref(size), buf)

            if spmm(_STAGE_SIZE, None) != 0:
                continue  # not offered for this format
            scratch = ctx.vals(max(size.value // 4 + 1, 4), np.float32)
            held.append(scratch)
            sp = p(scratch.device_ptr())
            if spmm(_STAGE_PRE, sp) != 0:
                continue
            out["spmm_us"][name] = timed(lambda: spmm(_STAGE_RUN, sp))
        size = ctypes.c_size_t(0)
        args = (handle, _OP_NONE, _OP_NONE, ctypes.byref(one), A, Bt, ctypes.byref(zero), S, dt, 0)
        _ok(rs.rocsparse_sddmm_buffer_size(*args, ctypes.byref(size)), "rocsparse_sddmm_buffer_size")
        scratch = ctx.vals(max(size.value // 4 + 1, 4), np.float32)
        held.append(scratch)
        sp = p(scratch.device_ptr())
        _ok(rs.rocsparse_sddmm_preprocess(*args, sp), "rocsparse_sddmm_preprocess")
        out["sddmm_us"] = timed(lambda: rs.rocsparse_sddmm(*args, sp))
        if out["spmm_us"]:
            best = min(out["spmm_us"], key=out["spmm_us"].get)
            out["spmm_best"] = {"alg": best, "us": out["spmm_us"][best]}
    finally:
        hip.hipDeviceSynchronize()
        for desc, kill in ((S, rs.rocsparse_destroy_spmat_descr), (X, rs.rocsparse_destroy_dnmat_descr),
                           (Y, rs.rocsparse_destroy_dnmat_descr), (A, rs.rocsparse_destroy_dnmat_descr),
                           (Bt, rs.rocsparse_destroy_dnmat_descr)):
            if desc:
                kill(desc)
        if handle:
            rs.rocsparse_destroy_handle(handle)
        for h in held:
            h.close()
    return out
