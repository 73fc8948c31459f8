"""The pack / unpack copies either side of a sparse exchange
(SparseComm::copy_to_sendbuff / copy_from_recvbuff / SUM_from_recvbuff,
src/comm.hpp:90-103,166-189): oracle pinned on the CPU, HIP kernels checked
against it bit for bit on the GPU (they only move and add in a fixed order)."""
import ctypes
import os

import numpy as np
import pytest

from spcomm3d_amd import _capi as capi
from tests import _oracle as oracle


def oracle_rows(op, panel, rows, buf):
    lib = oracle.load()
    fn = getattr(lib, "oracle_rows_" + ("f64" if panel.dtype == np.float64 else "f32"))
    fn.restype = ctypes.c_int
    fn.argtypes = [ctypes.c_int, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_void_p,
                   ctypes.c_uint64, ctypes.c_void_p, ctypes.c_void_p]
    panel = np.array(panel, copy=True, order="C")
    buf = np.array(buf, copy=True, order="C")
    rows = np.ascontiguousarray(rows, dtype=np.uint32)
    rc = fn(op, panel.shape[0], panel.shape[1], panel.ctypes.data_as(ctypes.c_void_p), rows.size,
            rows.ctypes.data_as(ctypes.c_void_p), buf.ctypes.data_as(ctypes.c_void_p))
    if rc != 0:
        raise IndexError("row out of range")
    return panel, buf


def case(seed, m, k, n, dtype, repeats=True):
    rng = np.random.default_rng(seed)
    P = rng.uniform(-1, 1, (m, k)).astype(dtype)
    rows = (rng.integers(0, m, n) if repeats else rng.permutation(m)[:n]).astype(np.uint32)
    buf = rng.uniform(-1, 1, (n, k)).astype(dtype)
    return P, rows, buf


# ---- the oracle ----------------------------------------------------------------
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_oracle_rows_against_numpy(dtype):
    P, rows, buf = case(1, 40, 6, 100, dtype)
    _, b = oracle_rows(0, P, rows, buf)
    assert np.array_equal(b, P[rows])
    p, _ = oracle_rows(1, P, rows, buf)
    want = P.copy()
    for i, r in enumerate(rows):  # sequential: the last slot of a row wins
        want[r] = buf[i]
    assert np.array_equal(p, want)
    p, _ = oracle_rows(2, P, rows, buf)
    want = P.astype(np.float64)
    np.add.at(want, rows, buf.astype(np.float64))
    np.testing.assert_allclose(p, want, rtol=0, atol=1e-5 if dtype == np.float32 else 1e-13)
    # unpack(pack(P)) is the identity on distinct rows
    P2, rows2, _ = case(2, 30, 5, 30, dtype, repeats=False)
    _, b = oracle_rows(0, P2, rows2, np.zeros((30, 5), dtype))
    p, _ = oracle_rows(1, np.zeros_like(P2), rows2, b)
    assert np.array_equal(p, P2)
    # slots add in ascending order: (x + big) - big differs from x + (big - big) in floating point
    big = dtype(2 ** 30 if dtype == np.float32 else 2 ** 60)
    P3 = np.zeros((1, 1), dtype)
    b3 = np.array([[1.0], [big], [-big]], dtype)
    p, _ = oracle_rows(2, P3, np.zeros(3, np.uint32), b3)
    assert p[0, 0] == dtype(0)  # (0 + 1 + big) - big == 0 because 1 is absorbed
    with pytest.raises(IndexError):
        oracle_rows(0, P, np.array([40], np.uint32), buf[:1])


GOLDEN = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                              "rows_golden.npz"))
REF_ROWS = os.path.join(oracle.ORACLE_DIR, "_ref", "libref_rows.so")


@pytest.mark.parametrize("name", ["k1", "k6", "k64"])
def test_oracle_rows_against_the_reference_vectors(name):
    # tests/golden/rows_golden.npz: the reference's own SparseComm copies (src/comm.hpp:90-103,
    # 166-189) on seeded inputs with repeated rows; bit for bit
    g = {k: GOLDEN[f"{name}.{k}"] for k in ("P", "rows", "buf", "packed", "unpacked", "summed")}
    assert np.array_equal(oracle_rows(0, g["P"], g["rows"], g["buf"])[1], g["packed"])
    assert np.array_equal(oracle_rows(1, g["P"], g["rows"], g["buf"])[0], g["unpacked"])
    assert np.array_equal(oracle_rows(2, g["P"], g["rows"], g["buf"])[0], g["summed"])


@pytest.mark.skipif(not os.path.exists(REF_ROWS),
                    reason="oracle/_ref is only built where the reference is mounted")
@pytest.mark.parametrize("seed", [1, 2])
def test_oracle_rows_bit_exact_vs_live_reference_build(seed):
    lib = ctypes.CDLL(REF_ROWS)
    lib.ref_rows_f64.restype = ctypes.c_int
    lib.ref_rows_f64.argtypes = [ctypes.c_int, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_void_p,
                                 ctypes.c_uint64, ctypes.c_void_p, ctypes.c_void_p]
    P, rows, buf = case(seed, 200, 17, 900, np.float64)
    vp = lambda a: a.ctypes.data_as(ctypes.c_void_p)  # noqa: E731
    for op in (0, 1, 2):
        p, b = P.copy(), buf.copy()
        assert lib.ref_rows_f64(op, 200, 17, vp(p), rows.size, vp(rows), vp(b)) == 0
        op_, ob = oracle_rows(op, P, rows, buf)
        assert np.array_equal(op_, p) and np.array_equal(ob, b)


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["k1", "k6", "k64"])
def test_rows_kernels_match_the_reference_vectors(ctx, name):
    from spcomm3d_amd import device

    g = {k: GOLDEN[f"{name}.{k}"] for k in ("P", "rows", "buf", "packed", "unpacked", "summed")}
    k = g["P"].shape[1]
    rm = device.RowMap(ctx, g["P"].shape[0], g["rows"])
    dP, dB = ctx.panel_from(g["P"]), ctx.vals(g["rows"].size * k, np.float64)
    rm.pack(dP, dB)
    assert np.array_equal(dB.download().reshape(-1, k), g["packed"])
    dB.upload(g["buf"].ravel())
    rm.unpack(dP, dB)
    assert np.array_equal(dP.download(), g["unpacked"])
    dP.upload(g["P"])
    rm.unpack_sum(dP, dB)
    assert np.array_equal(dP.download(), g["summed"])


def test_rowmap_validation_needs_no_gpu():
    lib = capi.load()
    rows = np.array([0, 5, 2], dtype=np.uint32)
    h = ctypes.c_void_p()
    rc = lib.spc3d_rowmap_create(None, 5, 3, rows.ctypes.data_as(ctypes.c_void_p), ctypes.byref(h))
    assert rc == capi.ERR_BAD_INDEX and b"slot 1" in lib.spc3d_last_error()
    rc = lib.spc3d_rowmap_create(None, 6, 3, None, ctypes.byref(h))
    assert rc == capi.ERR_INVALID_ARG


# ---- the kernels ---------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("k", [1, 3, 4, 32, 64, 100, 256])
def test_rows_kernels_match_oracle_bitwise(ctx, dtype, k):
    from spcomm3d_amd import device

    P, rows, buf = case(10 + k, 500, k, 1700, dtype)
    rm = device.RowMap(ctx, 500, rows)
    dP = ctx.panel_from(P)
    dB = ctx.vals(rows.size * k, dtype)
    rm.pack(dP, dB)
    assert np.array_equal(dB.download().reshape(-1, k), oracle_rows(0, P, rows, buf)[1])
    dB.upload(buf.ravel())
    rm.unpack(dP, dB)
    assert np.array_equal(dP.download(), oracle_rows(1, P, rows, buf)[0])
    dP.upload(P)
    rm.unpack_sum(dP, dB)
    assert np.array_equal(dP.download(), oracle_rows(2, P, rows, buf)[0])  # same order, same bits


@pytest.mark.gpu
def test_rows_edge_cases_and_refusals(ctx):
    from spcomm3d_amd import device

    P = np.arange(12, dtype=np.float64).reshape(4, 3)
    dP = ctx.panel_from(P)
    empty = device.RowMap(ctx, 4, np.zeros(0, np.uint32))
    dB = ctx.vals(0, np.float64)
    empty.pack(dP, dB)
    empty.unpack_sum(dP, dB)
    assert np.array_equal(dP.download(), P)
    with pytest.raises(IndexError):
        device.RowMap(ctx, 4, np.array([4], np.uint32))
    rm = device.RowMap(ctx, 4, np.array([1, 1, 3], np.uint32))
    with pytest.raises(capi.Spc3dError):
        rm.pack(dP, ctx.vals(8, np.float64))        # buffer too short
    with pytest.raises(capi.Spc3dError):
        rm.pack(dP, ctx.vals(9, np.float32))        # dtype
    with pytest.raises(capi.Spc3dError):
        rm.pack(ctx.panel_from(P[:3].copy()), ctx.vals(9, np.float64))  # panel too short


@pytest.mark.gpu
def test_expand_then_reduce_round_trip_at_size(ctx):
    # 1M slots of K=64 fp32 rows drawn from a 2^20-row panel: pack, zero, scatter-add back
    from spcomm3d_amd import device

    m, k, n = 1 << 20, 64, 1 << 20
    rng = np.random.default_rng(3)
    rows = rng.integers(0, m, n).astype(np.uint32)
    P = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    rm = device.RowMap(ctx, m, rows)
    dP, dB = ctx.panel_from(P), ctx.vals(n * k, np.float32)
    rm.pack(dP, dB)
    dP.fill(0.0)
    rm.unpack_sum(dP, dB)
    got = dP.download()
    mult = np.bincount(rows, minlength=m).astype(np.float32)
    # a row packed c times comes back as c * row, added one at a time from zero
    want = np.zeros_like(P)
    for c in range(1, int(mult.max()) + 1):
        sel = mult >= c
        want[sel] += P[sel]
    assert np.array_equal(got, want)
