"""CPU-only checks of the C-ABI library: it loads, exports every declared
symbol, validates patterns on the host, builds correct plans, and fails loudly
(no fallback) when there is no GPU.  No kernel is launched here."""
import ctypes

import numpy as np
import pytest

from spcomm3d_amd import _capi as capi
from spcomm3d_amd import device

WHOLE = 0xFFFFFFFF


def test_library_exports_every_declared_symbol():
    lib = capi.load()
    names = capi.header_symbols()
    assert len(names) >= 35
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/spcomm3d_hip.h but not exported"
    # and the binding table covers the header exactly
    assert sorted(capi.SIGNATURES) == names


def test_version_and_status_names():
    lib = capi.load()
    assert b"gfx950" in lib.spc3d_version()
    assert lib.spc3d_status_name(0) == b"SPC3D_OK"
    assert lib.spc3d_status_name(2) == b"SPC3D_ERR_BAD_INDEX"
    assert lib.spc3d_status_name(99) == b"SPC3D_ERR_UNKNOWN"


def test_validate_accepts_good_and_names_first_bad_entry():
    ii = np.array([0, 2, 1, 2], dtype=np.uint32)
    jj = np.array([1, 0, 3, 3], dtype=np.uint32)
    device.coo_validate(3, 4, ii, jj)
    with pytest.raises(capi.BadIndexError) as e:
        device.coo_validate(3, 3, ii, jj)  # column 3 is out of range
    assert "entry 2" in str(e.value) and "(1, 3)" in str(e.value)
    with pytest.raises(IndexError):  # the reference throws std::out_of_range here
        device.coo_validate(2, 4, ii, jj)
    device.coo_validate(0, 0, np.zeros(0, np.uint32), np.zeros(0, np.uint32))


def test_null_pointers_are_invalid_arg_not_crashes():
    lib = capi.load()
    assert lib.spc3d_coo_validate(3, 3, 5, None, None) == capi.ERR_INVALID_ARG
    assert lib.spc3d_device_count(None) == capi.ERR_INVALID_ARG
    assert lib.spc3d_ctx_create(0, None) == capi.ERR_INVALID_ARG
    assert lib.spc3d_ctx_destroy(None) == capi.ERR_INVALID_ARG
    assert lib.spc3d_panel_upload(None, None) == capi.ERR_INVALID_ARG
    assert lib.spc3d_sddmm(None, None, None, None, None) == capi.ERR_INVALID_ARG
    assert lib.spc3d_spmm(None, None, None, None) == capi.ERR_INVALID_ARG
    h = ctypes.c_void_p()
    assert lib.spc3d_panel_create(None, 0, 4, 4, ctypes.byref(h)) == capi.ERR_INVALID_ARG
    assert lib.spc3d_last_error() != b""


def test_bad_pattern_is_reported_before_any_device_is_needed():
    lib = capi.load()
    ii = np.array([0, 9], dtype=np.uint32)
    jj = np.array([0, 0], dtype=np.uint32)
    h = ctypes.c_void_p()
    rc = lib.spc3d_plan_create(None, capi.F64, 4, 4, 2, ii.ctypes.data_as(ctypes.c_void_p),
                               jj.ctypes.data_as(ctypes.c_void_p), None, ctypes.byref(h))
    assert rc == capi.ERR_BAD_INDEX
    rc = lib.spc3d_sddmm_host(None, capi.F64, 4, 4, 2, None, None, 2,
                              ii.ctypes.data_as(ctypes.c_void_p),
                              jj.ctypes.data_as(ctypes.c_void_p),
                              ii.ctypes.data_as(ctypes.c_void_p),
                              ii.ctypes.data_as(ctypes.c_void_p))
    assert rc == capi.ERR_BAD_INDEX


@pytest.mark.skipif(capi.device_count() > 0, reason="checks the no-GPU behaviour")
def test_no_device_fails_loudly_without_fallback():
    with pytest.raises(capi.Spc3dError) as e:
        device.Context(0)
    assert e.value.status == capi.ERR_NO_DEVICE


# ---- host plan builder --------------------------------------------------------
def _check_plan(nrows, ncols, ii, jj, seg_max):
    P = device.plan_build_host(nrows, ncols, ii, jj, seg_max)
    info, col, perm, segs, splits = P["info"], P["col"], P["perm"], P["segs"], P["splits"]
    nnz = ii.size
    assert info.nnz == nnz and info.seg_max == (seg_max or 128)
    # perm is a permutation; kernel order is grouped by row, stable within a row
    assert np.array_equal(np.sort(perm), np.arange(nnz, dtype=np.uint32))
    assert np.array_equal(col, jj[perm])
    rows_k = ii[perm]
    assert np.all(np.diff(rows_k.astype(np.int64)) >= 0)
    same = rows_k[1:] == rows_k[:-1]
    assert np.all(perm[1:][same] > perm[:-1][same]), "caller's order must survive inside a row"
    assert bool(info.order_is_identity) == bool(np.array_equal(perm, np.arange(nnz)))
    assert info.rows_touched == np.unique(ii).size and info.cols_touched == np.unique(jj).size
    assert info.max_row_nnz == (np.bincount(ii).max() if nnz else 0)
    # segments tile [0, nnz) exactly once and stay inside one row
    assert segs.shape[0] == info.nsegments
    cover = np.zeros(nnz, dtype=np.int32)
    for row, start, ln, slot in segs:
        assert 1 <= ln <= info.seg_max
        cover[start:start + ln] += 1
        assert np.all(rows_k[start:start + ln] == row)
    assert np.all(cover == 1)
    # longest first; ties keep row order
    lens = segs[:, 2].astype(np.int64)
    assert np.all(np.diff(lens) <= 0)
    tie = lens[1:] == lens[:-1]
    assert np.all((segs[1:, 1] > segs[:-1, 1])[tie])
    # cut rows: slots are a partition of [0, npartial_slots), whole rows carry the marker
    counts = np.bincount(ii, minlength=nrows) if nnz else np.zeros(nrows, dtype=np.int64)
    cut_rows = np.flatnonzero(counts > info.seg_max)
    assert np.array_equal(np.sort(splits[:, 0]), cut_rows)
    used = np.zeros(info.npartial_slots, dtype=np.int32)
    for row, first, n in splits:
        mine = segs[(segs[:, 0] == row)]
        assert mine.shape[0] == n and n == -(-counts[row] // info.seg_max)
        assert np.array_equal(np.sort(mine[:, 3]), np.arange(first, first + n))
        assert mine[:, 2].max() - mine[:, 2].min() <= 1  # balanced pieces
        used[first:first + n] += 1
    assert np.all(used == 1)
    whole = segs[~np.isin(segs[:, 0], cut_rows)]
    assert np.all(whole[:, 3] == WHOLE)
    return P


@pytest.mark.parametrize("seg_max", [0, 4, 7, 64])
def test_plan_random_unsorted_with_duplicates(seg_max):
    rng = np.random.default_rng(3)
    ii = rng.integers(0, 50, 900).astype(np.uint32)
    jj = rng.integers(0, 70, 900).astype(np.uint32)
    ii[:300] = 7  # a hub row
    o = rng.permutation(900)
    _check_plan(50, 70, ii[o], jj[o], seg_max)


def test_plan_sorted_input_is_identity_and_empty_rows_are_skipped():
    ii = np.array([1, 1, 4, 4, 4, 9], dtype=np.uint32)
    jj = np.array([5, 2, 0, 0, 3, 1], dtype=np.uint32)
    P = _check_plan(12, 6, ii, jj, 0)
    assert P["info"].order_is_identity == 1
    assert P["info"].nsegments == 3 and P["info"].nsplit_rows == 0
    assert sorted(P["segs"][:, 0]) == [1, 4, 9]


def test_plan_empty_and_single():
    e = np.zeros(0, dtype=np.uint32)
    P = device.plan_build_host(5, 5, e, e)
    assert P["info"].nsegments == 0 and P["info"].nnz == 0 and P["info"].order_is_identity == 1
    P = _check_plan(1, 1, np.zeros(1, np.uint32), np.zeros(1, np.uint32), 0)
    assert P["info"].nsegments == 1


def test_plan_build_host_rejects_bad_index_and_small_capacity():
    lib = capi.load()
    ii = np.array([0, 1, 1], dtype=np.uint32)
    jj = np.array([0, 1, 5], dtype=np.uint32)
    with pytest.raises(capi.BadIndexError):
        device.plan_build_host(2, 2, ii, jj)
    info = capi.PlanInfo()
    segs = np.zeros(4, dtype=np.uint32)
    vp = lambda a: a.ctypes.data_as(ctypes.c_void_p)  # noqa: E731
    rc = lib.spc3d_plan_build_host(2, 6, 3, vp(ii), vp(jj), 0, ctypes.byref(info), None, None,
                                   vp(segs), 1, None, 0)
    assert rc == capi.ERR_SIZE_MISMATCH and info.nsegments == 2
