"""CPU-only checks of the C-ABI library: it loads, exports every declared
symbol, validates patterns on the host, builds correct plans, and fails loudly
(no fallback) when there is no GPU.  No kernel is launched here."""
import ctypes
import os

import numpy as np
import pytest

from spcomm3d_amd import _capi as capi
from spcomm3d_amd import device
from spcomm3d_amd import workloads as W

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
def _check_plan(nrows, ncols, ii, jj, **opts):
    P = device.plan_build_host(nrows, ncols, ii, jj, "f32", **opts)
    info, col, perm, segs, splits = P["info"], P["col"], P["perm"], P["segs"], P["splits"]
    nnz = ii.size
    assert info.nnz == nnz
    if opts.get("seg_max"):
        assert info.seg_max == opts["seg_max"]
    # perm is a permutation; kernel order is grouped by row
    assert np.array_equal(np.sort(perm), np.arange(nnz, dtype=np.uint32))
    assert np.array_equal(col, jj[perm])
    rows_k = ii[perm]
    assert np.all(np.diff(rows_k.astype(np.int64)) >= 0)
    unsorted = bool(np.any(np.diff(ii.astype(np.int64)) < 0)) and not opts.get("keep_entry_order")
    assert info.entries_by_column == int(unsorted)
    if info.nqueues == 1:
        same = rows_k[1:] == rows_k[:-1]
        if not unsorted:  # no slicing: the caller's order survives inside every row
            assert np.all(perm[1:][same] > perm[:-1][same])
        else:  # rows that arrive unsorted: by column inside a row, equal columns in caller's order
            c = col.astype(np.int64)
            assert np.all((c[1:] >= c[:-1])[same])
            tie = same & (c[1:] == c[:-1])
            assert np.all(perm[1:][tie] > perm[:-1][tie])
    assert bool(info.order_is_identity) == bool(np.array_equal(perm, np.arange(nnz)))
    assert info.rows_touched == np.unique(ii).size and info.cols_touched == np.unique(jj).size
    assert info.max_row_nnz == (np.bincount(ii).max() if nnz else 0)
    # real segments tile [0, nnz) exactly once and stay inside one row; the rest is padding
    assert segs.shape[0] == info.nsegments_padded
    real = segs[segs[:, 2] > 0]
    assert real.shape[0] == info.nsegments
    assert np.all(segs[segs[:, 2] == 0][:, 3] == WHOLE)
    cover = np.zeros(nnz, dtype=np.int32)
    for row, start, ln, slot in real:
        assert 1 <= ln <= info.seg_max
        cover[start:start + ln] += 1
        assert np.all(rows_k[start:start + ln] == row)
        if info.nqueues == 1:
            continue
    assert np.all(cover == 1)
    # inside each queue: longest first; ties keep position order
    chunk = np.arange(segs.shape[0]) // 64
    for q in range(info.nqueues):
        mine = segs[(chunk % info.nqueues) == q]
        mine = mine[mine[:, 2] > 0]
        lens = mine[:, 2].astype(np.int64)
        assert np.all(np.diff(lens) <= 0)
        if info.nqueues == 1:
            tie = lens[1:] == lens[:-1]
            assert np.all((mine[1:, 1] > mine[:-1, 1])[tie])
    if info.nqueues == 8:
        assert segs.shape[0] % (8 * 64) == 0
    # cut rows: slots are a partition of [0, npartial_slots), whole rows carry the marker
    nseg_of_row = np.bincount(real[:, 0], minlength=nrows)
    cut_rows = np.flatnonzero(nseg_of_row > 1)
    assert np.array_equal(np.sort(splits[:, 0]), cut_rows)
    used = np.zeros(info.npartial_slots, dtype=np.int32)
    for row, first, n in splits:
        mine = real[real[:, 0] == row]
        assert mine.shape[0] == n
        assert np.array_equal(np.sort(mine[:, 3]), np.arange(first, first + n))
        used[first:first + n] += 1
    assert np.all(used == 1)
    whole = real[~np.isin(real[:, 0], cut_rows)]
    assert np.all(whole[:, 3] == WHOLE)
    if info.nqueues == 1:  # rows are cut only when longer than seg_max, into balanced pieces
        counts = np.bincount(ii, minlength=nrows) if nnz else np.zeros(nrows, dtype=np.int64)
        assert np.array_equal(cut_rows, np.flatnonzero(counts > info.seg_max))
        for row in cut_rows:
            mine = real[real[:, 0] == row]
            assert mine.shape[0] == -(-counts[row] // info.seg_max)
            assert mine[:, 2].max() - mine[:, 2].min() <= 1
    return P


@pytest.mark.parametrize("seg_max", [None, 4, 7, 64])
def test_plan_random_unsorted_with_duplicates(seg_max):
    rng = np.random.default_rng(3)
    ii = rng.integers(0, 50, 900).astype(np.uint32)
    jj = rng.integers(0, 70, 900).astype(np.uint32)
    ii[:300] = 7  # a hub row
    o = rng.permutation(900)
    _check_plan(50, 70, ii[o], jj[o], seg_max=seg_max)
    _check_plan(50, 70, ii[o], jj[o], seg_max=seg_max, keep_entry_order=True)


def test_plan_default_seg_max_follows_nnz():
    e = np.zeros(0, dtype=np.uint32)
    assert device.plan_build_host(5, 5, e, e)["info"].seg_max == 64
    w = W.rmat(14, 16, 64)
    assert device.plan_build_host(w.nrows, w.ncols, w.ii, w.jj)["info"].seg_max == 64
    w = W.rmat(17, 16, 64)
    s = device.plan_build_host(w.nrows, w.ncols, w.ii, w.jj)["info"].seg_max
    assert s == 1 << int(np.log2(w.nnz / 2048)) and 64 <= s <= 2048
    # narrow dense rows put more segments on a wavefront: the cap comes down with k_hint
    n = 2048 * 2048
    ii = (np.arange(n, dtype=np.uint32) // 4200).astype(np.uint32)
    jj = (np.arange(n, dtype=np.uint32) % 777).astype(np.uint32)
    def seg_max(**kw):
        return device.plan_build_host(1000, 777, ii, jj, **kw)["info"].seg_max
    assert seg_max() == 2048 and seg_max(dtype="f32", k_hint=64) == 2048
    assert seg_max(dtype="f64", k_hint=16) == 1024 and seg_max(dtype="f32", k_hint=32) == 1024
    assert seg_max(dtype="f32", k_hint=16) == 512 and seg_max(dtype="f32", k_hint=1) == 512
    assert seg_max(dtype="f32", k_hint=16, seg_max=2048) == 2048  # an explicit value wins


def test_plan_sorted_input_is_identity_and_empty_rows_are_skipped():
    ii = np.array([1, 1, 4, 4, 4, 9], dtype=np.uint32)
    jj = np.array([5, 2, 0, 0, 3, 1], dtype=np.uint32)
    P = _check_plan(12, 6, ii, jj)
    assert P["info"].order_is_identity == 1
    assert P["info"].nsegments == 3 and P["info"].nsplit_rows == 0
    assert sorted(P["segs"][:, 0]) == [1, 4, 9]


def test_plan_empty_and_single():
    e = np.zeros(0, dtype=np.uint32)
    P = device.plan_build_host(5, 5, e, e)
    assert P["info"].nsegments == 0 and P["info"].nnz == 0 and P["info"].order_is_identity == 1
    P = _check_plan(1, 1, np.zeros(1, np.uint32), np.zeros(1, np.uint32))
    assert P["info"].nsegments == 1


def test_plan_xcd_slicing_on_skewed_pattern():
    w = W.rmat(15, 16, 64).shuffled()
    # a small L2 share so that the 2^15-column panel does not fit and slicing engages
    P = _check_plan(w.nrows, w.ncols, w.ii, w.jj, xcd_slices=8, l2_hot_bytes=64 * 1024,
                    hub_min=32, seg_max=256)
    info, segs = P["info"], P["segs"]
    assert info.nqueues == 8 and info.hub_rows > 0 and 0 < info.hot_cols < info.cols_touched
    assert 0.2 * info.nnz < info.hot_entries <= info.nnz
    # the eight queues carry nearly the same number of entries
    chunk = np.arange(segs.shape[0]) // 64
    load = np.array([segs[(chunk % 8) == q][:, 2].sum() for q in range(8)], dtype=np.int64)
    assert load.max() - load.min() <= 0.02 * load.mean() + 256
    # the rows arrive unsorted: inside each piece the entries are ordered by column
    # (R-MAT patterns hold no duplicates), and with keep_entry_order in the caller's order
    perm, rows_k, col = P["perm"], w.ii[P["perm"]], P["col"]
    assert info.entries_by_column == 1
    for row, start, ln, slot in segs[segs[:, 2] > 1][:200]:
        assert np.all(np.diff(col[start:start + ln].astype(np.int64)) > 0)
    K = _check_plan(w.nrows, w.ncols, w.ii, w.jj, xcd_slices=8, l2_hot_bytes=64 * 1024,
                    hub_min=32, seg_max=256, keep_entry_order=True)
    assert K["info"].entries_by_column == 0
    for row, start, ln, slot in K["segs"][K["segs"][:, 2] > 1][:200]:
        assert np.all(np.diff(K["perm"][start:start + ln].astype(np.int64)) > 0)
    # every entry of one hub piece with a slice column sits in that slice's queue:
    # same column -> same queue, wherever it appears in hub rows
    counts = np.bincount(w.ii, minlength=w.nrows)
    qcol = {}
    for idx in np.flatnonzero(segs[:, 2] > 0):
        row, start, ln, slot = segs[idx]
        if counts[row] < 32 or slot == WHOLE:
            continue
        q = (idx // 64) % 8
        for c in P["col"][start:start + ln][:4]:
            qcol.setdefault(int(c), set()).add(int(q))
    sliced = [c for c, qs in qcol.items() if len(qs) == 1]
    assert len(sliced) > 0.3 * len(qcol)
    # rows under the hub threshold go, where there is room, to the queue of the slice most of
    # their sliced entries belong to: of their entries in columns with a queue of their own,
    # far more than the eighth that chance gives sit in that queue, and none of that without
    own = np.full(w.ncols, -1, dtype=np.int64)
    for c in sliced:
        own[c] = next(iter(qcol[c]))

    def at_home(plan):
        sg, cols = plan["segs"], plan["col"]
        home = total = 0
        for idx in np.flatnonzero(sg[:, 2] > 0):
            row, start, ln, slot = sg[idx]
            if counts[row] >= 32:
                continue
            o = own[cols[start:start + ln]]
            total += int((o >= 0).sum())
            home += int((o == (idx // 64) % 8).sum())
        return home / max(total, 1)

    F = _check_plan(w.nrows, w.ncols, w.ii, w.jj, xcd_slices=8, l2_hot_bytes=64 * 1024,
                    hub_min=32, seg_max=256, slice_affinity=False)
    assert at_home(P) > 0.25 and at_home(F) < 0.16
    fl = np.array([F["segs"][(np.arange(F["segs"].shape[0]) // 64 % 8) == q][:, 2].sum()
                   for q in range(8)], dtype=np.int64)
    assert fl.max() - fl.min() <= 0.02 * fl.mean() + 256


def test_plan_slicing_stays_off_for_uniform_columns():
    w = W.erdos_renyi(4096, 16, 32)
    P = _check_plan(w.nrows, w.ncols, w.ii, w.jj, xcd_slices=8, l2_hot_bytes=16 * 1024)
    assert P["info"].nqueues == 1 and P["info"].hot_cols == 0 and P["info"].order_is_identity == 1


def test_plan_build_host_rejects_bad_arguments():
    lib = capi.load()
    ii = np.array([0, 1, 1], dtype=np.uint32)
    jj = np.array([0, 1, 5], dtype=np.uint32)
    with pytest.raises(capi.BadIndexError):
        device.plan_build_host(2, 2, ii, jj)
    info = capi.PlanInfo()
    segs = np.zeros(4, dtype=np.uint32)
    vp = lambda a: a.ctypes.data_as(ctypes.c_void_p)  # noqa: E731
    rc = lib.spc3d_plan_build_host(capi.F32, 2, 6, 3, vp(ii), vp(jj), None, ctypes.byref(info),
                                   None, None, vp(segs), 1, None, 0)
    assert rc == capi.ERR_SIZE_MISMATCH and info.nsegments == 2
    with pytest.raises(capi.Spc3dError):
        device.plan_build_host(2, 6, ii, jj, xcd_slices=4)
    o = capi.PlanOpts()
    o.reserved[0] = 7
    rc = lib.spc3d_plan_build_host(capi.F32, 2, 6, 3, vp(ii), vp(jj), ctypes.byref(o),
                                   ctypes.byref(info), None, None, None, 0, None, 0)
    assert rc == capi.ERR_INVALID_ARG
    # row tiles: 0, 1, 2 are the modes; the host builder makes none, so asking it for them is an error
    for field, value in (("sweep", 3), ("flags", 64)):
        o = capi.PlanOpts()
        setattr(o, field, value)
        rc = lib.spc3d_plan_build_host(capi.F32, 2, 6, 3, vp(ii), vp(jj), ctypes.byref(o),
                                       ctypes.byref(info), None, None, None, 0, None, 0)
        assert rc == capi.ERR_INVALID_ARG, field
    o = capi.PlanOpts()
    o.sweep, o.builder = 2, 1
    rc = lib.spc3d_plan_build_host(capi.F32, 2, 6, 3, vp(ii), vp(jj), ctypes.byref(o),
                                   ctypes.byref(info), None, None, None, 0, None, 0)
    assert rc == capi.ERR_INVALID_ARG
    o = capi.PlanOpts()
    o.sweep, o.sweep_min_row, o.flags = 1, 5, capi.PLAN_SWEEP_STAGED  # valid, and without effect here
    rc = lib.spc3d_plan_build_host(capi.F32, 2, 6, 3, vp(ii), vp(jj), ctypes.byref(o),
                                   ctypes.byref(info), None, None, None, 0, None, 0)
    assert rc == capi.OK and info.sweep_entries == 0 and info.sweep_tiles == 0


def test_the_python_mirrors_of_the_structs_have_the_headers_layout():
    """sizeof and the offsets of the last fields, against a C program compiled from the header."""
    import subprocess
    import tempfile

    src = r"""
#include <stdio.h>
#include <stddef.h>
#include "spcomm3d_hip.h"
int main(void) {
    printf("%zu %zu %zu %zu %zu %zu\n", sizeof(spc3d_plan_opts), offsetof(spc3d_plan_opts, sweep_min_row),
           sizeof(spc3d_plan_info), offsetof(spc3d_plan_info, sweep_k), sizeof(spc3d_ctx_opts),
           offsetof(spc3d_plan_info, device_bytes));
    return 0;
}
"""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    with tempfile.TemporaryDirectory() as d:
        c = os.path.join(d, "layout.c")
        with open(c, "w") as f:
            f.write(src)
        exe = os.path.join(d, "layout")
        subprocess.run(["gcc", "-I", os.path.join(root, "include"), "-o", exe, c], check=True)
        got = [int(x) for x in subprocess.run([exe], capture_output=True, text=True,
                                              check=True).stdout.split()]
    want = [ctypes.sizeof(capi.PlanOpts), capi.PlanOpts.sweep_min_row.offset,
            ctypes.sizeof(capi.PlanInfo), capi.PlanInfo.sweep_k.offset,
            ctypes.sizeof(capi.CtxOpts), capi.PlanInfo.device_bytes.offset]
    assert got == want


def test_context_options_are_validated_before_any_device_is_touched():
    lib = capi.load()
    h = ctypes.c_void_p()
    o = capi.CtxOpts()
    o.flags = 4  # unknown bit
    assert lib.spc3d_ctx_create_ex(0, ctypes.byref(o), ctypes.byref(h)) == capi.ERR_INVALID_ARG
    o = capi.CtxOpts()
    o.reserved[2] = 1
    assert lib.spc3d_ctx_create_ex(0, ctypes.byref(o), ctypes.byref(h)) == capi.ERR_INVALID_ARG
    o = capi.CtxOpts()
    o.host_threads = 1000
    assert lib.spc3d_ctx_create_ex(0, ctypes.byref(o), ctypes.byref(h)) == capi.ERR_INVALID_ARG
    assert not h.value


def test_kernel_variant_for_every_kind_of_row_width():
    lib = capi.load()
    def v(dtype, k):
        r = lib.spc3d_kernel_variant(dtype, k)
        return r.decode() if r is not None else None
    F32, F64 = 0, 1
    # rows that fill a lane shape exactly: a power of two of 16-byte vectors, 1, 2 or 4 per lane
    assert v(F32, 64) == "seg<f32,LPR=16,VPL=1>" and v(F64, 64) == "seg<f64,LPR=32,VPL=1>"
    assert v(F32, 16) == "seg<f32,LPR=4,VPL=1>" and v(F64, 32) == "seg<f64,LPR=16,VPL=1>"
    assert v(F32, 512) == "seg<f32,LPR=64,VPL=2>" and v(F64, 512) == "seg<f64,LPR=64,VPL=4>"
    # whole vectors that leave lanes idle: clamped loads up to 16 vectors, masked loads above
    assert v(F32, 4) == "seg<f32,LPR=4,VPL=1,odd>" and v(F32, 48) == "seg<f32,LPR=16,VPL=1,odd>"
    assert v(F32, 100) == "seg<f32,LPR=32,VPL=1,ragged>" and v(F64, 100) == "seg<f64,LPR=64,VPL=1,ragged>"
    assert v(F32, 300) == "seg<f32,LPR=64,VPL=2,ragged>" and v(F64, 300) == "seg<f64,LPR=64,VPL=4,ragged>"
    # rows that end inside a vector
    assert v(F32, 50) == "seg<f32,LPR=16,VPL=1,odd>" and v(F32, 65) == "seg<f32,LPR=32,VPL=1,odd>"
    assert v(F64, 63) == "seg<f64,LPR=32,VPL=1,odd>" and v(F32, 1023) == "seg<f32,LPR=64,VPL=4,odd>"
    # rows shorter than a vector, rows over 4 KiB
    assert v(F32, 1) == v(F32, 3) == "seg<f32,LPR=4,VPL=1,thin>" and v(F64, 1) == "seg<f64,LPR=4,VPL=1,thin>"
    assert v(F64, 2) == "seg<f64,LPR=4,VPL=1,odd>"
    assert v(F32, 1024) == "seg<f32,LPR=64,VPL=4>" and "per 4 KiB slice" in v(F32, 1025)
    assert "per 4 KiB slice" in v(F64, 513) and v(F32, 0) == "none (no columns)"
    assert v(7, 64) is None



def test_an_absurd_seg_max_is_brought_down():
    """The builders keep one counter per segment length: a request of 2^30 must not
    turn into a 4 GiB array."""
    e = np.arange(5, dtype=np.uint32)
    info = device.plan_build_host(5, 5, e, e, seg_max=1 << 30)["info"]
    assert info.seg_max == 1 << 20 and info.nsegments == 5
