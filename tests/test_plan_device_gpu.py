"""The plan built on the GPU (histograms, scans, stable radix sorts) against the
plan built by the host builder: the same arrays bit for bit (index work, so no
tolerance), for every layout the host builder produces.  The host builder
itself is checked without a GPU in test_capi_host.py."""
import ctypes
import os

import numpy as np
import pytest

from spcomm3d_amd import _capi as capi
from spcomm3d_amd import device
from spcomm3d_amd import workloads as W

pytestmark = pytest.mark.gpu
GOLDEN_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                           "core_ops_golden.npz")

# how SDDMM's results are stored is decided on the device, after either builder: the
# host-only build leaves these 0
INFO_FIELDS = [name for name, _ in capi.PlanInfo._fields_
               if name not in ("sddmm_by_column", "staged_entries", "positions_by_segment",
                           "two_pass_results", "device_bytes")]


def assert_same_plan(dev: dict, host: dict):
    for f in INFO_FIELDS:
        assert getattr(dev["info"], f) == getattr(host["info"], f), f
    for k in ("col", "perm", "segs", "splits"):
        assert dev[k].shape == host[k].shape, k
        assert np.array_equal(dev[k], host[k]), k


def both(ctx, nrows, ncols, ii, jj, **opts):
    host = device.plan_build_host(nrows, ncols, ii, jj, dtype="f32", **opts)
    S = ctx.plan(nrows, ncols, ii, jj, dtype=np.float32, builder="device", **opts)
    dev = S.download()
    S.close()
    assert_same_plan(dev, host)
    return host


def hub_case(seed, m, n, nnz, hub):
    rng = np.random.default_rng(seed)
    ii = rng.integers(0, m, nnz).astype(np.uint32)
    jj = rng.integers(0, n, nnz).astype(np.uint32)
    ii[:hub] = m // 3
    if nnz > 8:
        ii[-3:], jj[-3:] = ii[:3], jj[:3]  # duplicates
    o = rng.permutation(nnz)
    return ii[o], jj[o]


@pytest.mark.parametrize("seg_max", [None, 1, 4, 7, 64, 1000])
def test_random_unsorted_with_hub_and_duplicates(ctx, seg_max):
    ii, jj = hub_case(3, 50, 70, 900, 300)
    P = both(ctx, 50, 70, ii, jj, seg_max=seg_max)
    assert P["info"].order_is_identity == 0


def test_sorted_input_keeps_identity_and_skips_empty_rows(ctx):
    ii = np.array([1, 1, 4, 4, 4, 9], dtype=np.uint32)
    jj = np.array([5, 2, 0, 0, 3, 1], dtype=np.uint32)
    P = both(ctx, 12, 6, ii, jj)
    assert P["info"].order_is_identity == 1 and P["info"].nsegments == 3


@pytest.mark.parametrize("nnz", [0, 1, 2, 63, 64, 65])
def test_tiny_patterns(ctx, nnz):
    rng = np.random.default_rng(nnz)
    ii = rng.integers(0, 5, nnz).astype(np.uint32)
    jj = rng.integers(0, 9, nnz).astype(np.uint32)
    both(ctx, 5, 9, ii, jj)


def test_one_row_and_one_column(ctx):
    n = 5000
    z = np.zeros(n, dtype=np.uint32)
    c = np.arange(n, dtype=np.uint32)
    both(ctx, 1, n, z, c, seg_max=64)          # one row holding everything
    both(ctx, n, 1, c[::-1].copy(), z)          # one column, rows in descending order


@pytest.mark.parametrize("shuffled", [False, True])
def test_sliced_layout_on_skewed_pattern(ctx, shuffled):
    w = W.rmat(15, 16, 64)
    if shuffled:
        w = w.shuffled()
    P = both(ctx, w.nrows, w.ncols, w.ii, w.jj, xcd_slices=8, l2_hot_bytes=64 * 1024, hub_min=32,
             seg_max=256)
    assert P["info"].nqueues == 8 and P["info"].hub_rows > 0 and P["info"].nsplit_rows > 0
    # free segments dealt by rank alone
    Q = both(ctx, w.nrows, w.ncols, w.ii, w.jj, xcd_slices=8, l2_hot_bytes=64 * 1024, hub_min=32,
             seg_max=256, slice_affinity=False)
    assert Q["info"].nqueues == 8 and not np.array_equal(Q["segs"], P["segs"])
    # the same pattern with slicing switched off
    P = both(ctx, w.nrows, w.ncols, w.ii, w.jj, xcd_slices=1, seg_max=256)
    assert P["info"].nqueues == 1


def test_sliced_layout_with_64_bit_sort_keys(ctx):
    # row ids above 2^28 leave no room for the 4 group bits in a 32-bit key
    w = W.rmat(13, 16, 64).shuffled()
    nrows = 2 ** 28 + 10
    ii = (w.ii.astype(np.uint64) * 300007 % nrows).astype(np.uint32)
    P = both(ctx, nrows, w.ncols, ii, w.jj, xcd_slices=8, l2_hot_bytes=16 * 1024,
             hub_min=16, seg_max=128)
    assert P["info"].nqueues == 8 and P["info"].hub_rows > 0


def test_uniform_and_banded_patterns_stay_unsliced(ctx):
    w = W.erdos_renyi(4096, 16, 32)
    P = both(ctx, w.nrows, w.ncols, w.ii, w.jj, xcd_slices=8, l2_hot_bytes=16 * 1024)
    assert P["info"].nqueues == 1 and P["info"].order_is_identity == 1
    w = W.stencil5(64, 32)
    both(ctx, w.nrows, w.ncols, w.ii, w.jj)
    w = W.hypergraph_zipf(3000, 2000, 128)
    both(ctx, w.nrows, w.ncols, w.ii, w.jj)


def test_random_patterns_and_options_differential(ctx):
    # many small skewed patterns under random tuning: every layout decision of the two
    # builders (slicing on/off, hub rows, cut rows, dealing, padding) must coincide
    rng = np.random.default_rng(2024)
    sliced = 0
    for _ in range(60):
        m, n = int(rng.integers(1, 400)), int(rng.integers(40, 400))
        nnz = int(rng.integers(1, 6000))
        # Zipf-like rows and columns so that hubs and hot columns exist
        ii = np.minimum((rng.pareto(0.7, nnz)).astype(np.int64), m - 1).astype(np.uint32)
        jj = np.minimum((rng.pareto(0.5, nnz) * 3).astype(np.int64), n - 1).astype(np.uint32)
        if rng.random() < 0.5:
            o = np.lexsort((jj, ii))
            ii, jj = ii[o], jj[o]
        opts = dict(seg_max=int(rng.choice([1, 3, 16, 64, 500])),
                    hub_min=int(rng.choice([1, 2, 8, 32, 128])),
                    l2_hot_bytes=int(rng.choice([64, 256, 1024, 4096])),
                    k_hint=int(rng.choice([1, 16, 64])),
                    xcd_slices=int(rng.choice([0, 8, 8, 1])),
                    slice_affinity=bool(rng.random() < 0.7))
        P = both(ctx, m, n, ii, jj, **opts)
        sliced += P["info"].nqueues == 8
    assert sliced >= 10  # the sliced layout was exercised, not only the plain one


def test_bad_index_is_reported_as_by_the_host_check(ctx):
    ii = np.array([0, 1, 1, 9, 1], dtype=np.uint32)
    jj = np.array([0, 1, 5, 0, 7], dtype=np.uint32)
    with pytest.raises(capi.BadIndexError) as dev_err:
        ctx.plan(2, 6, ii, jj, dtype=np.float32, builder="device")
    with pytest.raises(capi.BadIndexError) as host_err:
        device.plan_build_host(2, 6, ii, jj)
    assert "entry 3 = (9, 0)" in str(dev_err.value)
    assert str(dev_err.value).split(":")[-1] == str(host_err.value).split(":")[-1]


def test_pattern_already_on_the_device(ctx):
    w = W.rmat(14, 16, 64).shuffled()
    dii, djj = ctx.vals(w.nnz, np.float32), ctx.vals(w.nnz, np.float32)
    dii.upload(w.ii.view(np.float32))  # 32-bit words; the library never interprets them as reals
    djj.upload(w.jj.view(np.float32))
    S = device.Plan.from_device(ctx, w.nrows, w.ncols, dii, djj, w.nnz, np.float64, seg_max=128)
    host = device.plan_build_host(w.nrows, w.ncols, w.ii, w.jj, dtype="f64", seg_max=128)
    assert_same_plan(S.download(), host)
    # and it computes: values set afterwards, SDDMM against the host-built plan's result
    vv = w.values("f64")
    S.set_values(vv)
    H = ctx.plan(w.nrows, w.ncols, w.ii, w.jj, vv, builder="host", seg_max=128)
    dA, dB = ctx.panel_from(w.panel_A("f64")), ctx.panel_from(w.panel_B("f64"))
    c1, c2 = ctx.vals(w.nnz, np.float64), ctx.vals(w.nnz, np.float64)
    ctx.sddmm(S, dA, dB, c1)
    ctx.sddmm(H, dA, dB, c2)
    assert np.array_equal(c1.download(), c2.download())
    for h in (S, H, dA, dB, c1, c2, dii, djj):
        h.close()


def _words(ctx, a):
    v = ctx.vals(max(a.size, 1), np.float32)
    if a.size:
        v.upload(np.ascontiguousarray(a, dtype=np.uint32).view(np.float32))
    return v


def _first_appearance(a):
    ids, ltg, out = {}, [], np.empty(a.size, dtype=np.uint32)
    for e, g in enumerate(a.tolist()):  # src/SparseMatrix.hpp:69-99, one array
        if g not in ids:
            ids[g] = len(ltg)
            ltg.append(g)
        out[e] = ids[g]
    return out, np.array(ltg, dtype=np.uint32)


def test_localize_on_device_matches_the_reference_vectors(ctx):
    # tests/golden: the reference's own localizeIndices on an 80-entry pattern
    g = np.load(GOLDEN_PATH)
    for glob, loc, ltg in (("localize.gi", "localize.li", "localize.ltgR"),
                           ("localize.gj", "localize.lj", "localize.ltgC")):
        d = _words(ctx, g[glob])
        nlocal, dl = device.localize_device(ctx, d, g[glob].size)
        assert nlocal == g[ltg].size
        assert np.array_equal(d.download().view(np.uint32)[:g[glob].size], g[loc])
        assert np.array_equal(dl.download().view(np.uint32)[:nlocal], g[ltg])


@pytest.mark.parametrize("n,span", [(1, 5), (1000, 50), (100000, 2 ** 32 - 1), (300000, 70000)])
def test_localize_and_remap_on_device_random(ctx, n, span):
    rng = np.random.default_rng(n)
    a = rng.integers(0, span, n, dtype=np.uint64).astype(np.uint32)
    want, ltg = _first_appearance(a)
    d = _words(ctx, a)
    nlocal, dl = device.localize_device(ctx, d, n)
    assert nlocal == ltg.size
    assert np.array_equal(d.download().view(np.uint32)[:n], want)
    assert np.array_equal(dl.download().view(np.uint32)[:nlocal], ltg)
    # ReMapIndices with the inverse map gives the global ids back
    device.remap_device(ctx, d, n, dl, nlocal)
    assert np.array_equal(d.download().view(np.uint32)[:n], a)
    # an index outside the map is refused and nothing changes
    if nlocal > 1:
        with pytest.raises(capi.BadIndexError):
            device.remap_device(ctx, d, n, dl, int(a.max()))
        assert np.array_equal(d.download().view(np.uint32)[:n], a)


def test_download_refuses_short_buffers(ctx):
    ii, jj = hub_case(5, 20, 20, 300, 100)
    S = ctx.plan(20, 20, ii, jj, dtype=np.float32, seg_max=16)
    segs = np.zeros(4, dtype=np.uint32)
    rc = ctx._lib.spc3d_plan_download(S._h, None, None, segs.ctypes.data_as(ctypes.c_void_p), 1,
                                      None, 0)
    assert rc == capi.ERR_SIZE_MISMATCH
    S.close()


def test_full_size_rmat20_and_time(ctx):
    import time

    w = W.make("rmat20")
    t0 = time.perf_counter()
    host = device.plan_build_host(w.nrows, w.ncols, w.ii, w.jj, dtype="f64", k_hint=w.k)
    t1 = time.perf_counter()
    S = ctx.plan(w.nrows, w.ncols, w.ii, w.jj, dtype=np.float64, builder="device", k_hint=w.k)
    ctx.sync()
    t2 = time.perf_counter()
    assert_same_plan(S.download(), host)
    S.close()
    print(f"rmat20 plan: host builder, sizing pass + filling pass {1e3 * (t1 - t0):.1f} ms; "
          f"device builder with upload {1e3 * (t2 - t1):.1f} ms")
