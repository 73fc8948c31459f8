"""spc3d_spmm_noalloc: the SpMM entry point that allocates nothing (its partial-sum
rows live in an array inside the library's device code) must give what spc3d_spmm
gives, bit for bit, on calls in a row that share the array."""
import numpy as np
import pytest

from spcomm3d_amd import _capi as capi
from spcomm3d_amd import workloads as W
from tests import _oracle as oracle

pytestmark = pytest.mark.gpu


def both_ways(ctx, w, dtype, **plan_opts):
    vv = w.values(dtype)
    X, Y0 = w.panel_B(dtype), w.panel_Y0(dtype)
    S = ctx.plan(w.nrows, w.ncols, w.ii, w.jj, vv, **plan_opts)
    assert S.info.nsplit_rows > 0 and S.info.npartial_slots > 0  # the scratch is in use
    dX, dY1, dY2 = ctx.panel_from(X), ctx.panel_from(Y0), ctx.panel_from(Y0)
    ctx.spmm(S, dX, dY1)
    ctx.spmm_noalloc(S, dX, dY2)
    ctx.spmm_noalloc(S, dX, dY2)  # accumulates, as spc3d_spmm does
    ctx.spmm(S, dX, dY1)
    want, got = dY1.download(), dY2.download()
    for h in (S, dX, dY1, dY2):
        h.close()
    assert np.array_equal(got, want)
    once = oracle.spmm(X, w.ii, w.jj, vv, Y0)
    tol = 1e-12 if np.dtype(dtype) == np.float64 else 1e-5
    assert oracle.spmm_rel_err(X, w.ii, w.jj, vv, once, got) <= tol


def test_two_calls_in_a_row_the_second_smaller(ctx):
    # 16 k rows with hubs, every row over 32 entries cut: thousands of partial-sum rows
    both_ways(ctx, W.rmat(14, 16, 64).shuffled(), np.float64, seg_max=32)
    # then a smaller pattern with narrower rows of another type over the same array
    both_ways(ctx, W.rmat(11, 16, 24), np.float32, seg_max=16, k_hint=24)
    # and the XCD-sliced layout (hub rows cut by column slice)
    both_ways(ctx, W.rmat(16, 16, 64), np.float64)


def test_column_blocks_and_wide_rows_share_the_array(ctx):
    # a plan kept in column blocks: the blocks use the array one after the other, each
    # block's fix-up ordered before the next block's launches
    both_ways(ctx, W.rmat(14, 16, 64).shuffled(), np.float64, seg_max=32, col_blocks=4)
    both_ways(ctx, W.rmat(13, 16, 32), np.float32, seg_max=32, col_blocks=3, k_hint=32)
    # dense rows over 4 KiB run as column slices, every slice through the same partial rows
    w = W.rmat(11, 16, 1024)
    S = ctx.plan(w.nrows, w.ncols, w.ii, w.jj, w.values(np.float64), k_hint=w.k)
    need = S.info.npartial_slots * w.k * 8
    S.close()
    assert 0 < need <= 32 << 20  # few cut rows: fits the array at 8 KiB per partial row
    both_ways(ctx, w, np.float64, k_hint=w.k)


def test_a_plan_beyond_the_array_is_refused_and_nothing_runs(ctx):
    w = W.rmat(14, 16, 1024).shuffled()
    vv = w.values(np.float64)
    S = ctx.plan(w.nrows, w.ncols, w.ii, w.jj, vv, seg_max=8, k_hint=8)
    need = S.info.npartial_slots * w.k * 8
    assert need > 32 << 20
    Y0 = w.panel_Y0(np.float64)
    dX, dY = ctx.panel_from(w.panel_B(np.float64)), ctx.panel_from(Y0)
    with pytest.raises(capi.Spc3dError) as e:
        ctx.spmm_noalloc(S, dX, dY)
    assert e.value.status == capi.ERR_TOO_LARGE and "spc3d_spmm" in str(e.value)
    ctx.sync()
    assert np.array_equal(dY.download(), Y0)
    for h in (S, dX, dY):
        h.close()
