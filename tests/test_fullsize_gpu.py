"""The benchmark configurations at their full size on the GPU.

The oracle is serial, so at these sizes it runs on samples: SDDMM results are
independent per entry (any subset of entries is a valid smaller problem on the
same panels), SpMM results are independent per row (all entries of a subset of
rows).  Size-independent properties cover the rest: rows without entries keep Y
bit for bit, scaling the sparse values by 2 doubles every SDDMM result exactly,
and the adjoint identity <S X, A>_F = sum_e sddmm(A, X, S)_e ties the two
kernels to each other over all entries.
"""
import numpy as np
import pytest

from spcomm3d_amd import workloads as W
from tests import _oracle as oracle

pytestmark = pytest.mark.gpu


def _check_sampled(ctx, w, dtype, n_entries=200_000, n_rows=3000, seed=9, col_blocks=None,
                   how=None):
    """col_blocks: None = a plan with every option at its default; "auto" = the plan must
    have chosen column blocks by itself (k_hint given, as bench.py does).  how: the entry
    order, where the plan must have chosen the matching way of storing SDDMM's results."""
    tol = oracle.TOL[np.dtype(W.np_dtype(dtype))]
    rng = np.random.default_rng(seed)
    A, B, Y0, vv = w.panel_A(dtype), w.panel_B(dtype), w.panel_Y0(dtype), w.values(dtype)
    if col_blocks == "auto":
        S = ctx.plan(w.nrows, w.ncols, w.ii, w.jj, vv, k_hint=w.k)
        assert S.info.ncol_blocks > 1
    else:
        S = ctx.plan(w.nrows, w.ncols, w.ii, w.jj, vv)
    info = S.info
    assert info.nnz == w.nnz
    if info.sweep_entries:  # long rows in tiles, the segments are those of the other rows
        assert info.sweep_entries > info.nnz // 2 and info.sweep_tiles > 0 and info.sweep_k == w.k
    else:
        assert info.nsegments >= info.rows_touched
    if how == "sorted":
        assert info.staged_entries > 0 and info.positions_by_segment == 1
        assert info.two_pass_results == 0 and info.sddmm_by_column == 0
    elif how == "shuffled":
        assert info.two_pass_results == 1 and info.staged_entries == 0
        assert info.sddmm_by_column == 0
    elif how == "column-major":
        assert info.sddmm_by_column == 1 and info.two_pass_results == 1
    dA, dB, dY = ctx.panel_from(A), ctx.panel_from(B), ctx.panel_from(Y0)
    dC = ctx.vals(w.nnz, dtype)
    dC.fill(float("nan"))
    ctx.sddmm(S, dA, dB, dC)
    ctx.spmm(S, dB, dY)
    C = dC.download()
    Y = dY.download()

    # every entry was written
    assert np.all(np.isfinite(C))
    # SDDMM on a random subset of entries
    e = np.sort(rng.choice(w.nnz, size=min(n_entries, w.nnz), replace=False))
    err = oracle.sddmm_rel_err(A, B, w.ii[e], w.jj[e], vv[e], C[e])
    assert err <= tol, f"sddmm sample err {err:.3e}"
    # SpMM on a subset of rows: random ones plus the longest
    deg = np.bincount(w.ii, minlength=w.nrows)
    rows = np.union1d(rng.choice(w.nrows, size=min(n_rows, w.nrows), replace=False),
                      np.argsort(deg)[-8:])
    pick = np.flatnonzero(np.isin(w.ii, rows))
    local = np.searchsorted(rows, w.ii[pick]).astype(np.uint32)
    Ysub = oracle.spmm(B, local, w.jj[pick], vv[pick], Y0[rows])
    scale = oracle.spmm_scale(B, local, w.jj[pick], vv[pick], Y0[rows])
    err = oracle.rel_err(Y[rows], Ysub, scale)
    assert err <= tol, f"spmm sample err {err:.3e}"
    # rows without entries are untouched, bit for bit
    empty = np.flatnonzero(deg == 0)
    if empty.size:
        take = empty[:: max(1, empty.size // 100_000)]
        assert np.array_equal(Y[take], Y0[take])
    # adjoint identity over all entries (fp64 accumulation on the host)
    lhs = float(np.sum((Y.astype(np.float64) - Y0.astype(np.float64)) * A.astype(np.float64)))
    rhs = float(np.sum(C.astype(np.float64)))
    mag = float(np.sum(np.abs(C.astype(np.float64)))) + 1.0
    assert abs(lhs - rhs) <= (1e-10 if tol < 1e-9 else 2e-5) * mag
    # doubling the sparse values doubles every result exactly
    S.set_values(vv * 2)
    ctx.sddmm(S, dA, dB, dC)
    assert np.array_equal(dC.download(), C * 2)
    for h in (S, dA, dB, dY, dC):
        h.close()


@pytest.mark.parametrize("dtype", ["f32", "f64"])
@pytest.mark.parametrize("order", ["sorted", "shuffled", "column-major"])
def test_config2_rmat20_full(ctx, dtype, order):
    w = W.rmat(20, 16, 64)
    assert w.nnz == 16_086_740  # the realised nnz of the seeded generator after dedup
    if order == "shuffled":
        w = w.shuffled()
    elif order == "column-major":
        w = w.column_major()
    _check_sampled(ctx, w, dtype, how=order)


def test_config3_rmat24_block_full(ctx):
    w = W.rmat_block(24, 16, 64, 4, 4, 0, 0)
    assert w.nrows == w.ncols == 4_194_304
    _check_sampled(ctx, w, "f32")


def test_config4_stencil_full(ctx):
    w = W.stencil5(4096, 4096, 32)
    assert w.nnz == 83_869_696
    _check_sampled(ctx, w, "f32", n_entries=400_000, n_rows=20_000)


def test_config5_hypergraph_full(ctx):
    w = W.hypergraph_zipf(2_000_000, 500_000, 128, 1.2, 1024)
    assert w.nrows == 2_000_000 and w.ncols == 500_000 and w.k == 128
    _check_sampled(ctx, w, "f32", n_entries=200_000, n_rows=2000, col_blocks="auto")
