"""Row tiles x column blocks (spc3d_plan_opts.sweep): long rows kept in LDS while their
workgroups walk the column blocks.  Same results as the ordinary plan to the tolerance of
the parity tests, the same bits run to run, through every entry point."""
import numpy as np
import pytest

from spcomm3d_amd import _capi as capi
from tests import _oracle as oracle

pytestmark = pytest.mark.gpu

TOL = {np.dtype(np.float32): 1e-5, np.dtype(np.float64): 1e-12}


def long_rows(seed, m, n, k, dtype, lens, shuffle=True):
    """Rows of the given lengths over uniform columns (repeats allowed), in a shuffled
    order or sorted by row and column, with values and panels."""
    rng = np.random.default_rng(seed)
    lens = np.asarray(lens, dtype=np.int64)
    ii = np.repeat(np.arange(m, dtype=np.uint32), lens)
    jj = rng.integers(0, n, ii.size).astype(np.uint32)
    o = rng.permutation(ii.size) if shuffle else np.lexsort((jj, ii))  # or by row, then column
    ii, jj = np.ascontiguousarray(ii[o]), np.ascontiguousarray(jj[o])
    vv = rng.random(ii.size).astype(dtype)
    A = rng.uniform(-1, 1, (m, k)).astype(dtype)
    B = rng.uniform(-1, 1, (n, k)).astype(dtype)
    Y0 = rng.uniform(-1, 1, (m, k)).astype(dtype)
    return ii, jj, vv, A, B, Y0


def run_all(ctx, m, n, ii, jj, vv, A, B, Y0, **opts):
    """C of sddmm, Y of spmm (twice: bits), Y of spmm_noalloc, C and Y of the one-pass call
    plain and chained; and the plan's info."""
    S = ctx.plan(m, n, ii, jj, vv, **opts)
    info = S.info
    dA, dB = ctx.panel_from(A), ctx.panel_from(B)
    dC = ctx.vals(ii.size, A.dtype)
    dC.fill(-7.0)
    ctx.sddmm(S, dA, dB, dC)
    out = {"C": dC.download()}
    for name, call in (("Y", ctx.spmm), ("Y_again", ctx.spmm), ("Y_noalloc", ctx.spmm_noalloc)):
        dY = ctx.panel_from(Y0)
        call(S, dB, dY)
        out[name] = dY.download()
        dY.close()
    for name, chained in (("one", False), ("chain", True)):
        dY = ctx.panel_from(Y0)
        dC.fill(3.0)
        ctx.sddmm_spmm(S, dA, dB, dC, dY, chained=chained)
        out["C_" + name], out["Y_" + name] = dC.download(), dY.download()
        dY.close()
    for h in (S, dA, dB, dC):
        h.close()
    return out, info


def check(out, ii, jj, vv, A, B, Y0):
    tol = TOL[A.dtype]
    assert oracle.sddmm_rel_err(A, B, ii, jj, vv, out["C"]) <= tol
    assert oracle.spmm_rel_err(B, ii, jj, vv, Y0, out["Y"]) <= tol
    assert np.array_equal(out["Y"], out["Y_again"])
    assert np.array_equal(out["Y"], out["Y_noalloc"])
    assert np.array_equal(out["C_one"], out["C"]) and np.array_equal(out["C_chain"], out["C"])
    assert oracle.spmm_rel_err(B, ii, jj, vv, Y0, out["Y_one"]) <= tol
    assert oracle.spmm_rel_err(B, ii, jj, out["C"], Y0, out["Y_chain"]) <= tol


@pytest.mark.parametrize("shuffle", [True, False])
@pytest.mark.parametrize("dtype,k", [(np.float32, 64), (np.float32, 128), (np.float32, 256),
                                     (np.float64, 32), (np.float64, 64), (np.float64, 128)])
def test_tiles_and_rest_against_the_oracle(ctx, dtype, k, shuffle):
    rng = np.random.default_rng(k)
    m, n = 700, 3000
    lens = rng.integers(0, 400, m)
    lens[::7] = rng.integers(1, 12, lens[::7].size)  # short rows: the plan of the rest
    lens[5] = 0
    lens[11] = 5000                                  # more entries than columns
    case = long_rows(1000 + k, m, n, k, dtype, lens, shuffle)
    ii, jj, vv, A, B, Y0 = case
    out, info = run_all(ctx, m, n, *case, k_hint=k, sweep=True, sweep_min_row=12, col_blocks=7)
    assert info.sweep_k == k and info.sweep_tiles > 0 and info.ncol_blocks == 7
    want = int(lens[lens >= 12].sum())
    assert info.sweep_entries == want and info.nsegments > 0
    # sorted, the tiles store straight to the caller's positions; shuffled, they stage
    assert info.staged_entries == (want if shuffle else 0)
    if not shuffle:
        forced, finfo = run_all(ctx, m, n, *case, k_hint=k, sweep=True, sweep_min_row=12,
                                col_blocks=7, sweep_staged=True)
        assert finfo.staged_entries == want
        for name in out:
            assert np.array_equal(out[name], forced[name]), name
    assert info.device_bytes > ii.size * 10
    check(out, *case)
    # against the ordinary plan: the same products, another summation order
    ref, rinfo = run_all(ctx, m, n, *case, k_hint=k, sweep=False)
    assert rinfo.sweep_entries == 0
    scale = oracle.sddmm_scale(A, B, ii, jj, vv)
    assert oracle.rel_err(out["C"], ref["C"], scale) <= TOL[A.dtype]


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_every_row_in_the_tiles_and_more_tiles_than_one_launch_takes(ctx, dtype):
    # 512-byte dense rows: 256 rows per tile, one launch per CU-count tiles; 150 k rows of
    # a few entries each make more than two launches' worth of tiles, the last one partial
    k = 128 if dtype == np.float32 else 64
    m, n = 150_000, 4096
    rng = np.random.default_rng(5)
    lens = rng.integers(1, 9, m)
    case = long_rows(77, m, n, k, dtype, lens)
    out, info = run_all(ctx, m, n, *case, k_hint=k, sweep=True, sweep_min_row=1, col_blocks=3)
    assert info.sweep_entries == case[0].size and info.nsegments == 0
    # a launch deals its rows over as many tiles as there are CUs: two full launches of 256
    # rows per tile, and the last one's 18,928 rows thinly over its tiles
    cus = info.sweep_tiles // 3
    assert info.sweep_tiles == 3 * cus and 2 * cus * 256 < m <= 3 * cus * 256
    check(out, *case)


def test_a_single_block_and_as_many_as_fit(ctx):
    k, m, n = 128, 300, 5000
    lens = np.full(m, 200)
    case = long_rows(3, m, n, k, np.float32, lens)
    for nb in (1, 192, 4000):  # 4000: cut down to what a tile's range bounds allow
        out, info = run_all(ctx, m, n, *case, k_hint=k, sweep=True, sweep_min_row=1, col_blocks=nb)
        assert info.sweep_entries == case[0].size and info.ncol_blocks == min(nb, 1027)
        check(out, *case)


def test_another_k_runs_an_ordinary_plan_made_on_first_use(ctx):
    k, m, n = 128, 300, 1000
    rng = np.random.default_rng(4)
    lens = rng.integers(0, 200, m)
    case = long_rows(9, m, n, k, np.float32, lens)
    ii, jj, vv, A, B, Y0 = case
    S = ctx.plan(m, n, ii, jj, vv, k_hint=k, sweep=True, sweep_min_row=16, col_blocks=3)
    assert 0 < S.info.sweep_entries < ii.size
    before = S.info.device_bytes
    k2 = 48
    A2, B2, Y2 = (np.ascontiguousarray(x[:, :k2]) for x in (A, B, Y0))
    dA, dB, dY = ctx.panel_from(A2), ctx.panel_from(B2), ctx.panel_from(Y2)
    dC = ctx.vals(ii.size, np.float32)
    # the call that allocates nothing cannot make that plan, and says who can
    with pytest.raises(capi.Spc3dError) as e:
        ctx.spmm_noalloc(S, dB, dY)
    assert e.value.status == capi.ERR_INVALID_ARG and "spc3d_spmm" in str(e.value)
    # nor can a call that is being recorded
    ctx.capture_begin()
    with pytest.raises(capi.Spc3dError):
        ctx.sddmm(S, dA, dB, dC)
    ctx.capture_end().close()
    ctx.sync()
    assert np.array_equal(dY.download(), Y2) and S.info.device_bytes == before
    # the first ordinary call makes it; every entry point then runs at that K, and at a third
    ctx.sddmm(S, dA, dB, dC)
    assert S.info.device_bytes > before and S.info.sweep_entries > 0
    assert oracle.sddmm_rel_err(A2, B2, ii, jj, vv, dC.download()) <= 1e-5
    ctx.spmm(S, dB, dY)
    Y_spmm = dY.download()
    assert oracle.spmm_rel_err(B2, ii, jj, vv, Y2, Y_spmm) <= 1e-5
    dY.upload(Y2)
    ctx.spmm_noalloc(S, dB, dY)
    assert np.array_equal(dY.download(), Y_spmm)
    dY.upload(Y2)
    ctx.sddmm_spmm(S, dA, dB, dC, dY, chained=True)
    C = dC.download()
    assert oracle.spmm_rel_err(B2, ii, jj, C, Y2, dY.download()) <= 1e-5
    A3, B3 = np.ascontiguousarray(A[:, :7]), np.ascontiguousarray(B[:, :7])
    dA3, dB3 = ctx.panel_from(A3), ctx.panel_from(B3)
    ctx.sddmm(S, dA3, dB3, dC)
    assert oracle.sddmm_rel_err(A3, B3, ii, jj, vv, dC.download()) <= 1e-5
    # new values reach both forms of the plan
    S.set_values(2 * vv)
    ctx.sddmm(S, dA, dB, dC)
    assert np.array_equal(dC.download(), 2 * C)
    dA4, dB4 = ctx.panel_from(A), ctx.panel_from(B)
    ctx.sddmm(S, dA4, dB4, dC)  # and the tiles still run at their own K
    assert oracle.sddmm_rel_err(A, B, ii, jj, 2 * vv, dC.download()) <= 1e-5
    for h in (S, dA, dB, dY, dC, dA3, dB3, dA4, dB4):
        h.close()
    # a width the tile kernels do not take, or no k_hint: the ordinary plan from the start
    for opts in ({"k_hint": 100, "sweep": True}, {"sweep": True}):
        S = ctx.plan(m, n, ii, jj, vv, **opts)
        assert S.info.sweep_entries == 0 and S.info.nsegments > 0
        S.close()


def test_values_set_later_and_from_the_device(ctx):
    k, m, n = 64, 400, 2000
    rng = np.random.default_rng(1)
    lens = rng.integers(0, 150, m)
    ii, jj, vv, A, B, Y0 = long_rows(21, m, n, k, np.float64, lens)
    S = ctx.plan(m, n, ii, jj, None, dtype=np.float64, k_hint=k, sweep=True, sweep_min_row=20,
                 col_blocks=4)
    assert 0 < S.info.sweep_entries < ii.size
    dA, dB = ctx.panel_from(A), ctx.panel_from(B)
    dC = ctx.vals(ii.size, np.float64)
    S.set_values(vv)
    ctx.sddmm(S, dA, dB, dC)
    first = dC.download()
    assert oracle.sddmm_rel_err(A, B, ii, jj, vv, first) <= 1e-12
    dV = ctx.vals(ii.size, np.float64)
    dV.upload(2 * vv)
    S.set_values_device(dV)
    ctx.sddmm(S, dA, dB, dC)
    assert np.array_equal(dC.download(), 2 * first)
    for h in (S, dA, dB, dC, dV):
        h.close()


def test_random_shapes_differential(ctx):
    """Seeded random patterns, tile and block counts: few rows per tile, blocks without entries,
    rows longer than a block's share of the lane groups, single-entry rows, every row width."""
    rng = np.random.default_rng(2024)
    widths = [(np.float32, 64), (np.float32, 128), (np.float32, 256),
              (np.float64, 32), (np.float64, 64), (np.float64, 128)]
    for case_no in range(24):
        dtype, k = widths[case_no % len(widths)]
        m = int(rng.choice([1, 3, 40, 300, 1500]))
        n = int(rng.choice([1, 7, 100, 5000]))
        shape = rng.choice(["short", "mixed", "long", "one_huge"])
        if shape == "short":
            lens = rng.integers(0, 4, m)
        elif shape == "mixed":
            lens = rng.integers(0, 60, m)
        elif shape == "long":
            lens = rng.integers(100, 400, m) if m <= 300 else rng.integers(0, 80, m)
        else:
            lens = rng.integers(0, 3, m)
            lens[rng.integers(0, m)] = 20000
        if lens.sum() == 0:
            lens[0] = 1
        case = long_rows(int(rng.integers(1 << 30)), m, n, k, dtype, lens,
                         shuffle=bool(rng.random() < 0.5))
        nb = int(rng.choice([1, 2, 5, 33, 1000]))
        min_row = int(rng.choice([1, 1, 2, 10, 50]))
        out, info = run_all(ctx, m, n, *case, k_hint=k, sweep=True, sweep_min_row=min_row,
                            col_blocks=nb, sweep_staged=bool(rng.random() < 0.3))
        want = int(lens[lens >= min_row].sum())
        assert info.sweep_entries == want, (case_no, shape, m, n, nb, min_row)
        if want and nb > 1:  # (1 leaves the number of blocks to the rule)
            assert info.ncol_blocks == min(nb, n)
        check(out, *case)
