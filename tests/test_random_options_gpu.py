"""Seeded random patterns, row widths and plan options through every entry point of the hot
path, judged against the oracle run in double on the same inputs (the same-type oracle adds
its own rounding on rows of thousands of entries, core_ops.cpp:28-33 accumulates in order).

What the options may refuse by contract (a plan too wide for spc3d_spmm_noalloc's array, the
chained one-pass call on rows over 4 KiB, the host builder with column blocks) is skipped per
case; everything else must give SDDMM, SpMM and both one-pass results within the parity
tolerance, SpMM the same bits from call to call and from spc3d_spmm_noalloc, and the one-pass
SDDMM the bits of spc3d_sddmm."""
import numpy as np
import pytest

from spcomm3d_amd import _capi as capi
from tests import _oracle as oracle
from tests.test_sweep_gpu import long_rows, run_all

pytestmark = pytest.mark.gpu

TOL = {np.dtype(np.float32): 1e-5, np.dtype(np.float64): 1e-12}
WIDTHS = [1, 2, 3, 4, 5, 7, 8, 12, 16, 17, 24, 32, 33, 48, 64, 65, 100, 128, 129, 192, 256, 257,
          512, 520, 1030]
REFUSALS = ("spc3d_spmm_noalloc has", "the chained form needs dense rows",
            "column blocks are built on the GPU")


def draw_case(rng):
    dtype = [np.float32, np.float64][int(rng.integers(2))]
    k = int(rng.choice(WIDTHS))
    m = int(rng.choice([1, 2, 3, 40, 255, 300, 1500, 5000, 20000]))
    n = int(rng.choice([1, 2, 7, 100, 5000, 70000]))
    shape = str(rng.choice(["short", "mixed", "long", "one_huge", "skew"]))
    if shape == "short":
        lens = rng.integers(0, 4, m)
    elif shape == "mixed":
        lens = rng.integers(0, 60, m)
    elif shape == "long":
        lens = rng.integers(100, 400, m) if m <= 300 else rng.integers(0, 80, m)
    elif shape == "skew":
        lens = np.minimum((rng.pareto(1.0, m) * 3).astype(np.int64), 5000)
    else:
        lens = rng.integers(0, 3, m)
        lens[rng.integers(0, m)] = int(rng.choice([17, 1000, 20000]))
    if lens.sum() == 0:
        lens[0] = 1
    if lens.sum() * k > 1e8:  # keeps the oracle's share of a case under a second
        k = 16
    case = list(long_rows(int(rng.integers(1 << 30)), m, n, k, dtype, lens,
                          shuffle=bool(rng.random() < 0.5)))
    if shape == "skew" and n >= 100:  # hot columns, so that the XCD slices have something to hold
        jj = np.minimum(rng.pareto(0.8, case[1].size).astype(np.int64), n - 1).astype(np.uint32)
        case[1] = jj
        if rng.random() < 0.5:
            o = np.lexsort((jj, case[0]))
            case[0], case[1] = np.ascontiguousarray(case[0][o]), np.ascontiguousarray(jj[o])
    opts = dict(k_hint=int(rng.choice([0, k])) or None, sweep=False)
    if rng.random() < 0.5:
        opts["seg_max"] = int(rng.choice([4, 16, 64, 300, 2048]))
    if rng.random() < 0.5:
        opts["hub_min"] = int(rng.choice([2, 8, 64, 128]))
    if rng.random() < 0.5:
        opts["xcd_slices"] = int(rng.choice([1, 8]))
    if rng.random() < 0.3:
        opts["l2_hot_bytes"] = int(rng.choice([4096, 1 << 16, 1 << 20]))
    if rng.random() < 0.3:
        opts["col_blocks"] = int(rng.choice([2, 3, 17]))
    if rng.random() < 0.3:
        opts["builder"] = "host"
    if rng.random() < 0.3:
        opts["two_pass_min"] = 1
    for flag in ("staged_stores", "sddmm_by_column", "slice_affinity"):
        if rng.random() < 0.2:
            opts[flag] = False
    if rng.random() < 0.2:
        opts["keep_entry_order"] = True
    return (shape, m, n, k, np.dtype(dtype).name), case, opts


@pytest.mark.parametrize("seed", [300, 301, 302, 303, 304, 305])
def test_random_patterns_and_options_against_the_double_oracle(ctx, seed):
    rng = np.random.default_rng(seed)
    ran = 0
    for case_no in range(20):
        what, case, opts = draw_case(rng)
        ii, jj, vv, A, B, Y0 = case
        try:
            out, _ = run_all(ctx, A.shape[0], B.shape[0], *case, **opts)
        except capi.Spc3dError as e:
            if any(r in str(e) for r in REFUSALS):
                continue
            raise AssertionError((seed, case_no, what, opts)) from e
        ran += 1
        tol = TOL[A.dtype]
        tag = (seed, case_no, what, opts)
        assert oracle.sddmm_rel_err_exact(A, B, ii, jj, vv, out["C"]) <= tol, tag
        assert oracle.spmm_rel_err_exact(B, ii, jj, vv, Y0, out["Y"]) <= tol, tag
        assert oracle.spmm_rel_err_exact(B, ii, jj, vv, Y0, out["Y_one"]) <= tol, tag
        assert oracle.spmm_rel_err_exact(B, ii, jj, out["C"], Y0, out["Y_chain"]) <= tol, tag
        assert np.array_equal(out["Y"], out["Y_again"]), tag
        assert np.array_equal(out["Y"], out["Y_noalloc"]), tag
        assert np.array_equal(out["C_one"], out["C"]), tag
        assert np.array_equal(out["C_chain"], out["C"]), tag
    assert ran >= 10
