"""GPU parity: the HIP path, called through the C ABI, against the CPU oracle on
the same seeded inputs.

Bar: sparsity pattern / output position exact; values within 1e-12 (fp64) or
1e-5 (fp32), relative to max(|reference value|, sum of |terms|) per output
element (U[-1,1] dot products cancel towards zero, so the plain ratio to the
value is meaningless there).  fp32 is additionally held to 1e-5 against the
fp64 oracle on the same inputs.
"""
import numpy as np
import pytest

from spcomm3d_amd import _capi as capi
from spcomm3d_amd import device
from spcomm3d_amd import workloads as W
from tests import _oracle as oracle

pytestmark = pytest.mark.gpu

GOLDEN = np.load(oracle.os.path.join(oracle.ROOT, "tests", "golden", "core_ops_golden.npz"),
                 allow_pickle=False)
DTYPES = [np.float32, np.float64]


def tol_of(dtype):
    return oracle.TOL[np.dtype(dtype)]


def rand_case(seed, m, n, k, nnz, dtype, hub=None):
    rng = np.random.default_rng(seed)
    ii = rng.integers(0, m, nnz).astype(np.uint32)
    jj = rng.integers(0, n, nnz).astype(np.uint32)
    if hub:
        ii[:hub] = m // 2
    if nnz > 8:
        ii[-3:], jj[-3:] = ii[:3], jj[:3]  # exact duplicates
    o = rng.permutation(nnz)
    ii, jj = np.ascontiguousarray(ii[o]), np.ascontiguousarray(jj[o])
    vv = rng.random(nnz).astype(dtype)
    A = rng.uniform(-1, 1, (m, k)).astype(dtype)
    B = rng.uniform(-1, 1, (n, k)).astype(dtype)
    Y0 = rng.uniform(-1, 1, (m, k)).astype(dtype)
    return ii, jj, vv, A, B, Y0


def gpu_sddmm(ctx, m, n, ii, jj, vv, A, B, seg_max=None, prefill=None):
    S = ctx.plan(m, n, ii, jj, vv, seg_max=seg_max)
    dA, dB = ctx.panel_from(A), ctx.panel_from(B)
    dC = ctx.vals(ii.size, A.dtype)
    if prefill is not None:
        dC.fill(prefill)
    ctx.sddmm(S, dA, dB, dC)
    out = dC.download()
    for h in (S, dA, dB, dC):
        h.close()
    return out


def gpu_spmm(ctx, m, n, ii, jj, vv, X, Y0, seg_max=None, times=1):
    S = ctx.plan(m, n, ii, jj, vv, seg_max=seg_max)
    dX, dY = ctx.panel_from(X), ctx.panel_from(Y0)
    for _ in range(times):
        ctx.spmm(S, dX, dY)
    out = dY.download()
    for h in (S, dX, dY):
        h.close()
    return out


def check_sddmm(A, B, ii, jj, vv, got):
    assert got.dtype == A.dtype and got.shape == (ii.size,)
    tol = tol_of(A.dtype)
    err = oracle.sddmm_rel_err(A, B, ii, jj, vv, got)
    assert err <= tol, f"sddmm rel err {err:.3e} > {tol}"
    if A.dtype == np.float32:
        assert oracle.sddmm_rel_err_exact(A, B, ii, jj, vv, got) <= tol


def check_spmm(X, ii, jj, vv, Y0, got):
    assert got.dtype == X.dtype and got.shape == Y0.shape
    tol = tol_of(X.dtype)
    err = oracle.spmm_rel_err(X, ii, jj, vv, Y0, got)
    assert err <= tol, f"spmm rel err {err:.3e} > {tol}"
    if X.dtype == np.float32:
        assert oracle.spmm_rel_err_exact(X, ii, jj, vv, Y0, got) <= tol


# ---- the reference's own outputs (golden vectors made from its compiled code) -
@pytest.mark.parametrize("name", ["small", "k64", "hub", "k1"])
def test_golden_reference_vectors_fp64(ctx, name):
    g = {k: GOLDEN[f"{name}.{k}"] for k in ("ii", "jj", "vv", "A", "B", "Y0", "C", "Y")}
    m, n = g["A"].shape[0], g["B"].shape[0]
    C = gpu_sddmm(ctx, m, n, g["ii"], g["jj"], g["vv"], g["A"], g["B"], prefill=123.0)
    scale = oracle.sddmm_scale(g["A"], g["B"], g["ii"], g["jj"], g["vv"])
    assert oracle.rel_err(C, g["C"], scale) <= 1e-12
    Y = gpu_spmm(ctx, m, n, g["ii"], g["jj"], g["vv"], g["B"], g["Y0"])
    scale = oracle.spmm_scale(g["B"], g["ii"], g["jj"], g["vv"], g["Y0"])
    assert oracle.rel_err(Y, g["Y"], scale) <= 1e-12


def test_golden_numcheck_closed_form(ctx):
    # miniapp/numCheckSeq.cpp:125-131
    g = {k: GOLDEN[f"numcheck.{k}"] for k in ("ii", "jj", "vv", "A", "B", "C")}
    C = gpu_sddmm(ctx, 6, 5, g["ii"], g["jj"], g["vv"], g["A"], g["B"])
    np.testing.assert_allclose(C, g["C"], rtol=1e-13, atol=0)
    assert abs(C.sum() - g["C"].sum()) < 1e-16


# ---- K sweep: rows that fill a kernel shape exactly (a power of two of 16-byte
# vectors), rows that do not (the "ragged" variants: 12, 20, 48, 100, 300 ...), rows
# that are no whole number of vectors (the "odd" variants: 5, 7, 50, 63, 65, 1023 ...),
# rows shorter than 16 bytes (the "thin" variant: 1, 2, 3), rows longer than 4 KiB (run
# as 4 KiB column slices plus a rest, which may be thin: 1025 in fp32, 513 in fp64)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("k", [1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 15, 16, 17, 20, 24, 31, 32,
                               33, 36, 48, 50, 63, 64, 65, 72, 96, 100, 127, 128, 129, 130, 200,
                               255, 256, 257, 300, 384, 511, 512, 513, 1023, 1024, 1025, 1028, 1500,
                               2048, 2500])
def test_k_sweep_random_unsorted(ctx, dtype, k):
    ii, jj, vv, A, B, Y0 = rand_case(100 + k, 300, 257, k, 6000, dtype, hub=700)
    check_sddmm(A, B, ii, jj, vv, gpu_sddmm(ctx, 300, 257, ii, jj, vv, A, B, prefill=-5.0))
    check_spmm(B, ii, jj, vv, Y0, gpu_spmm(ctx, 300, 257, ii, jj, vv, B, Y0))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("seg_max", [1, 3, 16, 17, 128, 1000])
def test_segment_lengths_and_cut_rows(ctx, dtype, seg_max):
    ii, jj, vv, A, B, Y0 = rand_case(7, 64, 500, 64, 5000, dtype, hub=2000)
    check_sddmm(A, B, ii, jj, vv, gpu_sddmm(ctx, 64, 500, ii, jj, vv, A, B, seg_max=seg_max))
    check_spmm(B, ii, jj, vv, Y0, gpu_spmm(ctx, 64, 500, ii, jj, vv, B, Y0, seg_max=seg_max))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("k", [1, 2, 3, 5, 7, 12, 48, 50, 63, 65, 100, 129, 136, 257, 264, 511, 1030,
                               2051])
def test_cut_rows_with_ragged_k(ctx, dtype, k):
    # partial rows of cut segments and the fix-up pass at row widths that leave lanes idle
    # or end inside a 16-byte vector
    ii, jj, vv, A, B, Y0 = rand_case(11 + k, 40, 300, k, 4000, dtype, hub=1500)
    check_sddmm(A, B, ii, jj, vv, gpu_sddmm(ctx, 40, 300, ii, jj, vv, A, B, seg_max=64))
    check_spmm(B, ii, jj, vv, Y0, gpu_spmm(ctx, 40, 300, ii, jj, vv, B, Y0, seg_max=64))


# ---- both kernels in one pass over the gathered rows ---------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("chained", [False, True])
@pytest.mark.parametrize("k", [1, 2, 3, 4, 5, 20, 50, 63, 64, 100, 256, 257, 511])
def test_fused_sddmm_spmm_equals_the_two_calls(ctx, dtype, chained, k):
    m, n, nnz = 120, 90, 4000
    ii, jj, vv, A, B, Y0 = rand_case(500 + k, m, n, k, nnz, dtype, hub=900)
    S = ctx.plan(m, n, ii, jj, vv, seg_max=64)  # cut rows: partial sums and the fix-up
    dA, dB, dY, dC = ctx.panel_from(A), ctx.panel_from(B), ctx.panel_from(Y0), ctx.vals(nnz, dtype)
    ctx.sddmm_spmm(S, dA, dB, dC, dY, chained=chained)
    C, Y = dC.download(), dY.download()
    check_sddmm(A, B, ii, jj, vv, C)
    # the SpMM half against the oracle, with the weights it is defined to use: S.vv, or
    # the C this very call produced (C itself was held to the SDDMM oracle above)
    check_spmm(B, ii, jj, C if chained else vv, Y0, Y)
    # and the plan's own values are untouched: a plain SpMM afterwards still uses S.vv
    dY.upload(Y0)
    ctx.spmm(S, dB, dY)
    check_spmm(B, ii, jj, vv, Y0, dY.download())
    for h in (S, dA, dB, dY, dC):
        h.close()


@pytest.mark.parametrize("dtype", DTYPES)
def test_fused_call_on_the_sliced_layout_and_odd_widths(ctx, dtype):
    w = W.rmat(14, 16, 64).shuffled()
    A, B, Y0, vv = w.panel_A(dtype), w.panel_B(dtype), w.panel_Y0(dtype), w.values(dtype)
    S = ctx.plan(w.nrows, w.ncols, w.ii, w.jj, vv, xcd_slices=8, l2_hot_bytes=64 * 1024,
                 hub_min=32, seg_max=256)
    assert S.info.nqueues == 8
    dA, dB, dY, dC = ctx.panel_from(A), ctx.panel_from(B), ctx.panel_from(Y0), ctx.vals(w.nnz, dtype)
    ctx.sddmm_spmm(S, dA, dB, dC, dY)
    check_sddmm(A, B, w.ii, w.jj, vv, dC.download())
    check_spmm(B, w.ii, w.jj, vv, Y0, dY.download())
    dY.upload(Y0)
    ctx.sddmm_spmm(S, dA, dB, dC, dY, chained=True)
    check_sddmm(A, B, w.ii, w.jj, vv, dC.download())
    check_spmm(B, w.ii, w.jj, dC.download(), Y0, dY.download())
    # rows over 4 KiB: the plain form falls back to the two calls, the chained one refuses
    ii, jj, vv, A, B, Y0 = rand_case(3, 30, 30, 1030, 200, dtype)
    S2 = ctx.plan(30, 30, ii, jj, vv)
    dA, dB, dY, dC = ctx.panel_from(A), ctx.panel_from(B), ctx.panel_from(Y0), ctx.vals(200, dtype)
    ctx.sddmm_spmm(S2, dA, dB, dC, dY)
    check_sddmm(A, B, ii, jj, vv, dC.download())
    check_spmm(B, ii, jj, vv, Y0, dY.download())
    with pytest.raises(capi.Spc3dError):
        ctx.sddmm_spmm(S2, dA, dB, dC, dY, chained=True)


@pytest.mark.parametrize("dtype", DTYPES)
def test_random_shapes_widths_and_plan_options(ctx, dtype):
    # every knob at once: skewed patterns, sorted or not, exact / ragged / odd / sliced row widths,
    # cut rows, the sliced layout on small inputs, both plan builders
    rng = np.random.default_rng(99)
    for case in range(40):
        m, n = int(rng.integers(1, 300)), int(rng.integers(40, 300))
        nnz = int(rng.integers(1, 5000))
        k = int(rng.choice([1, 2, 4, 5, 7, 8, 12, 16, 19, 24, 32, 40, 50, 64, 65, 68, 96, 127, 128, 160,
                            250, 256, 516, 1030]))
        ii = np.minimum(rng.pareto(0.7, nnz).astype(np.int64), m - 1).astype(np.uint32)
        jj = np.minimum((rng.pareto(0.5, nnz) * 3).astype(np.int64), n - 1).astype(np.uint32)
        if rng.random() < 0.5:
            o = np.lexsort((jj, ii))
            ii, jj = np.ascontiguousarray(ii[o]), np.ascontiguousarray(jj[o])
        vv = rng.uniform(-1, 1, nnz).astype(dtype)
        A = rng.uniform(-1, 1, (m, k)).astype(dtype)
        B = rng.uniform(-1, 1, (n, k)).astype(dtype)
        Y0 = rng.uniform(-1, 1, (m, k)).astype(dtype)
        opts = dict(seg_max=int(rng.choice([1, 5, 16, 64, 500])),
                    hub_min=int(rng.choice([1, 8, 32, 128])),
                    l2_hot_bytes=int(rng.choice([64, 256, 4096])), k_hint=k,
                    xcd_slices=int(rng.choice([0, 8, 1])),
                    builder=str(rng.choice(["device", "host"])))
        S = ctx.plan(m, n, ii, jj, vv, **opts)
        dA, dB, dY, dC = ctx.panel_from(A), ctx.panel_from(B), ctx.panel_from(Y0), ctx.vals(nnz, dtype)
        ctx.sddmm(S, dA, dB, dC)
        ctx.spmm(S, dB, dY)
        try:
            check_sddmm(A, B, ii, jj, vv, dC.download())
            check_spmm(B, ii, jj, vv, Y0, dY.download())
        except AssertionError as e:
            raise AssertionError(f"case {case}: m={m} n={n} nnz={nnz} k={k} {opts}: {e}") from None
        for h in (S, dA, dB, dY, dC):
            h.close()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("k", [64, 20, 50, 7, 129, 1, 3, 1030])
def test_rows_the_pattern_never_names_are_never_read(ctx, dtype, k):
    # the reference touches A[ii[e]], B[jj[e]] and Y[ii[e]] only (core_ops.cpp:16,32): NaN
    # in every other dense row must not reach any result, whatever the batching loads
    m, n, nnz = 90, 120, 1500
    ii, jj, vv, A, B, Y0 = rand_case(77 + k, m, n, k, nnz, dtype, hub=400)
    ii = (ii // 2 * 2).astype(np.uint32)       # odd rows are never named
    jj = (jj // 3 * 3).astype(np.uint32)       # two columns in three are never named
    A[1::2] = np.nan
    B[np.arange(n) % 3 != 0] = np.nan
    C = gpu_sddmm(ctx, m, n, ii, jj, vv, A, B)
    assert np.all(np.isfinite(C))
    Aclean, Bclean = np.nan_to_num(A), np.nan_to_num(B)
    check_sddmm(Aclean, Bclean, ii, jj, vv, C)
    Y0[1::2] = np.nan
    Y = gpu_spmm(ctx, m, n, ii, jj, vv, B, Y0)
    assert np.all(np.isnan(Y[1::2])) and np.all(np.isfinite(Y[0::2]))
    check_spmm(Bclean, ii, jj, vv, np.nan_to_num(Y0), np.nan_to_num(Y))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("k", [64, 50, 7, 129, 3, 2, 1, 1027])
def test_non_finite_inputs_propagate_as_in_the_reference(ctx, dtype, k):
    # an infinite X row named with weight a gives a * inf in Y, not NaN from 0 * inf
    # (nor, at widths that end inside a vector, from the elements a lane loads but does
    # not count)
    m, n = 8, 8
    ii = np.array([0, 0, 0, 0, 0, 3], dtype=np.uint32)
    jj = np.array([1, 2, 3, 4, 5, 5], dtype=np.uint32)
    vv = np.array([1, 1, 1, 1, 2, 1], dtype=dtype)
    X = np.ones((n, k), dtype=dtype)
    X[5] = np.inf
    Y = gpu_spmm(ctx, m, n, ii, jj, vv, X, np.zeros((m, k), dtype=dtype))
    assert np.all(np.isposinf(Y[0])) and np.all(np.isposinf(Y[3])) and np.all(Y[1] == 0)
    C = gpu_sddmm(ctx, m, n, ii, jj, vv, np.ones((m, k), dtype=dtype), X)
    assert np.array_equal(C[:4], np.full(4, k, dtype=dtype)) and np.all(np.isposinf(C[4:]))
    # one infinite element at a time, in each of the last positions of a row (those a lane
    # may hold twice at such widths): inf in C and in that one element of Y, never NaN
    for back in range(1, min(k, 5)):
        X = np.ones((n, k), dtype=dtype)
        X[6, k - back] = np.inf
        A = np.ones((m, k), dtype=dtype)
        A[2, k - back] = np.inf
        ii2, jj2 = np.array([1, 2], dtype=np.uint32), np.array([6, 0], dtype=np.uint32)
        C = gpu_sddmm(ctx, m, n, ii2, jj2, np.ones(2, dtype=dtype), A, X)
        assert np.all(np.isposinf(C)), (back, C)
        Y = gpu_spmm(ctx, m, n, ii2, jj2, np.ones(2, dtype=dtype), X, np.zeros((m, k), dtype=dtype))
        want = np.zeros((m, k), dtype=dtype)
        want[1], want[2] = X[6], X[0]
        assert np.array_equal(Y, want), back


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nnz", [0, 1, 2, 15, 16, 17, 63, 65])
def test_tiny_and_ragged(ctx, dtype, nnz):
    ii, jj, vv, A, B, Y0 = rand_case(nnz, 5, 9, 64, nnz, dtype)
    C = gpu_sddmm(ctx, 5, 9, ii, jj, vv, A, B)
    Y = gpu_spmm(ctx, 5, 9, ii, jj, vv, B, Y0)
    if nnz == 0:
        assert C.size == 0 and np.array_equal(Y, Y0)
        return
    check_sddmm(A, B, ii, jj, vv, C)
    check_spmm(B, ii, jj, vv, Y0, Y)


@pytest.mark.parametrize("dtype", DTYPES)
def test_rectangular_empty_rows_untouched(ctx, dtype):
    # only rows 3 and 40 of 100 have entries; every other Y row must come back bit-identical
    rng = np.random.default_rng(5)
    ii = np.concatenate([np.full(20, 3), np.full(300, 40)]).astype(np.uint32)
    jj = rng.integers(0, 7, 320).astype(np.uint32)
    vv = rng.random(320).astype(dtype)
    X = rng.uniform(-1, 1, (7, 32)).astype(dtype)
    Y0 = rng.uniform(-1, 1, (100, 32)).astype(dtype)
    Y = gpu_spmm(ctx, 100, 7, ii, jj, vv, X, Y0)
    untouched = np.setdiff1d(np.arange(100), [3, 40])
    assert np.array_equal(Y[untouched], Y0[untouched])
    check_spmm(X, ii, jj, vv, Y0, Y)


# ---- semantics the reference fixes ----------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
def test_sddmm_overwrites_every_entry_in_callers_order(ctx, dtype):
    ii, jj, vv, A, B, _ = rand_case(21, 40, 40, 16, 900, dtype)
    C1 = gpu_sddmm(ctx, 40, 40, ii, jj, vv, A, B, prefill=np.nan)
    assert np.all(np.isfinite(C1))
    p = np.random.default_rng(2).permutation(ii.size)
    C2 = gpu_sddmm(ctx, 40, 40, ii[p], jj[p], vv[p], A, B)
    # per-entry results do not depend on where the entry sits in the stream
    assert np.array_equal(C2, C1[p])


@pytest.mark.parametrize("dtype", DTYPES)
def test_spmm_accumulates_over_calls(ctx, dtype):
    # miniapp/bench_spmm.cpp:185-186 never resets Y between its five calls
    ii, jj, vv, _, X, Y0 = rand_case(22, 50, 60, 32, 2000, dtype, hub=300)
    Y3 = gpu_spmm(ctx, 50, 60, ii, jj, vv, X, Y0, times=3)
    ref = Y0
    for _ in range(3):
        ref = oracle.spmm(X, ii, jj, vv, ref)
    scale = oracle.spmm_scale(X, ii, jj, 3 * vv.astype(np.float64), Y0)
    assert oracle.rel_err(Y3, ref, scale) <= tol_of(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_exact_cases(ctx, dtype):
    # ones panels: C = K * S exactly (miniapp/bench_both.cpp:191-192); X = 1: row sums
    ii, jj, vv, _, _, _ = rand_case(23, 30, 30, 64, 700, dtype)
    one = np.ones((30, 64), dtype)
    C = gpu_sddmm(ctx, 30, 30, ii, jj, vv, one, one)
    assert np.array_equal(C, (64 * vv).astype(dtype))
    eye = np.arange(30, dtype=np.uint32)
    X = np.random.default_rng(3).uniform(-1, 1, (30, 64)).astype(dtype)
    Y0 = np.random.default_rng(4).uniform(-1, 1, (30, 64)).astype(dtype)
    Y = gpu_spmm(ctx, 30, 30, eye, eye, np.ones(30, dtype), X, Y0)
    assert np.array_equal(Y, Y0 + X)


@pytest.mark.parametrize("dtype", DTYPES)
def test_runs_are_bitwise_reproducible(ctx, dtype):
    ii, jj, vv, A, B, Y0 = rand_case(24, 64, 64, 64, 9000, dtype, hub=4000)
    a = gpu_spmm(ctx, 64, 64, ii, jj, vv, B, Y0)
    b = gpu_spmm(ctx, 64, 64, ii, jj, vv, B, Y0)
    assert np.array_equal(a, b)
    c = gpu_sddmm(ctx, 64, 64, ii, jj, vv, A, B)
    d = gpu_sddmm(ctx, 64, 64, ii, jj, vv, A, B)
    assert np.array_equal(c, d)


# ---- the other entry points -------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
def test_one_shot_host_entry_points(ctx, dtype):
    ii, jj, vv, A, B, Y0 = rand_case(31, 70, 90, 64, 3000, dtype, hub=500)
    check_sddmm(A, B, ii, jj, vv, ctx.sddmm_host(A, B, ii, jj, vv))
    Y = Y0.copy()
    ctx.spmm_host(B, ii, jj, vv, Y)
    check_spmm(B, ii, jj, vv, Y0, Y)


def test_one_shot_host_calls_at_the_edges(ctx):
    """Repeated one-shot calls that alternate types, widths and shapes over one context:
    whatever the context keeps between calls, every result is the oracle's.  Also an empty
    pattern, a single entry, and a dense operand of one column."""
    rng = np.random.default_rng(5)
    for rep in range(2):
        for dtype, k, m, n, nnz in ((np.float64, 1, 9, 7, 20), (np.float32, 3, 9, 7, 20),
                                    (np.float64, 64, 300, 200, 5000), (np.float32, 64, 300, 200, 5000),
                                    (np.float64, 33, 300, 200, 1), (np.float32, 50, 1, 1, 1)):
            ii, jj, vv, A, B, Y0 = rand_case(40 + rep, m, n, k, nnz, dtype)
            check_sddmm(A, B, ii, jj, vv, ctx.sddmm_host(A, B, ii, jj, vv))
            Y = Y0.copy()
            ctx.spmm_host(B, ii, jj, vv, Y)
            check_spmm(B, ii, jj, vv, Y0, Y)
            Y1 = Y.copy()
            ctx.spmm_host(B, ii, jj, vv, Y)  # accumulates over calls (core_ops.cpp:32)
            check_spmm(B, ii, jj, vv, Y1, Y)
    # an empty pattern: nothing is written
    A, B = rng.uniform(-1, 1, (5, 8)), rng.uniform(-1, 1, (6, 8))
    none = np.zeros(0, dtype=np.uint32)
    assert ctx.sddmm_host(A, B, none, none, np.zeros(0)).size == 0
    Y = np.ones((5, 8))
    ctx.spmm_host(B, none, none, np.zeros(0), Y)
    assert np.array_equal(Y, np.ones((5, 8)))


def test_values_can_be_replaced_from_host_and_device(ctx):
    ii, jj, vv, A, B, _ = rand_case(32, 40, 40, 32, 1500, np.float64)
    S = ctx.plan(40, 40, ii, jj, dtype=np.float64)  # pattern only
    dA, dB, dC = ctx.panel_from(A), ctx.panel_from(B), ctx.vals(1500, np.float64)
    with pytest.raises(capi.Spc3dError):
        ctx.sddmm(S, dA, dB, dC)  # no values yet
    S.set_values(vv)
    ctx.sddmm(S, dA, dB, dC)
    check_sddmm(A, B, ii, jj, vv, dC.download())
    v2 = (vv * 0.5 + 0.125)
    dV = ctx.vals(1500, np.float64)
    dV.upload(v2)
    S.set_values_device(dV)
    ctx.sddmm(S, dA, dB, dC)
    check_sddmm(A, B, ii, jj, v2, dC.download())
    # SDDMM output feeding the next SpMM as its values, all on the device
    S.set_values_device(dC)
    dY = ctx.panel_from(np.zeros((40, 32)))
    ctx.spmm(S, dB, dY)
    check_spmm(B, ii, jj, oracle.sddmm(A, B, ii, jj, v2), np.zeros((40, 32)), dY.download())


def test_shape_and_dtype_mismatches_are_refused(ctx):
    ii, jj, vv, A, B, Y0 = rand_case(33, 20, 30, 16, 200, np.float64)
    S = ctx.plan(20, 30, ii, jj, vv)
    dA, dB = ctx.panel_from(A), ctx.panel_from(B)
    dC = ctx.vals(200, np.float64)
    cases = [
        lambda: ctx.sddmm(S, dA, ctx.panel_from(B[:, :8].copy()), dC),       # A.n != B.n
        lambda: ctx.sddmm(S, ctx.panel_from(A[:10].copy()), dB, dC),         # A too short
        lambda: ctx.sddmm(S, dA, dB, ctx.vals(199, np.float64)),             # C.vv too short
        lambda: ctx.sddmm(S, dA, dB, ctx.vals(200, np.float32)),             # dtype
        lambda: ctx.spmm(S, dB, ctx.panel_from(Y0[:, :8].copy())),           # X.n != Y.n
        lambda: ctx.spmm(S, ctx.panel_from(B[:29].copy()), ctx.panel_from(Y0)),  # X too short
        lambda: ctx.spmm(S, dB, dB),                                         # aliasing
    ]
    for c in cases:
        with pytest.raises(capi.Spc3dError) as e:
            c()
        assert e.value.status in (capi.ERR_SIZE_MISMATCH, capi.ERR_INVALID_ARG)
    with pytest.raises(IndexError):
        ctx.plan(20, 29, ii, np.full_like(jj, 29), vv)


# ---- the benchmark configurations at oracle-sized scale -----------------------------
@pytest.mark.parametrize("dtype", DTYPES)
def test_config1_erdos_renyi_full(ctx, dtype):
    w = W.erdos_renyi(16384, 16, 32)
    A, B, vv = w.panel_A(dtype), w.panel_B(dtype), w.values(dtype)
    C = gpu_sddmm(ctx, w.nrows, w.ncols, w.ii, w.jj, vv, A, B)
    check_sddmm(A, B, w.ii, w.jj, vv, C)
    Y0 = np.zeros_like(A)
    Y = gpu_spmm(ctx, w.nrows, w.ncols, w.ii, w.jj, C, B, Y0)  # SDDMM then SpMM
    check_spmm(B, w.ii, w.jj, C, Y0, Y)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("order", ["sorted", "shuffled"])
def test_config2_rmat_scale16(ctx, dtype, order):
    w = W.rmat(16, 16, 64)
    if order == "shuffled":
        w = w.shuffled()
    A, B, Y0, vv = w.panel_A(dtype), w.panel_B(dtype), w.panel_Y0(dtype), w.values(dtype)
    check_sddmm(A, B, w.ii, w.jj, vv, gpu_sddmm(ctx, w.nrows, w.ncols, w.ii, w.jj, vv, A, B))
    check_spmm(B, w.ii, w.jj, vv, Y0, gpu_spmm(ctx, w.nrows, w.ncols, w.ii, w.jj, vv, B, Y0))


def test_config4_stencil_256(ctx):
    w = W.stencil5(256, 256, 32)
    A, B, Y0, vv = (w.panel_A("f32"), w.panel_B("f32"), w.panel_Y0("f32"), w.values("f32"))
    check_sddmm(A, B, w.ii, w.jj, vv, gpu_sddmm(ctx, w.nrows, w.ncols, w.ii, w.jj, vv, A, B))
    check_spmm(B, w.ii, w.jj, vv, Y0, gpu_spmm(ctx, w.nrows, w.ncols, w.ii, w.jj, vv, B, Y0))


def test_config5_hypergraph_small_k128(ctx):
    w = W.hypergraph_zipf(20000, 5000, 128)
    A, B, Y0, vv = (w.panel_A("f32"), w.panel_B("f32"), w.panel_Y0("f32"), w.values("f32"))
    check_sddmm(A, B, w.ii, w.jj, vv, gpu_sddmm(ctx, w.nrows, w.ncols, w.ii, w.jj, vv, A, B))
    check_spmm(B, w.ii, w.jj, vv, Y0, gpu_spmm(ctx, w.nrows, w.ncols, w.ii, w.jj, vv, B, Y0))


# ---- optional plan layouts ------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
def test_xcd_sliced_plan_matches_oracle(ctx, dtype):
    # a small planned L2 share so that slicing engages on this 2^15-column panel
    w = W.rmat(15, 16, 64).shuffled()
    A, B, Y0, vv = w.panel_A(dtype), w.panel_B(dtype), w.panel_Y0(dtype), w.values(dtype)
    S = ctx.plan(w.nrows, w.ncols, w.ii, w.jj, vv, xcd_slices=8, l2_hot_bytes=64 * 1024,
                 hub_min=32, seg_max=256)
    assert S.info.nqueues == 8 and S.info.hub_rows > 0
    dA, dB, dY, dC = ctx.panel_from(A), ctx.panel_from(B), ctx.panel_from(Y0), ctx.vals(w.nnz, dtype)
    ctx.sddmm(S, dA, dB, dC)
    ctx.spmm(S, dB, dY)
    check_sddmm(A, B, w.ii, w.jj, vv, dC.download())
    check_spmm(B, w.ii, w.jj, vv, Y0, dY.download())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("k", [64, 50, 3, 1030])
def test_staged_results_of_hub_row_pieces_reach_the_callers_positions(ctx, dtype, k):
    """Sorted input whose hub rows are cut by column slice: the pieces' results are written
    in kernel order to a staging vector and brought to C by one ordered pass (plan info
    staged_entries > 0), the other segments read one position each.  Every entry of C must be
    overwritten, through spc3d_sddmm and both forms of spc3d_sddmm_spmm, call after call,
    also for dense rows over 4 KiB (several launches that accumulate in place)."""
    w = W.rmat(14, 16, k)
    A, B, Y0, vv = w.panel_A(dtype), w.panel_B(dtype), w.panel_Y0(dtype), w.values(dtype)
    S = ctx.plan(w.nrows, w.ncols, w.ii, w.jj, vv, xcd_slices=8, l2_hot_bytes=64 * 1024,
                 hub_min=32, seg_max=256)
    I = S.info
    assert I.nqueues == 8 and I.hub_rows > 0 and I.order_is_identity == 0
    assert 0 < I.staged_entries < w.nnz, I.staged_entries
    dA, dB, dY, dC = ctx.panel_from(A), ctx.panel_from(B), ctx.panel_from(Y0), ctx.vals(w.nnz, dtype)
    for _ in range(2):
        dC.fill(np.nan)
        ctx.sddmm(S, dA, dB, dC)
        check_sddmm(A, B, w.ii, w.jj, vv, dC.download())
    first = dC.download()
    if k * np.dtype(dtype).itemsize <= 4096:
        dC.fill(np.nan)
        ctx.sddmm_spmm(S, dA, dB, dC, dY)
        assert np.array_equal(dC.download(), first)
        check_spmm(B, w.ii, w.jj, vv, Y0, dY.download())
        dC.fill(np.nan)
        dY.upload(Y0)
        ctx.sddmm_spmm(S, dA, dB, dC, dY, chained=True)
        assert np.array_equal(dC.download(), first)
        check_spmm(B, w.ii, w.jj, first, Y0, dY.download())
    # new values through the original order, then the same plan again
    vv2 = (vv * 0.5 + 1).astype(dtype)
    S.set_values(vv2)
    dC.fill(np.nan)
    ctx.sddmm(S, dA, dB, dC)
    check_sddmm(A, B, w.ii, w.jj, vv2, dC.download())
    for h in (S, dA, dB, dY, dC):
        h.close()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("k", [64, 7, 1030])
def test_column_sorted_input_runs_sddmm_through_the_exchanged_plan(ctx, dtype, k):
    """A pattern sorted by column (the order of a MatrixMarket file): spc3d_sddmm runs the plan
    of the same entries with rows and columns exchanged, A and B exchanged with them (plan info
    sddmm_by_column).  The results are those of the row-major plan bit for bit (the one-pass
    call still runs that one), SpMM is untouched, new values reach both plans."""
    w = W.rmat(14, 16, k)
    o = np.lexsort((w.ii, w.jj))
    ii, jj = np.ascontiguousarray(w.ii[o]), np.ascontiguousarray(w.jj[o])
    A, B, Y0 = w.panel_A(dtype), w.panel_B(dtype), w.panel_Y0(dtype)
    vv = np.ascontiguousarray(w.values(dtype)[o])
    S = ctx.plan(w.nrows, w.ncols, ii, jj, vv, xcd_slices=8, l2_hot_bytes=64 * 1024, hub_min=32,
                 seg_max=256)
    assert S.info.sddmm_by_column == 1 and S.info.order_is_identity == 0
    dA, dB, dY, dC = ctx.panel_from(A), ctx.panel_from(B), ctx.panel_from(Y0), ctx.vals(w.nnz, dtype)
    for _ in range(2):
        dC.fill(np.nan)
        ctx.sddmm(S, dA, dB, dC)
        check_sddmm(A, B, ii, jj, vv, dC.download())
    by_col = dC.download()
    ctx.spmm(S, dB, dY)
    check_spmm(B, ii, jj, vv, Y0, dY.download())
    if k * np.dtype(dtype).itemsize <= 4096:
        dC.fill(np.nan)
        dY.upload(Y0)
        ctx.sddmm_spmm(S, dA, dB, dC, dY)
        assert np.array_equal(dC.download(), by_col)
        check_spmm(B, ii, jj, vv, Y0, dY.download())
    vv2 = (vv * 0.25 - 1).astype(dtype)
    S.set_values(vv2)
    dC.fill(np.nan)
    ctx.sddmm(S, dA, dB, dC)
    check_sddmm(A, B, ii, jj, vv2, dC.download())
    dv = ctx.vals(w.nnz, dtype)
    dv.upload(vv)
    S.set_values_device(dv)
    ctx.sddmm(S, dA, dB, dC)
    assert np.array_equal(dC.download(), by_col)
    # rectangular, and sorted by column only (rows inside a column in any order)
    ii2, jj2, vv3, A2, B2, _ = rand_case(11, 300, 90, k, 5000, dtype, hub=900)
    o2 = np.argsort(jj2, kind="stable")
    ii2, jj2, vv3 = (np.ascontiguousarray(x[o2]) for x in (ii2, jj2, vv3))
    S2 = ctx.plan(300, 90, ii2, jj2, vv3)
    assert S2.info.sddmm_by_column == 1
    dA2, dB2, dC2 = ctx.panel_from(A2), ctx.panel_from(B2), ctx.vals(5000, dtype)
    dC2.fill(np.nan)
    ctx.sddmm(S2, dA2, dB2, dC2)
    check_sddmm(A2, B2, ii2, jj2, vv3, dC2.download())
    for h in (S, S2, dA, dB, dY, dC, dv, dA2, dB2, dC2):
        h.close()


@pytest.mark.parametrize("dtype", DTYPES)
def test_arbitrary_order_brings_results_home_in_two_passes(ctx, dtype):
    """An arbitrary entry order: the kernels write in kernel order, two passes of tile-local
    moves bring the results to the caller's positions (plan info two_pass_results; from 1.5 M
    entries on by default, here from the smallest size the scheme takes).  Bit for bit what the
    plain plan stores, through spc3d_sddmm and both one-pass forms, wide rows included, and
    into a wrapped value vector."""
    w = W.rmat(14, 16, 64).shuffled()
    A, B, Y0, vv = w.panel_A(dtype), w.panel_B(dtype), w.panel_Y0(dtype), w.values(dtype)
    plain = ctx.plan(w.nrows, w.ncols, w.ii, w.jj, vv, two_pass=False, two_pass_min=1)
    S = ctx.plan(w.nrows, w.ncols, w.ii, w.jj, vv, two_pass_min=1)
    tiny = ctx.plan(w.nrows, w.ncols, w.ii[:1000], w.jj[:1000], vv[:1000],
                    two_pass_min=1)  # under two tiles
    assert plain.info.two_pass_results == 0 and tiny.info.two_pass_results == 0
    assert S.info.two_pass_results == 1 and S.info.staged_entries == 0
    dA, dB, dY, dC = ctx.panel_from(A), ctx.panel_from(B), ctx.panel_from(Y0), ctx.vals(w.nnz, dtype)
    ctx.sddmm(plain, dA, dB, dC)
    want = dC.download()
    check_sddmm(A, B, w.ii, w.jj, vv, want)
    for _ in range(2):
        dC.fill(np.nan)
        ctx.sddmm(S, dA, dB, dC)
        assert np.array_equal(dC.download(), want)
    for chained in (False, True):
        dC.fill(np.nan)
        dY.upload(Y0)
        ctx.sddmm_spmm(S, dA, dB, dC, dY, chained=chained)
        assert np.array_equal(dC.download(), want)
        check_spmm(B, w.ii, w.jj, want if chained else vv, Y0, dY.download())
    lead = 16 // np.dtype(dtype).itemsize  # C some way into a vector the caller owns
    big = ctx.vals(w.nnz + 3 * lead, dtype)
    big.fill(np.nan)
    inner = device.Vals(ctx, w.nnz, dtype, dev=big.device_ptr() + 3 * 16)
    ctx.sddmm(S, dA, dB, inner)
    assert np.array_equal(big.download()[3 * lead:], want)
    inner.close()
    big.close()
    # SpMM and the plan's own arrays know nothing of it
    dY.upload(Y0)
    ctx.spmm(S, dB, dY)
    check_spmm(B, w.ii, w.jj, vv, Y0, dY.download())
    assert np.array_equal(S.download()["perm"], plain.download()["perm"])
    # rows over 4 KiB: several launches that accumulate in the staging vector
    wk = W.rmat(14, 16, 1030).shuffled()
    Ak, Bk = wk.panel_A(dtype), wk.panel_B(dtype)
    dAk, dBk = ctx.panel_from(Ak), ctx.panel_from(Bk)
    dC.fill(np.nan)
    ctx.sddmm(S, dAk, dBk, dC)
    check_sddmm(Ak, Bk, w.ii, w.jj, vv, dC.download())
    for h in (S, plain, tiny, dA, dB, dY, dC, dAk, dBk):
        h.close()


def test_a_shuffled_pattern_keeps_its_stores_unstaged(ctx):
    # every segment's positions are scattered and so would be the final pass: no staging
    w = W.rmat(14, 16, 64).shuffled()
    S = ctx.plan(w.nrows, w.ncols, w.ii, w.jj, w.values(np.float32))
    assert S.info.order_is_identity == 0 and S.info.staged_entries == 0
    assert S.info.sddmm_by_column == 0
    S.close()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nblocks", [2, 7, 300])
def test_plan_in_column_blocks_matches_oracle(ctx, dtype, nblocks):
    """A pattern kept in column blocks (one plan per block, run one after the other):
    same results as the whole plan up to summation order, in the caller's order."""
    w = W.rmat(12, 24, 40).shuffled()
    A, B, Y0, vv = w.panel_A(dtype), w.panel_B(dtype), w.panel_Y0(dtype), w.values(dtype)
    S = ctx.plan(w.nrows, w.ncols, w.ii, w.jj, vv, col_blocks=nblocks, seg_max=32, k_hint=w.k)
    info = S.info
    assert 1 < info.ncol_blocks <= nblocks and info.nnz == w.nnz
    assert info.nsegments >= info.rows_touched and not info.order_is_identity
    with pytest.raises(capi.Spc3dError):
        S.download()  # one set of arrays per block, none for the pattern
    dA, dB, dY = ctx.panel_from(A), ctx.panel_from(B), ctx.panel_from(Y0)
    dC = ctx.vals(w.nnz, dtype)
    dC.fill(float("nan"))
    ctx.sddmm(S, dA, dB, dC)
    ctx.spmm(S, dB, dY)
    check_sddmm(A, B, w.ii, w.jj, vv, dC.download())
    check_spmm(B, w.ii, w.jj, vv, Y0, dY.download())
    # the one-pass call and the call that allocates nothing go block by block as well
    dY2, dY3, dC2 = ctx.panel_from(Y0), ctx.panel_from(Y0), ctx.vals(w.nnz, dtype)
    ctx.sddmm_spmm(S, dA, dB, dC2, dY2)
    ctx.spmm_noalloc(S, dB, dY3)
    check_sddmm(A, B, w.ii, w.jj, vv, dC2.download())
    check_spmm(B, w.ii, w.jj, vv, Y0, dY2.download())
    assert np.array_equal(dY3.download(), dY.download())
    # new values, from the host and from the device
    vv2 = (vv * 3 + 1).astype(vv.dtype)
    S.set_values(vv2)
    ctx.sddmm(S, dA, dB, dC)
    check_sddmm(A, B, w.ii, w.jj, vv2, dC.download())
    dv = ctx.vals(w.nnz, dtype)
    dv.upload(vv)
    S.set_values_device(dv)
    ctx.sddmm(S, dA, dB, dC)
    check_sddmm(A, B, w.ii, w.jj, vv, dC.download())
    for h in (S, dA, dB, dY, dY2, dY3, dC, dC2, dv):
        h.close()


def test_column_blocks_are_chosen_for_long_rows_over_a_wide_unskewed_panel(ctx):
    # 140 k columns of 512 bytes (68 MiB, uniform), rows of 890 entries in the weighted
    # mean: the rule picks blocks; R-MAT (skewed columns) and short rows stay whole
    w = W.hypergraph_zipf(3000, 140_000, 128)
    vv = w.values("f32")
    S = ctx.plan(w.nrows, w.ncols, w.ii, w.jj, vv, k_hint=w.k, sweep=False)
    assert 12 <= S.info.ncol_blocks <= 14 and S.info.nqueues == 1, S.info.ncol_blocks
    # 512-byte rows are a width the row-tile kernels take: by default the long rows go there
    T = ctx.plan(w.nrows, w.ncols, w.ii, w.jj, vv, k_hint=w.k)
    assert T.info.sweep_entries > w.nnz // 2 and 20 <= T.info.ncol_blocks <= 22
    T.close()
    whole = ctx.plan(w.nrows, w.ncols, w.ii, w.jj, vv, k_hint=w.k, col_blocks=1)
    assert whole.info.ncol_blocks == 1
    A, B, Y0 = w.panel_A("f32"), w.panel_B("f32"), w.panel_Y0("f32")
    dA, dB, dY, dC = ctx.panel_from(A), ctx.panel_from(B), ctx.panel_from(Y0), ctx.vals(w.nnz, "f32")
    ctx.sddmm(S, dA, dB, dC)
    ctx.spmm(S, dB, dY)
    check_sddmm(A, B, w.ii, w.jj, vv, dC.download())
    check_spmm(B, w.ii, w.jj, vv, Y0, dY.download())
    for h in (S, whole, dA, dB, dY, dC):
        h.close()
    for other in (W.rmat(16, 16, 64), W.stencil5(256, 256, 32), W.erdos_renyi(16384, 16, 32)):
        P = ctx.plan(other.nrows, other.ncols, other.ii, other.jj, other.values("f32"),
                     k_hint=other.k)
        assert P.info.ncol_blocks == 1
        P.close()


def test_workgroups_are_dealt_to_xcds_round_robin(ctx):
    # what the XCD-sliced plan layout relies on for its speed (not for its results)
    # round-robin by workgroup id, from a starting XCD that is fixed per hardware queue
    x = ctx.probe_xcd(1024).astype(np.int64)
    assert np.array_equal((x - x[0]) % 8, np.arange(1024) % 8)
    assert np.array_equal(ctx.probe_xcd(13).astype(np.int64)[:8], x[:8])  # same start every time


@pytest.mark.parametrize("shape", [(1000, 33), (1001, 33), (3, 1), (70000, 64)])
def test_panel_copy_on_device(ctx, shape):
    # sizes with and without a 16-byte tail, below and above one block's span
    a = np.random.default_rng(0).uniform(-1, 1, shape).astype(np.float32)
    src, dst = ctx.panel_from(a), ctx.panel(shape[0], shape[1], np.float32)
    dst.fill(7.0)
    dst.copy_from(src)
    assert np.array_equal(dst.download(), a)
    with pytest.raises(capi.Spc3dError):
        ctx.panel(shape[0], shape[1] + 1, np.float32).copy_from(src)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("col_blocks", [None, 3, "tiles"])
def test_probe_columns_keeps_the_launches_and_moves_the_gathers(ctx, dtype, col_blocks):
    """spc3d_plan_probe_columns (a measurement aid): after the all-hit rewrite the plan
    computes the pattern (ii, c % modulus inside the entry's block of columns), entry by
    entry at the caller's positions; after the all-miss one every column is in range."""
    w = W.rmat(12, 16, 32).shuffled()
    vv, A, B, Y0 = w.values(dtype), w.panel_A(dtype), w.panel_B(dtype), w.panel_Y0(dtype)
    if col_blocks == "tiles":  # row tiles for the rows of 8 entries and more, in 3 blocks:
        # one range of columns for every block, in the tiles and in the plan of the rest
        w = W.rmat(12, 16, 64).shuffled()
        vv, A, B, Y0 = w.values(dtype), w.panel_A(dtype), w.panel_B(dtype), w.panel_Y0(dtype)
        S = ctx.plan(w.nrows, w.ncols, w.ii, w.jj, vv, k_hint=w.k, sweep=True, sweep_min_row=8,
                     col_blocks=3)
        assert 0 < S.info.sweep_entries < w.nnz
        col_blocks = None
    else:
        S = ctx.plan(w.nrows, w.ncols, w.ii, w.jj, vv, k_hint=w.k, col_blocks=col_blocks)
    dA, dB, dY, dC = ctx.panel_from(A), ctx.panel_from(B), ctx.panel_from(Y0), ctx.vals(w.nnz, dtype)
    modulus = 61
    S.probe_columns("all_hit", modulus)
    nb = S.info.ncol_blocks if col_blocks else 1
    bc = (w.ncols + nb - 1) // nb if nb > 1 else w.ncols
    base = (w.jj // bc) * bc
    jj2 = (base + (w.jj - base) % modulus).astype(np.uint32)
    ctx.sddmm(S, dA, dB, dC)
    ctx.spmm(S, dB, dY)
    check_sddmm(A, B, w.ii, jj2, vv, dC.download())
    check_spmm(B, w.ii, jj2, vv, Y0, dY.download())
    S.probe_columns("all_miss")
    dY.upload(Y0)
    ctx.sddmm(S, dA, dB, dC)
    ctx.spmm(S, dB, dY)
    ctx.sync()  # every gather stayed inside B: nothing to fault on, finite results
    assert np.isfinite(dC.download()).all() and np.isfinite(dY.download()).all()
    for h in (S, dA, dB, dY, dC):
        h.close()
