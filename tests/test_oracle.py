"""Pins the CPU oracle (oracle/spc3d_oracle.c) before anything is checked against it.

Each check is chosen so that a plausible slip in the restatement fails it:
a scale applied before / inside the sum, a transposed operand, `=` vs `+=`,
duplicates overwritten instead of added, a wrong panel stride, output written
at the sorted position instead of the caller's.
"""
import numpy as np
import pytest
import scipy.sparse as sp

from tests import _oracle as oracle

GOLDEN = np.load(oracle.os.path.join(oracle.ROOT, "tests", "golden", "core_ops_golden.npz"),
                 allow_pickle=False)
CASES = ["small", "k64", "hub", "k1"]


def _rand_case(seed, m, n, k, nnz, dtype=np.float64):
    rng = np.random.default_rng(seed)
    ii = rng.integers(0, m, nnz).astype(np.uint32)
    jj = rng.integers(0, n, nnz).astype(np.uint32)
    vv = rng.random(nnz).astype(dtype)
    A = rng.uniform(-1, 1, (m, k)).astype(dtype)
    B = rng.uniform(-1, 1, (n, k)).astype(dtype)
    Y0 = rng.uniform(-1, 1, (m, k)).astype(dtype)
    return ii, jj, vv, A, B, Y0


# ---- against the reference's own compiled code (golden vectors) -------------
@pytest.mark.parametrize("name", CASES)
def test_sddmm_f64_bit_exact_vs_reference_golden(name):
    g = {k: GOLDEN[f"{name}.{k}"] for k in ("ii", "jj", "vv", "A", "B", "C")}
    got = oracle.sddmm(g["A"], g["B"], g["ii"], g["jj"], g["vv"])
    assert np.array_equal(got, g["C"])


@pytest.mark.parametrize("name", CASES)
def test_spmm_f64_bit_exact_vs_reference_golden(name):
    g = {k: GOLDEN[f"{name}.{k}"] for k in ("ii", "jj", "vv", "B", "Y0", "Y")}
    got = oracle.spmm(g["B"], g["ii"], g["jj"], g["vv"], g["Y0"])
    assert np.array_equal(got, g["Y"])


def test_numcheck_golden_and_closed_form():
    # miniapp/numCheckSeq.cpp:125-131: A[i,:] = i/1000, B[j,:] = j/1000
    # => C_e = S_e * K * r_e * c_e / 1e6
    g = {k: GOLDEN[f"numcheck.{k}"] for k in ("ii", "jj", "vv", "A", "B", "C")}
    got = oracle.sddmm(g["A"], g["B"], g["ii"], g["jj"], g["vv"])
    assert np.array_equal(got, g["C"])
    closed = g["vv"] * 4 * g["ii"].astype(float) * g["jj"].astype(float) / 1e6
    np.testing.assert_allclose(got, closed, rtol=1e-14, atol=0)


@pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref is only built where the reference is mounted")
@pytest.mark.parametrize("seed", [1, 2, 3])
def test_f64_bit_exact_vs_live_reference_build(seed):
    ref = oracle.load_ref()
    ii, jj, vv, A, B, Y0 = _rand_case(seed, 300, 211, 33, 5000)
    p = lambda a: a.ctypes.data_as(oracle._vp)  # noqa: E731
    C = np.zeros(ii.size)
    assert ref.ref_sddmm_f64(300, 211, 33, p(A), p(B), ii.size, p(ii), p(jj), p(vv), p(C)) == 0
    assert np.array_equal(oracle.sddmm(A, B, ii, jj, vv), C)
    Y = Y0.copy()
    assert ref.ref_spmm_f64(211, 300, 33, p(B), ii.size, p(ii), p(jj), p(vv), p(Y)) == 0
    assert np.array_equal(oracle.spmm(B, ii, jj, vv, Y0), Y)


@pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref is only built where the reference is mounted")
def test_timed_reference_pass_computes_what_the_oracle_computes():
    # the entry bench.py times as the CPU baseline: SDDMM, then SpMM with the same values
    import ctypes

    ref = oracle.load_ref()
    ii, jj, vv, A, B, Y0 = _rand_case(9, 120, 120, 16, 3000)
    p = lambda a: a.ctypes.data_as(oracle._vp)  # noqa: E731
    ts, tp, cs = ctypes.c_double(), ctypes.c_double(), ctypes.c_double()
    ref.ref_time_f64.restype = ctypes.c_int
    ref.ref_time_f64.argtypes = ([ctypes.c_uint32] * 3 + [oracle._vp] * 3 + [ctypes.c_uint64] +
                                 [oracle._vp] * 3 + [ctypes.POINTER(ctypes.c_double)] * 3)
    assert ref.ref_time_f64(120, 120, 16, p(A), p(B), p(Y0), ii.size, p(ii), p(jj), p(vv),
                            ctypes.byref(ts), ctypes.byref(tp), ctypes.byref(cs)) == 0
    want = float(np.sum(oracle.sddmm(A, B, ii, jj, vv))) + float(np.sum(oracle.spmm(B, ii, jj, vv, Y0)))
    assert abs(cs.value - want) <= 1e-9 * max(1.0, abs(want))
    assert ts.value > 0 and tp.value > 0


@pytest.mark.skipif(not oracle.have_ref(), reason="oracle/_ref is only built where the reference is mounted")
def test_reference_rejects_bad_index_like_oracle():
    ref = oracle.load_ref()
    ii, jj, vv, A, B, _ = _rand_case(5, 10, 10, 4, 20)
    ii[7] = 10
    p = lambda a: a.ctypes.data_as(oracle._vp)  # noqa: E731
    C = np.zeros(20)
    assert ref.ref_sddmm_f64(10, 10, 4, p(A), p(B), 20, p(ii), p(jj), p(vv), p(C)) == -1
    with pytest.raises(IndexError):
        oracle.sddmm(A, B, ii, jj, vv)
    with pytest.raises(IndexError):
        oracle.spmm(B, ii, jj, vv, np.zeros((10, 4)))


# ---- what the mathematics fixes ----------------------------------------------
@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_sddmm_dense_brute_force(dtype):
    ii, jj, vv, A, B, _ = _rand_case(11, 23, 17, 9, 150, dtype)
    full = (A.astype(np.float64) @ B.astype(np.float64).T)
    want = full[ii, jj] * vv.astype(np.float64)
    got = oracle.sddmm(A, B, ii, jj, vv)
    tol = 1e-13 if dtype == np.float64 else 2e-6
    np.testing.assert_allclose(got, want, rtol=0, atol=tol * 9)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_sddmm_ones_gives_k_times_s(dtype):
    # miniapp/bench_both.cpp:191-192 fills both panels with one constant
    ii, jj, vv, _, _, _ = _rand_case(12, 40, 30, 16, 300, dtype)
    A = np.ones((40, 16), dtype)
    B = np.ones((30, 16), dtype)
    assert np.array_equal(oracle.sddmm(A, B, ii, jj, vv), (16 * vv).astype(dtype))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_sddmm_k1_is_elementwise_and_scale_comes_last(dtype):
    ii, jj, vv, A, B, _ = _rand_case(13, 20, 21, 1, 100, dtype)
    want = (A[ii, 0] * B[jj, 0]) * vv  # (a*b)*s in the working precision, exactly
    assert np.array_equal(oracle.sddmm(A, B, ii, jj, vv), want)


def test_sddmm_one_hot_rows_select_single_products():
    m, n, k = 6, 7, 8
    A = np.zeros((m, k))
    B = np.random.default_rng(0).uniform(-1, 1, (n, k))
    hot = np.array([3, 0, 7, 2, 5, 1])
    A[np.arange(m), hot] = 2.0
    ii = np.repeat(np.arange(m, dtype=np.uint32), n)
    jj = np.tile(np.arange(n, dtype=np.uint32), m)
    vv = np.full(ii.size, 0.5)
    got = oracle.sddmm(A, B, ii, jj, vv).reshape(m, n)
    assert np.array_equal(got, B[:, hot].T)  # 2 * b * 0.5 exactly


def test_sddmm_transpose_symmetry_and_output_position():
    ii, jj, vv, A, B, _ = _rand_case(14, 31, 19, 12, 200)
    c1 = oracle.sddmm(A, B, ii, jj, vv)
    c2 = oracle.sddmm(B, A, jj, ii, vv)  # S^T with the panels swapped
    np.testing.assert_allclose(c1, c2, rtol=1e-13)
    # result e belongs to entry e of the caller's order: permuting the entries permutes C
    perm = np.random.default_rng(1).permutation(ii.size)
    c3 = oracle.sddmm(A, B, ii[perm], jj[perm], vv[perm])
    assert np.array_equal(c3, c1[perm])


def test_sddmm_overwrites_and_ignores_previous_c():
    ii, jj, vv, A, B, _ = _rand_case(15, 9, 9, 3, 30)
    lib = oracle.load()
    p = lambda a: a.ctypes.data_as(oracle._vp)  # noqa: E731
    C = np.full(30, 1e9)
    assert lib.oracle_sddmm_f64(9, 9, 3, p(A), p(B), 30, p(ii), p(jj), p(vv), p(C)) == 0
    assert np.array_equal(C, oracle.sddmm(A, B, ii, jj, vv))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_spmm_matches_scipy_csr(dtype):
    ii, jj, vv, _, X, Y0 = _rand_case(21, 50, 40, 10, 600, dtype)
    S = sp.coo_matrix((vv.astype(np.float64), (ii, jj)), shape=(50, 40)).tocsr()  # sums duplicates
    want = Y0.astype(np.float64) + S @ X.astype(np.float64)
    got = oracle.spmm(X, ii, jj, vv, Y0)
    tol = 1e-13 if dtype == np.float64 else 3e-6
    np.testing.assert_allclose(got, want, rtol=0, atol=tol * 20)


def test_spmm_ones_gives_row_sums_identity_gives_x():
    ii, jj, vv, _, _, Y0 = _rand_case(22, 16, 16, 4, 100)
    X1 = np.ones((16, 4))
    rows = np.bincount(ii, weights=vv, minlength=16)
    np.testing.assert_allclose(oracle.spmm(X1, ii, jj, vv, Y0), Y0 + rows[:, None], rtol=1e-13)
    eye = np.arange(16, dtype=np.uint32)
    X = np.random.default_rng(2).uniform(-1, 1, (16, 4))
    assert np.array_equal(oracle.spmm(X, eye, eye, np.ones(16), Y0), Y0 + X)


def test_spmm_accumulates_duplicates_add_and_is_linear():
    ii, jj, vv, _, X, Y0 = _rand_case(23, 12, 14, 6, 80)
    y1 = oracle.spmm(X, ii, jj, vv, Y0)
    y2 = oracle.spmm(X, ii, jj, vv, y1)  # second call keeps adding
    np.testing.assert_allclose(y2 - Y0, 2 * (y1 - Y0), rtol=1e-12, atol=1e-14)
    # one entry given twice == the entry with doubled value
    e = np.array([3], dtype=np.uint32), np.array([5], dtype=np.uint32)
    twice = oracle.spmm(X, np.repeat(e[0], 2), np.repeat(e[1], 2), np.array([0.25, 0.25]), Y0)
    once = oracle.spmm(X, e[0], e[1], np.array([0.5]), Y0)
    np.testing.assert_allclose(twice, once, rtol=1e-15)
    # linear in the sparse values
    y3 = oracle.spmm(X, ii, jj, 3.0 * vv, np.zeros_like(Y0))
    np.testing.assert_allclose(y3, 3.0 * (y1 - Y0), rtol=1e-12, atol=1e-14)


def test_adjoint_identity_ties_spmm_to_sddmm():
    # <S X, A>_F == sum_e sddmm(A, X, S)_e
    ii, jj, vv, A, X, _ = _rand_case(24, 33, 27, 8, 400)
    y = oracle.spmm(X, ii, jj, vv, np.zeros((33, 8)))
    c = oracle.sddmm(A, X, ii, jj, vv)
    np.testing.assert_allclose(np.sum(y * A), np.sum(c), rtol=1e-12)


def test_f32_agrees_with_f64_within_rounding():
    ii, jj, vv, A, B, Y0 = _rand_case(31, 200, 180, 64, 4000, np.float32)
    c32 = oracle.sddmm(A, B, ii, jj, vv)
    assert c32.dtype == np.float32
    assert oracle.sddmm_rel_err_exact(A, B, ii, jj, vv, c32) < 5e-6
    y32 = oracle.spmm(B, ii, jj, vv, Y0)
    assert oracle.spmm_rel_err_exact(B, ii, jj, vv, Y0, y32) < 5e-6


def test_empty_and_scale_helpers():
    e = np.zeros(0, dtype=np.uint32)
    A = np.ones((3, 2))
    assert oracle.sddmm(A, A, e, e, np.zeros(0)).size == 0
    assert np.array_equal(oracle.spmm(A, e, e, np.zeros(0), A), A)
    ii, jj, vv, A, B, Y0 = _rand_case(41, 10, 10, 5, 40)
    s = oracle.sddmm_scale(A, B, ii, jj, vv)
    want = np.abs(vv) * np.sum(np.abs(A[ii] * B[jj]), axis=1)
    np.testing.assert_allclose(s, want, rtol=1e-13)
    assert oracle.rel_err(np.array([1.0, 0.0]), np.array([1.0, 0.0]), np.array([1.0, 0.0])) == 0.0
    assert oracle.rel_err(np.array([1.0, 1e-3]), np.array([1.0, 0.0]), np.array([1.0, 0.0])) == np.inf
