"""Seeded random sequences of the one-shot host calls (spc3d_sddmm_host, spc3d_spmm_host) over
operands that change in place between calls, the way the reference's benches reuse their
arrays (ReMapIndices rewrites ii / jj at the same addresses, miniapp/bench_both.cpp:200-205):
what the context kept from earlier calls may only answer for operands whose contents still
hold.  Every result is judged against the oracle run in double."""
import numpy as np
import pytest

from spcomm3d_amd import device
from tests import _oracle as oracle

pytestmark = pytest.mark.gpu

TOL = {np.dtype(np.float32): 1e-5, np.dtype(np.float64): 1e-12}


def new_state(rng):
    dtype = [np.float32, np.float64][int(rng.integers(2))]
    m, n = (int(rng.choice([50, 3000, 40000])) for _ in range(2))
    k = int(rng.choice([8, 64, 130]))
    nnz = int(rng.choice([100, 100000, 1500000]))  # (panels and index arrays over one 4 MiB block too)
    ii = rng.integers(0, m, nnz).astype(np.uint32)
    jj = rng.integers(0, n, nnz).astype(np.uint32)
    if rng.random() < 0.5:
        o = np.lexsort((jj, ii))
        ii, jj = np.ascontiguousarray(ii[o]), np.ascontiguousarray(jj[o])
    return dict(dtype=dtype, m=m, n=n, k=k, ii=ii, jj=jj, vv=rng.random(nnz).astype(dtype),
                A=rng.uniform(-1, 1, (m, k)).astype(dtype),
                B=rng.uniform(-1, 1, (n, k)).astype(dtype),
                Y=rng.uniform(-1, 1, (m, k)).astype(dtype))


def mutate(rng, s):
    """One change in place (or none): the addresses stay, the contents do not."""
    what = str(rng.choice(["none", "A1", "B1", "v1", "Y1", "swap", "col", "scaleA", "pattern",
                           "Yall", "Bblock", "none"]))
    nnz = s["ii"].size
    if what == "A1":
        s["A"][rng.integers(s["m"]), rng.integers(s["k"])] += 1
    elif what == "B1":
        s["B"][rng.integers(s["n"]), rng.integers(s["k"])] += 1
    elif what == "v1":
        s["vv"][rng.integers(nnz)] += 1
    elif what == "Y1":
        s["Y"][rng.integers(s["m"]), rng.integers(s["k"])] += 1
    elif what == "swap":  # two entries trade places: the same pattern in another order
        a, b = rng.integers(nnz, size=2)
        for key in ("ii", "jj"):
            s[key][a], s[key][b] = s[key][b], s[key][a]
    elif what == "col":
        s["jj"][rng.integers(nnz)] = rng.integers(s["n"])
    elif what == "scaleA":
        s["A"] *= s["dtype"](0.5)
    elif what == "pattern":
        s["ii"][:] = rng.integers(0, s["m"], nnz)
        s["jj"][:] = rng.integers(0, s["n"], nnz)
    elif what == "Yall":
        s["Y"][:] = rng.uniform(-1, 1, s["Y"].shape)
    elif what == "Bblock":
        r = int(rng.integers(s["n"]))
        s["B"][r:r + 1000] *= s["dtype"](-1)
    return what


@pytest.mark.parametrize("threads,seed", [(1, 500), (4, 501)])
def test_random_sequences_of_one_shot_calls_over_operands_changed_in_place(threads, seed):
    rng = np.random.default_rng(seed)
    with device.Context(0, host_threads=threads) as ctx:
        states = [new_state(rng) for _ in range(3)]
        for step in range(60):
            si = int(rng.integers(len(states)))
            if rng.random() < 0.05:
                states[si] = new_state(rng)
            s = states[si]
            what = mutate(rng, s)
            op = str(rng.choice(["sddmm", "spmm", "sddmm_swapped"]))
            tag = (threads, seed, step, si, what, op)
            tol = TOL[np.dtype(s["dtype"])]
            if op == "sddmm":
                C = ctx.sddmm_host(s["A"], s["B"], s["ii"], s["jj"], s["vv"])
                err = oracle.sddmm_rel_err_exact(s["A"], s["B"], s["ii"], s["jj"], s["vv"], C)
            elif op == "sddmm_swapped":  # the panels trade places, the pattern its axes
                C = ctx.sddmm_host(s["B"], s["A"], s["jj"], s["ii"], s["vv"])
                err = oracle.sddmm_rel_err_exact(s["B"], s["A"], s["jj"], s["ii"], s["vv"], C)
            else:
                Y0 = s["Y"].copy()
                ctx.spmm_host(s["B"], s["ii"], s["jj"], s["vv"], s["Y"])
                err = oracle.spmm_rel_err_exact(s["B"], s["ii"], s["jj"], s["vv"], Y0, s["Y"])
            assert err <= tol, (tag, err)
