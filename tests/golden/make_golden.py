"""Writes tests/golden/core_ops_golden.npz: inputs and expected outputs of the
reference's own SpKernels::sddmm / spmm / localizeIndices.

Run in the build container only (needs oracle/_ref, which is compiled from the
reference tree by `make -C oracle ref`):

    python tests/golden/make_golden.py

The file holds data only (numpy arrays, loaded with allow_pickle=False): small
seeded inputs and the reference's fp64 outputs for them.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from tests import _oracle as oracle  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "core_ops_golden.npz")


def p(a):
    return a.ctypes.data_as(oracle._vp)


def ref_sddmm(A, B, ii, jj, vv):
    ref = oracle.load_ref()
    out = np.full(ii.size, -7.0)  # the reference overwrites every entry
    rc = ref.ref_sddmm_f64(A.shape[0], B.shape[0], A.shape[1], p(A), p(B), ii.size, p(ii), p(jj),
                           p(vv), p(out))
    assert rc == 0
    return out


def ref_spmm(X, ii, jj, vv, Y0):
    ref = oracle.load_ref()
    Y = Y0.copy()
    rc = ref.ref_spmm_f64(X.shape[0], Y.shape[0], X.shape[1], p(X), ii.size, p(ii), p(jj), p(vv),
                          p(Y))
    assert rc == 0
    return Y


def case(rng, m, n, k, nnz, hub_row=None, hub_len=0):
    ii = rng.integers(0, m, nnz).astype(np.uint32)
    jj = rng.integers(0, n, nnz).astype(np.uint32)
    if hub_row is not None:
        ii[:hub_len] = hub_row
    # a few exact duplicates (legal in COO; SpMM must add them)
    ii[-3:] = ii[:3]
    jj[-3:] = jj[:3]
    order = rng.permutation(nnz)
    ii, jj = np.ascontiguousarray(ii[order]), np.ascontiguousarray(jj[order])
    vv = rng.random(nnz)
    A = rng.uniform(-1, 1, (m, k))
    B = rng.uniform(-1, 1, (n, k))
    Y0 = rng.uniform(-1, 1, (m, k))
    return dict(ii=ii, jj=jj, vv=vv, A=A, B=B, Y0=Y0,
                C=ref_sddmm(A, B, ii, jj, vv), Y=ref_spmm(B, ii, jj, vv, Y0))


def main():
    assert oracle.have_ref(), "build oracle/_ref first: make -C oracle ref"
    rng = np.random.default_rng(20240501)
    out = {}
    cases = {
        "small": case(rng, 37, 29, 5, 200),
        "k64": case(rng, 50, 61, 64, 400),
        "hub": case(rng, 8, 300, 7, 600, hub_row=3, hub_len=400),
        "k1": case(rng, 13, 11, 1, 60),
    }
    for name, c in cases.items():
        for key, arr in c.items():
            out[f"{name}.{key}"] = arr
    # the reference's checker fill (miniapp/numCheckSeq.cpp:125-128) on a 6x5, 9-entry pattern
    ii = np.array([0, 1, 1, 2, 3, 4, 5, 5, 2], dtype=np.uint32)
    jj = np.array([1, 0, 4, 2, 3, 1, 0, 4, 2], dtype=np.uint32)
    vv = np.arange(1, 10, dtype=np.float64)
    k = 4
    A = np.repeat((np.arange(6) / 1000.0)[:, None], k, axis=1).copy()
    B = np.repeat((np.arange(5) / 1000.0)[:, None], k, axis=1).copy()
    out.update({"numcheck.ii": ii, "numcheck.jj": jj, "numcheck.vv": vv, "numcheck.A": A,
                "numcheck.B": B, "numcheck.C": ref_sddmm(A, B, ii, jj, vv)})
    # localizeIndices (src/SparseMatrix.hpp:69-99) on global ids
    gi = rng.integers(0, 1000, 80).astype(np.uint32)
    gj = rng.integers(0, 5000, 80).astype(np.uint32)
    li, lj = gi.copy(), gj.copy()
    nr, nc = oracle._u32(), oracle._u32()
    import ctypes
    ltgR = np.zeros(80, dtype=np.uint32)
    ltgC = np.zeros(80, dtype=np.uint32)
    rc = oracle.load_ref().ref_localize_indices(80, p(li), p(lj), ctypes.byref(nr),
                                                ctypes.byref(nc), p(ltgR), p(ltgC))
    assert rc == 0
    out.update({"localize.gi": gi, "localize.gj": gj, "localize.li": li, "localize.lj": lj,
                "localize.ltgR": ltgR[:nr.value].copy(), "localize.ltgC": ltgC[:nc.value].copy()})
    np.savez_compressed(OUT, **out)
    print("wrote", OUT, os.path.getsize(OUT), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
