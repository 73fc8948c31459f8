"""Byte and flop models for the local SDDMM / SpMM kernels.

Strict (compulsory) model: every operand is moved between HBM and the chip
exactly once.  With w = sizeof(real), m_t / n_t = rows / columns that have at
least one entry, and the index structure I = 4(m+1) + 4 nnz (CSR row pointers
and column indices; + 4 nnz when a permutation back to the caller's COO order
has to be read):

    B_sddmm = I + w nnz (S.vv) + w nnz (C.vv) + w K m_t (A) + w K n_t (B)
    B_spmm  = I + w nnz (A.vv) + w K n_t (X) + 2 w K m_t (Y read + write)

Gather (no-reuse) model: one dense row fetched per entry, i.e. w K n_t is
replaced by w K nnz.  Flops are 2 nnz K for either kernel (the SDDMM scale is
not counted).
"""
from __future__ import annotations

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, GB/s


def index_bytes(nrows: int, nnz: int, with_perm: bool) -> int:
    return 4 * (nrows + 1) + 4 * nnz + (4 * nnz if with_perm else 0)


def flops(nnz: int, k: int) -> int:
    return 2 * nnz * k


def sddmm_bytes(nrows, nnz, k, w, m_t, n_t, with_perm=False, gather=False) -> int:
    b_side = nnz if gather else n_t
    return index_bytes(nrows, nnz, with_perm) + 2 * w * nnz + w * k * m_t + w * k * b_side


def spmm_bytes(nrows, nnz, k, w, m_t, n_t, gather=False) -> int:
    x_side = nnz if gather else n_t
    return index_bytes(nrows, nnz, False) + w * nnz + w * k * x_side + 2 * w * k * m_t


def fused_bytes(nrows, nnz, k, w, m_t, n_t, with_perm=False, gather=False) -> int:
    """SDDMM and the SpMM of the same pattern over the same B in one pass: every
    operand of either kernel once (A, B, the Y read-modify-write, S.vv, C.vv)."""
    b_side = nnz if gather else n_t
    return (index_bytes(nrows, nnz, with_perm) + 2 * w * nnz + w * k * m_t + w * k * b_side +
            2 * w * k * m_t)
