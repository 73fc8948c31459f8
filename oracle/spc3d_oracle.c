/*
 * CPU oracle for the local SDDMM / SpMM path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the algorithm of the reference's two local
 * kernels.  It exists so that the GPU path can be checked against an
 * independent serial implementation on the same inputs.  Nothing in the
 * product (the HIP library, the host shim, the generators) may link, load or
 * call it; only the test-suite, the smoke check and the benchmark's
 * cpu_baseline leg do.
 *
 * Reference semantics followed (paths relative to the reference tree):
 *   sddmm : src/core_ops.cpp:5-22   k = A.n (:6); per COO entry i, in input
 *           order: vp = 0; for j ascending: vp += A[r,j]*B[c,j] (:14-17);
 *           C.vv[i] = vp * S.vv[i] (overwrite, scale after the sum, :18).
 *   spmm  : src/core_ops.cpp:24-35  k = X.n (:25); per COO entry i, in input
 *           order: Y[r,j] += a * X[c,j] for j ascending (:31-33).  Y is
 *           read-modify-write; duplicates add.
 *   panel : src/basic.hpp:30-36     row-major, element (x,y) at data[x*n+y].
 *   types : src/basic.hpp:16-18     idx_t = uint32, real_t = double,
 *           idx_large_t = uint64.  The reference is fp64-only; the *_f32
 *           functions are this build's extension with identical loop order.
 *
 * What pins each function (see tests/test_oracle.py):
 *   oracle_sddmm_f64 : bit-exact against the reference's own compiled
 *                      core_ops.cpp (oracle/_ref) and the committed golden
 *                      vectors made from it; closed form of the reference's
 *                      checker (numCheckSeq.cpp:125-131); K=1, one-hot rows,
 *                      dense brute force, transpose symmetry.
 *   oracle_spmm_f64  : bit-exact against oracle/_ref and golden vectors;
 *                      X=1 row sums, S=I, += semantics, duplicates add,
 *                      scipy csr @ X, adjoint identity with sddmm.
 *   *_f32            : the same closed forms (exact in fp32 for the chosen
 *                      inputs) and agreement with the f64 functions within
 *                      fp32 rounding; no reference build exists for fp32.
 *
 * Bounds: the reference checks every access with .at() and terminates on a
 * bad index (core_ops.cpp:16,18,32).  The oracle returns -1 instead of
 * touching memory out of range.
 *
 * Build:  make -C oracle        (gcc -O3 -ffp-contract=off, no FMA fusion, so
 * the fp64 results equal the reference's serial mul-then-add bit for bit).
 */
#include <stddef.h>
#include <stdint.h>

#define ORACLE_API __attribute__((visibility("default")))

#define DEFINE_SDDMM(NAME, REAL)                                               \
    ORACLE_API int NAME(uint32_t m, uint32_t n, uint32_t k, const REAL *A,     \
                        const REAL *B, uint64_t nnz, const uint32_t *ii,       \
                        const uint32_t *jj, const REAL *svv, REAL *cvv)        \
    {                                                                          \
        for (uint64_t e = 0; e < nnz; ++e) {                                   \
            uint32_t r = ii[e], c = jj[e];                                     \
            if (r >= m || c >= n)                                              \
                return -1;                                                     \
            const REAL *ar = A + (size_t)r * k;                                \
            const REAL *bc = B + (size_t)c * k;                                \
            REAL dot = (REAL)0;                                                \
            for (uint32_t j = 0; j < k; ++j)                                   \
                dot += ar[j] * bc[j];                                          \
            cvv[e] = dot * svv[e];                                             \
        }                                                                      \
        return 0;                                                              \
    }

#define DEFINE_SPMM(NAME, REAL)                                                \
    ORACLE_API int NAME(uint32_t ncols, uint32_t nrows, uint32_t k,            \
                        const REAL *X, uint64_t nnz, const uint32_t *ii,       \
                        const uint32_t *jj, const REAL *avv, REAL *Y)          \
    {                                                                          \
        for (uint64_t e = 0; e < nnz; ++e) {                                   \
            uint32_t r = ii[e], c = jj[e];                                     \
            if (r >= nrows || c >= ncols)                                      \
                return -1;                                                     \
            const REAL a = avv[e];                                             \
            const REAL *xc = X + (size_t)c * k;                                \
            REAL *yr = Y + (size_t)r * k;                                      \
            for (uint32_t j = 0; j < k; ++j)                                   \
                yr[j] += a * xc[j];                                            \
        }                                                                      \
        return 0;                                                              \
    }

/* A is m x k, B is n x k, both row-major; ii in [0,m), jj in [0,n). */
DEFINE_SDDMM(oracle_sddmm_f64, double)
DEFINE_SDDMM(oracle_sddmm_f32, float)

/* X is ncols x k, Y is nrows x k; argument order follows spmm(X, A, Y). */
DEFINE_SPMM(oracle_spmm_f64, double)
DEFINE_SPMM(oracle_spmm_f32, float)

/*
 * Per-entry magnitude scale used by the parity tests to define "relative"
 * error where a dot product of U[-1,1] values cancels towards zero:
 *   sddmm: scale[e] = |S.vv[e]| * sum_j |A[r,j]*B[c,j]|
 *   spmm : scale[r,j] = |Y0[r,j]| + sum_e |a_e * X[c_e,j]|   (Y holds |Y0| on entry)
 * Always computed in double.
 */
ORACLE_API int oracle_sddmm_scale_f64(uint32_t m, uint32_t n, uint32_t k,
                                      const double *A, const double *B,
                                      uint64_t nnz, const uint32_t *ii,
                                      const uint32_t *jj, const double *svv,
                                      double *scale)
{
    for (uint64_t e = 0; e < nnz; ++e) {
        uint32_t r = ii[e], c = jj[e];
        if (r >= m || c >= n)
            return -1;
        const double *ar = A + (size_t)r * k;
        const double *bc = B + (size_t)c * k;
        double s = 0.0;
        for (uint32_t j = 0; j < k; ++j) {
            double p = ar[j] * bc[j];
            s += p < 0 ? -p : p;
        }
        double v = svv[e] < 0 ? -svv[e] : svv[e];
        scale[e] = s * v;
    }
    return 0;
}

ORACLE_API int oracle_spmm_scale_f64(uint32_t ncols, uint32_t nrows, uint32_t k,
                                     const double *X, uint64_t nnz,
                                     const uint32_t *ii, const uint32_t *jj,
                                     const double *avv, double *Yabs)
{
    for (uint64_t e = 0; e < nnz; ++e) {
        uint32_t r = ii[e], c = jj[e];
        if (r >= nrows || c >= ncols)
            return -1;
        const double a = avv[e] < 0 ? -avv[e] : avv[e];
        const double *xc = X + (size_t)c * k;
        double *yr = Yabs + (size_t)r * k;
        for (uint32_t j = 0; j < k; ++j) {
            double x = xc[j] < 0 ? -xc[j] : xc[j];
            yr[j] += a * x;
        }
    }
    return 0;
}

/*
 * The copies either side of the reference's sparse exchanges, restated from
 * SparseComm (src/comm.hpp): slot i of the buffer holds `unit` reals that
 * belong to dense row rows[i] of a row-major panel with `unit` columns
 * (sendptr[i] / recvptr[i] point at the start of that row, comm_setup.cpp:121,131).
 *   op 0  copy_to_sendbuff   (:90-103)   buf[i,:]  = panel[rows[i],:]
 *   op 1  copy_from_recvbuff (:166-177)  panel[rows[i],:]  = buf[i,:]
 *   op 2  SUM_from_recvbuff  (:178-189)  panel[rows[i],:] += buf[i,:]
 * Slots are visited in ascending order, so for a repeated row the last slot
 * wins (op 1) and the slots add up in order (op 2).
 * Pinned in tests/test_rows.py by numpy fancy indexing / np.add.at, by
 * unpack(pack(P)) == P on distinct rows, and by the slot-order rule on repeats.
 */
#define DEFINE_ROWS(NAME, REAL)                                                \
    ORACLE_API int NAME(int op, uint32_t panel_rows, uint32_t unit,            \
                        REAL *panel, uint64_t n, const uint32_t *rows,         \
                        REAL *buf)                                             \
    {                                                                          \
        for (uint64_t i = 0; i < n; ++i) {                                     \
            if (rows[i] >= panel_rows)                                         \
                return -1;                                                     \
            REAL *p = panel + (size_t)rows[i] * unit;                          \
            REAL *b = buf + (size_t)i * unit;                                  \
            for (uint32_t j = 0; j < unit; ++j) {                              \
                if (op == 0)                                                   \
                    b[j] = p[j];                                               \
                else if (op == 1)                                              \
                    p[j] = b[j];                                               \
                else                                                           \
                    p[j] += b[j];                                              \
            }                                                                  \
        }                                                                      \
        return 0;                                                              \
    }

DEFINE_ROWS(oracle_rows_f64, double)
DEFINE_ROWS(oracle_rows_f32, float)
