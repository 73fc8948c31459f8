// C entry points around the reference's own SpKernels::sddmm / SpKernels::spmm.
// TEST INFRASTRUCTURE ONLY: built in the build container from the reference's
// sources where they lie (see oracle/Makefile, target `ref`), output into
// oracle/_ref/.  Used to check the oracle's restatement bit for bit and to
// write the golden vectors under tests/golden/.  fp64 only: the reference's
// real_t is a fixed macro (src/basic.hpp:17).
//
// This file contains no reference code; it includes the reference headers by
// path (-I<reference>/src) and links the reference's core_ops.cpp.
#include <chrono>
#include <cstdint>
#include <cstring>
#include <exception>

#include "SparseMatrix.hpp"
#include "basic.hpp"
#include "core_ops.hpp"

using namespace SpKernels;

namespace {
void fill_panel(denseMatrix &M, uint32_t rows, uint32_t k, const double *src)
{
    M.m = rows;
    M.n = k;
    M.data.assign(src, src + (size_t)rows * k);
}
void fill_coo(cooMat &S, uint32_t nrows, uint32_t ncols, uint64_t nnz,
              const uint32_t *ii, const uint32_t *jj, const double *vv)
{
    S.nrows = S.gnrows = nrows;
    S.ncols = S.gncols = ncols;
    S.nnz = S.gnnz = nnz;
    S.ii.assign(ii, ii + nnz);
    S.jj.assign(jj, jj + nnz);
    S.vv.assign(vv, vv + nnz);
}
} // namespace

extern "C" {

// returns 0, or -1 if the reference threw (std::out_of_range from .at()).
__attribute__((visibility("default"))) int
ref_sddmm_f64(uint32_t m, uint32_t n, uint32_t k, const double *A,
              const double *B, uint64_t nnz, const uint32_t *ii,
              const uint32_t *jj, const double *svv, double *cvv)
{
    try {
        denseMatrix a, b;
        cooMat S, C;
        fill_panel(a, m, k, A);
        fill_panel(b, n, k, B);
        fill_coo(S, m, n, nnz, ii, jj, svv);
        C = S;
        std::memcpy(C.vv.data(), cvv, nnz * sizeof(double));
        sddmm(a, b, S, C);
        std::memcpy(cvv, C.vv.data(), nnz * sizeof(double));
        return 0;
    } catch (const std::exception &) {
        return -1;
    }
}

__attribute__((visibility("default"))) int
ref_spmm_f64(uint32_t ncols, uint32_t nrows, uint32_t k, const double *X,
             uint64_t nnz, const uint32_t *ii, const uint32_t *jj,
             const double *avv, double *Y)
{
    try {
        denseMatrix x, y;
        cooMat A;
        fill_panel(x, ncols, k, X);
        fill_panel(y, nrows, k, Y);
        fill_coo(A, nrows, ncols, nnz, ii, jj, avv);
        spmm(x, A, y);
        std::memcpy(Y, y.data.data(), (size_t)nrows * k * sizeof(double));
        return 0;
    } catch (const std::exception &) {
        return -1;
    }
}

// One SDDMM then one SpMM of the reference over the same operands, timed as the
// reference times its kernel (a chrono pair around the call,
// src/distributed_comp.cpp:176-179); building the reference's objects from the
// caller's arrays is outside the timed regions.  The results are discarded but
// for one checksum each, so that the calls cannot be optimised away.
__attribute__((visibility("default"))) int
ref_time_f64(uint32_t m, uint32_t n, uint32_t k, const double *A, const double *B,
             const double *Y0, uint64_t nnz, const uint32_t *ii, const uint32_t *jj,
             const double *vv, double *sddmm_seconds, double *spmm_seconds, double *checksum)
{
    try {
        denseMatrix a, b, y;
        cooMat S, C;
        fill_panel(a, m, k, A);
        fill_panel(b, n, k, B);
        fill_panel(y, m, k, Y0);
        fill_coo(S, m, n, nnz, ii, jj, vv);
        C = S;
        using clock = std::chrono::steady_clock;
        const auto t0 = clock::now();
        sddmm(a, b, S, C);
        const auto t1 = clock::now();
        spmm(b, S, y);
        const auto t2 = clock::now();
        *sddmm_seconds = std::chrono::duration<double>(t1 - t0).count();
        *spmm_seconds = std::chrono::duration<double>(t2 - t1).count();
        double sum = 0;
        for (uint64_t e = 0; e < nnz; ++e)
            sum += C.vv[e];
        for (double v : y.data)
            sum += v;
        *checksum = sum;
        return 0;
    } catch (const std::exception &) {
        return -1;
    }
}

// COOMatrix::localizeIndices (src/SparseMatrix.hpp:69-99) on a caller's
// arrays; nrows_out/ncols_out receive the touched row/col counts and
// ltgR/ltgC (capacity nnz each) the local->global maps.
__attribute__((visibility("default"))) int
ref_localize_indices(uint64_t nnz, uint32_t *ii, uint32_t *jj,
                     uint32_t *nrows_out, uint32_t *ncols_out, uint32_t *ltgR,
                     uint32_t *ltgC)
{
    try {
        cooMat S;
        S.nnz = nnz;
        S.ii.assign(ii, ii + nnz);
        S.jj.assign(jj, jj + nnz);
        S.vv.assign(nnz, 1.0);
        S.localizeIndices();
        std::memcpy(ii, S.ii.data(), nnz * sizeof(uint32_t));
        std::memcpy(jj, S.jj.data(), nnz * sizeof(uint32_t));
        *nrows_out = S.nrows;
        *ncols_out = S.ncols;
        std::memcpy(ltgR, S.ltgR.data(), S.ltgR.size() * sizeof(uint32_t));
        std::memcpy(ltgC, S.ltgC.data(), S.ltgC.size() * sizeof(uint32_t));
        return 0;
    } catch (const std::exception &) {
        return -1;
    }
}
}
