// The binding a maintainer of the reference would add as src/core_ops_hip.cpp in
// place of src/core_ops.cpp: the reference's two kernels over the C ABI, in the
// drop-in form (operands stay in the caller's std::vectors).  TEST
// INFRASTRUCTURE here: oracle/Makefile (target `ref`) compiles it against the
// reference's own headers and links it with the reference's own driver
// miniapp/numCheckSeq.cpp into oracle/_ref/numCheckSeq_hip, which
// tests/test_reference_driver.py runs beside the all-reference build of the same
// driver.  It contains no reference code.
#include "SparseMatrix.hpp"
#include "basic.hpp"
#include "spcomm3d_hip.h"
#include <stdexcept>

namespace {
spc3d_ctx* ctx() {
    static spc3d_ctx* c = nullptr;
    if (!c && spc3d_ctx_create(0, &c) != SPC3D_OK) throw std::runtime_error(spc3d_last_error());
    return c;
}
void check(int rc) {
    if (rc == SPC3D_ERR_BAD_INDEX) throw std::out_of_range(spc3d_last_error()); // what .at() throws
    if (rc != SPC3D_OK) throw std::runtime_error(spc3d_last_error());
}
}
namespace SpKernels {
void sddmm(denseMatrix& A, denseMatrix& B, cooMat& S, cooMat& C) {
    if (C.vv.size() < S.nnz) throw std::out_of_range("C.vv");            // core_ops.cpp:18
    check(spc3d_sddmm_host(ctx(), SPC3D_F64, A.m, B.m, A.n, A.data.data(), B.data.data(),
                           S.nnz, S.ii.data(), S.jj.data(), S.vv.data(), C.vv.data()));
}
void spmm(denseMatrix& X, cooMat& A, denseMatrix& Y) {
    check(spc3d_spmm_host(ctx(), SPC3D_F64, X.m, Y.m, X.n, X.data.data(),
                          A.nnz, A.ii.data(), A.jj.data(), A.vv.data(), Y.data.data()));
}
}
