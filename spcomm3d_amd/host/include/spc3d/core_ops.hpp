// The local compute step with the reference's two signatures
// (src/core_ops.hpp:9-12), running on the GPU through the C ABI of
// include/spcomm3d_hip.h.  Link spcomm3d_amd/host/src/core_ops_hip.cpp in place
// of the reference's src/core_ops.cpp.
//
// Drop-in mode (these two functions): operands live in the caller's
// std::vectors, as in the reference; each call uploads the dense panels, runs
// the kernel and downloads the result, so C.vv / Y.data are valid on return
// (the reference's comm plans keep raw pointers into them, src/comm.hpp:41,49).
// The benches call the kernels five times on one pattern and the same panels
// (miniapp/bench_both.cpp:202-203, bench_spmm.cpp:185-186): the library keeps the
// plan and the device panels between calls and reuses what still holds the
// operands' content (spc3d_sddmm_host / spc3d_spmm_host); calls may come from
// several threads, they run one at a time.
//
// Failures: the reference fails by std::out_of_range from .at()
// (core_ops.cpp:16,18,32).  Here a bad index or a too-short C.vv throws
// std::out_of_range; any other failure (no GPU, HIP error, shape mismatch)
// throws std::runtime_error.  Nothing falls back to a CPU loop.
#pragma once

#include "SparseMatrix.hpp"
#include "basic.hpp"

namespace SpKernels {

// C.vv[i] = S.vv[i] * sum_j A[S.ii[i], j] * B[S.jj[i], j] for i < S.nnz; k = A.n.
// Only C.vv is written; it must hold at least S.nnz values.
void sddmm(denseMatrix &A, denseMatrix &B, cooMat &S, cooMat &C);

// Y[A.ii[i], :] += A.vv[i] * X[A.jj[i], :] for i < A.nnz; k = X.n.
void spmm(denseMatrix &X, cooMat &A, denseMatrix &Y);

namespace hip {

// Device the shim runs on (default 0); call before the first kernel.
void set_device(int device);

// Drop everything kept between calls (plans, device panels).  Never needed for
// correctness, the keys cover every byte of the operands; it frees device memory.
void invalidate(const cooMat *S = nullptr);

// Device time of the last sddmm / spmm kernel (without transfers), microseconds.
double last_kernel_us();

// Free all device memory the shim holds and destroy its context.
void shutdown();

} // namespace hip
} // namespace SpKernels
