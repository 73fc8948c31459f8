// SpKernels::sddmm / SpKernels::spmm over host vectors, executed on the GPU.
// Replaces the reference's src/core_ops.cpp at link time (same two symbols,
// src/core_ops.hpp:9-12).  See spc3d/core_ops.hpp for the contract.
//
// The work is the C ABI's: spc3d_sddmm_host / spc3d_spmm_host keep the plan of a
// pattern, the device panels and the result vector between calls, keyed by what the
// operands hold.  This file checks what the reference's .at() would check, turns status
// codes into the reference's exceptions, and owns the one context.
#include "spc3d/core_ops.hpp"

#include <cstring>
#include <memory>
#include <mutex>
#include <stdexcept>
#include <string>
#include <vector>

#include "spc3d/device.hpp"

namespace SpKernels {
namespace {

struct Shim {
    std::mutex mutex; // the reference's kernels are reentrant; these share one context
    int device = 0;
    std::unique_ptr<spc3d::Context> ctx;
    double last_us = 0;

    spc3d::Context &context()
    {
        if (!ctx)
            ctx.reset(new spc3d::Context(device));
        return *ctx;
    }
    void note_kernel_time()
    {
        last_us = 1e3 * ctx->elapsed_ms(SPC3D_TIMER_HOST_CALL_BEGIN, SPC3D_TIMER_HOST_CALL_END);
    }
};

// Never destroyed: at process exit the HIP runtime may already be gone, and
// freeing device memory then is not safe.  hip::shutdown() releases everything.
Shim &shim()
{
    static Shim *s = new Shim;
    return *s;
}

void require_panel(const denseMatrix &M, const char *name)
{
    if (M.data.size() < static_cast<size_t>(M.m) * M.n)
        throw std::out_of_range(std::string("denseMatrix ") + name +
                                ": data holds fewer than m*n values");
}

void require_coo(const cooMat &S)
{
    if (S.ii.size() < S.nnz || S.jj.size() < S.nnz || S.vv.size() < S.nnz)
        throw std::out_of_range("cooMat: ii / jj / vv hold fewer than nnz entries");
}

} // namespace

void sddmm(denseMatrix &A, denseMatrix &B, cooMat &S, cooMat &C)
{
    if (S.nnz == 0)
        return;
    require_panel(A, "A");
    require_panel(B, "B");
    require_coo(S);
    if (C.vv.size() < S.nnz)
        throw std::out_of_range("sddmm: C.vv holds fewer than S.nnz values");
    if (B.n != A.n)
        throw std::runtime_error("sddmm: B.n != A.n is not supported");
    Shim &s = shim();
    std::lock_guard<std::mutex> lock(s.mutex);
    spc3d::check(spc3d_sddmm_host(s.context().get(), spc3d::dtype_of<real_t>(), A.m, B.m, A.n,
                                  A.data.data(), B.data.data(), S.nnz, S.ii.data(), S.jj.data(),
                                  S.vv.data(), C.vv.data()), // the first S.nnz values of C.vv
                 "spc3d_sddmm_host");
    s.note_kernel_time();
}

void spmm(denseMatrix &X, cooMat &A, denseMatrix &Y)
{
    if (A.nnz == 0)
        return;
    require_panel(X, "X");
    require_panel(Y, "Y");
    require_coo(A);
    if (Y.n != X.n)
        throw std::runtime_error("spmm: Y.n != X.n is not supported");
    Shim &s = shim();
    std::lock_guard<std::mutex> lock(s.mutex);
    spc3d::check(spc3d_spmm_host(s.context().get(), spc3d::dtype_of<real_t>(), X.m, Y.m, X.n,
                                 X.data.data(), A.nnz, A.ii.data(), A.jj.data(), A.vv.data(),
                                 Y.data.data()),
                 "spc3d_spmm_host");
    s.note_kernel_time();
}

namespace hip {

void set_device(int device)
{
    Shim &s = shim();
    std::lock_guard<std::mutex> lock(s.mutex);
    if (s.ctx && s.device != device)
        s.ctx.reset();
    s.device = device;
}

void invalidate(const cooMat *)
{
    // Plans are keyed by content, not by address: dropping everything kept is
    // always enough and costs one re-plan and one upload per operand.
    Shim &s = shim();
    std::lock_guard<std::mutex> lock(s.mutex);
    if (s.ctx)
        spc3d::check(spc3d_host_cache_clear(s.ctx->get()), "spc3d_host_cache_clear");
}

double last_kernel_us()
{
    Shim &s = shim();
    std::lock_guard<std::mutex> lock(s.mutex);
    return s.last_us;
}

void shutdown()
{
    Shim &s = shim();
    std::lock_guard<std::mutex> lock(s.mutex);
    s.ctx.reset(); // destroys the context and what its one-shot calls kept
}

} // namespace hip
} // namespace SpKernels
