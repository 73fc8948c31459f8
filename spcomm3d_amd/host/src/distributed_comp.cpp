// Single-rank forms of the reference's six distributed wrappers
// (src/distributed_comp.cpp:17,141,194,237,285,349).  Phase order, what is
// timed, and the statistics lines follow the reference; the exchanges are the
// single-rank stand-ins of spc3d/distributed_comp.hpp.
#include "spc3d/distributed_comp.hpp"

#include <chrono>
#include <numeric>

#include "spc3d/core_ops.hpp"

#include "dist_internal.hpp"

using namespace SpKernels;
using DComm::DenseComm;

namespace {

std::FILE *g_stats = stdout;
thread_local distTiming g_last;

using clk = std::chrono::high_resolution_clock;
using spc3d_dist::print_line;
using spc3d_dist::require_single;
using spc3d_dist::stats_sparse;
using spc3d_dist::stats_sparse2;

idx_t ms_since(clk::time_point t0)
{
    return (idx_t)std::chrono::duration_cast<std::chrono::milliseconds>(clk::now() - t0).count();
}

spc3d_dist::DenseShape shape_of(const DenseComm &d)
{
    spc3d_dist::DenseShape s;
    s.reduce_scatter = d.OP == 1 && d.commXflag && d.commYflag;
    s.x = d.commXflag;
    s.y = d.commYflag;
    if (!d.bcastXcnt.empty()) {
        s.cnt0 = d.bcastXcnt[0];
        s.last_end = (d.bcastXdisp.empty() ? 0 : d.bcastXdisp.back()) + d.bcastXcnt.back();
        s.x0 = d.bcastXcnt[0];
    }
    if (!d.bcastYcnt.empty())
        s.y0 = d.bcastYcnt[0];
    s.all_x = (idx_large_t)std::accumulate(d.bcastXcnt.begin(), d.bcastXcnt.end(), 0.0);
    s.all_y = (idx_large_t)std::accumulate(d.bcastYcnt.begin(), d.bcastYcnt.end(), 0.0);
    s.outDegreeX = d.outDegreeX;
    s.outDegreeY = d.outDegreeY;
    return s;
}

void stats_dense(const std::string &mtx, const char *alg, const DenseComm &d, idx_t f,
                 const parallelTiming &pt, const Mesh &mesh)
{
    spc3d_dist::stats_dense(mtx, alg, shape_of(d), f, pt, mesh);
}

// Times fn with the wall clock (integer ms, as the reference) and takes the
// device time of the kernel inside it in microseconds.
template <typename F> void timed_kernel(parallelTiming &pt, F fn)
{
    const auto t0 = clk::now();
    fn();
    pt.compTime = ms_since(t0);
    g_last.compTimeUs = (idx_large_t)hip::last_kernel_us();
}

} // namespace

std::FILE *&spc3d_dist::stats_stream() { return g_stats; }
distTiming &spc3d_dist::last_timing() { return g_last; }

void dist_set_stats_stream(std::FILE *f) { g_stats = f; }

const distTiming &dist_last_timing() { return g_last; }

void setup_sddmm_reduce_single_rank(cooMat &C, DenseComm &comm_post)
{
    C.ownedNnz = (idx_t)C.nnz;
    C.ownedVals.assign(C.nnz, (real_t)0);
    comm_post.OP = 1;
    comm_post.commXflag = comm_post.commYflag = true;
    comm_post.bufferptrX = C.vv.data();
    comm_post.bufferptrY = C.ownedVals.data();
    comm_post.bcastXcnt.assign(1, (idx_t)C.nnz);
    comm_post.bcastXdisp.assign(1, 0);
    comm_post.outDegreeX = 1;
}

// src/distributed_comp.cpp:17-76.  The reference's post phase calls
// comm_pre.copy_from_recvbuff() where comm_post.copy_to_sendbuff() is evidently
// meant (:59); the call is kept as it is there.  With one rank both are empty.
void dist_spmm_spcomm(denseMatrix &X, cooMat &A, denseMatrix &Y,
                                SparseComm<real_t> &comm_pre, SparseComm<real_t> &comm_post,
                                const Mesh &mesh)
{
    require_single(mesh);
    parallelTiming pt;
    const auto tot = clk::now();
    auto t = clk::now();
    comm_pre.issue_Irecvs();
    auto t2 = clk::now();
    comm_pre.copy_to_sendbuff();
    pt.commcpyTime = ms_since(t2);
    comm_pre.issue_Sends();
    comm_pre.issue_Waitall();
    t2 = clk::now();
    comm_pre.copy_from_recvbuff();
    pt.commcpyTime += ms_since(t2);
    pt.comm1Time = ms_since(t);
    timed_kernel(pt, [&] { spmm(X, A, Y); });
    t = clk::now();
    comm_post.issue_Irecvs();
    t2 = clk::now();
    comm_pre.copy_from_recvbuff(); // sic, as the reference (:59)
    pt.commcpyTime += ms_since(t2);
    comm_post.issue_Sends();
    comm_post.issue_Waitall();
    t2 = clk::now();
    comm_post.SUM_from_recvbuff();
    pt.commcpyTime += ms_since(t2);
    pt.comm2Time = ms_since(t);
    pt.totalTime = ms_since(tot);
    stats_sparse(A.mtxName, "sparse spmm PRE", comm_pre, X.n, pt, mesh);
    stats_sparse(A.mtxName, "sparse spmm POST", comm_post, X.n, pt, mesh);
    g_last.pt = pt;
}

// src/distributed_comp.cpp:285-348
void dist_spmm_dcomm(denseMatrix &X, denseMatrix &Y, cooMat &A, DenseComm &comm_pre,
                               DenseComm &comm_post, const Mesh &mesh)
{
    require_single(mesh);
    parallelTiming pt;
    const auto tot = clk::now();
    auto t = clk::now();
    comm_pre.perform_dense_comm();
    pt.comm1Time = ms_since(t);
    timed_kernel(pt, [&] { spmm(X, A, Y); });
    t = clk::now();
    comm_post.perform_dense_comm();
    pt.comm2Time = ms_since(t);
    pt.totalTime = ms_since(tot);
    stats_dense(A.mtxName, "dense spmm PRE", comm_pre, X.n, pt, mesh);
    stats_dense(A.mtxName, "dense spmm POST", comm_post, X.n, pt, mesh);
    g_last.pt = pt;
}

// src/distributed_comp.cpp:141-193
void dist_sddmm_spcomm(denseMatrix &A, denseMatrix &B, cooMat &S,
                                 SparseComm<real_t> &comm_pre, DenseComm &comm_post, cooMat &C,
                                 const Mesh &mesh)
{
    require_single(mesh);
    parallelTiming pt;
    const auto tot = clk::now();
    auto t = clk::now();
    comm_pre.issue_Irecvs();
    auto t2 = clk::now();
    comm_pre.copy_to_sendbuff();
    pt.commcpyTime = ms_since(t2);
    comm_pre.issue_Sends();
    comm_pre.issue_Waitall();
    t2 = clk::now();
    comm_pre.copy_from_recvbuff();
    pt.commcpyTime += ms_since(t2);
    pt.comm1Time = ms_since(t);
    timed_kernel(pt, [&] { sddmm(A, B, S, C); });
    t = clk::now();
    comm_post.perform_dense_comm();
    pt.comm2Time = ms_since(t);
    pt.totalTime = ms_since(tot);
    stats_sparse(C.mtxName, "sparse sddmm PRE", comm_pre, A.n, pt, mesh);
    stats_dense(C.mtxName, "sparse sddmm POST", comm_post, A.n, pt, mesh);
    g_last.pt = pt;
}

namespace {
// Shared body of spcomm2 / spcomm3 (src/distributed_comp.cpp:194-284): the two
// differ in how the expand is sent (derived datatypes vs. no receive buffer),
// which has no single-rank counterpart.
void sddmm_two_sided(denseMatrix &A, denseMatrix &B, cooMat &S,
                               SparseComm<real_t> &preA, SparseComm<real_t> &preB,
                               DenseComm &comm_post, cooMat &C, const Mesh &mesh,
                               const char *pre_name, const char *post_name, bool with_dt)
{
    require_single(mesh);
    parallelTiming pt;
    const auto tot = clk::now();
    auto t = clk::now();
    preA.issue_Irecvs();
    preB.issue_Irecvs();
    preA.issue_Sends(with_dt);
    preB.issue_Sends(with_dt);
    preA.issue_Waitall();
    preB.issue_Waitall();
    pt.comm1Time = ms_since(t);
    timed_kernel(pt, [&] { sddmm(A, B, S, C); });
    t = clk::now();
    comm_post.perform_dense_comm();
    pt.comm2Time = ms_since(t);
    pt.totalTime = ms_since(tot);
    stats_sparse2(C.mtxName, pre_name, preA, preB, A.n, pt, mesh);
    stats_dense(C.mtxName, post_name, comm_post, A.n, pt, mesh);
    g_last.pt = pt;
}
} // namespace

// src/distributed_comp.cpp:237-284
void dist_sddmm_spcomm2(denseMatrix &A, denseMatrix &B, cooMat &S,
                                  SparseComm<real_t> &comm_preA, SparseComm<real_t> &comm_preB,
                                  DenseComm &comm_post, cooMat &C, const Mesh &mesh)
{
    sddmm_two_sided(A, B, S, comm_preA, comm_preB, comm_post, C, mesh,
                           "sparseNRB sddmm PRE", "sparseNRB sddmm POST", false);
}

// src/distributed_comp.cpp:194-236
void dist_sddmm_spcomm3(denseMatrix &A, denseMatrix &B, cooMat &S,
                                  SparseComm<real_t> &comm_preA, SparseComm<real_t> &comm_preB,
                                  DenseComm &comm_post, cooMat &C, const Mesh &mesh)
{
    sddmm_two_sided(A, B, S, comm_preA, comm_preB, comm_post, C, mesh,
                           "sparseNB sddmm PRE", "sparseNB sddmm POST", true);
}

// src/distributed_comp.cpp:349-413
void dist_sddmm_dcomm(denseMatrix &A, denseMatrix &B, cooMat &S, DenseComm &comm_pre,
                                DenseComm &comm_post, cooMat &C, const Mesh &mesh)
{
    require_single(mesh);
    parallelTiming pt;
    const auto tot = clk::now();
    auto t = clk::now();
    comm_pre.perform_dense_comm();
    pt.comm1Time = ms_since(t);
    timed_kernel(pt, [&] { sddmm(A, B, S, C); });
    t = clk::now();
    comm_post.perform_dense_comm();
    pt.comm2Time = ms_since(t);
    pt.totalTime = ms_since(tot);
    stats_dense(C.mtxName, "dense sddmm PRE", comm_pre, A.n, pt, mesh);
    stats_dense(C.mtxName, "dense sddmm POST", comm_post, A.n, pt, mesh);
    g_last.pt = pt;
}
