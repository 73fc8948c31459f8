// Single-rank forms of the reference's six distributed wrappers
// (src/distributed_comp.cpp:17,141,194,237,285,349).  Phase order, what is
// timed, and the statistics lines follow the reference; the exchanges are the
// single-rank stand-ins of spc3d/distributed_comp.hpp.
#include "spc3d/distributed_comp.hpp"

#include <chrono>
#include <numeric>

#include "spc3d/core_ops.hpp"

using namespace SpKernels;
using DComm::DenseComm;

namespace {

std::FILE *g_stats = stdout;
thread_local distTiming g_last;

using clk = std::chrono::high_resolution_clock;

idx_t ms_since(clk::time_point t0)
{
    return (idx_t)std::chrono::duration_cast<std::chrono::milliseconds>(clk::now() - t0).count();
}

void require_single(const Mesh &mesh)
{
    if (mesh.X != 1 || mesh.Y != 1 || mesh.Z != 1)
        throw std::runtime_error("dist_*: this library runs one rank on one GPU; the mesh must be "
                                 "1 x 1 x 1");
}

// "mtx alg P Kloc Z avgSendMsg avgSendVol avgRecvMsg avgRecvVol maxSendMsg
//  maxSendVol maxRecvMsg maxRecvVol comm1 comm2 commcpy comp total"
// (src/comm_stats.cpp:33-36,53,71-73) with P = 1: averages equal maxima.
void print_line(const std::string &mtx, const char *alg, idx_t f, const Mesh &mesh,
                idx_large_t sendMsg, idx_large_t sendVol, idx_large_t recvMsg,
                idx_large_t recvVol, const parallelTiming &pt)
{
    if (!g_stats)
        return;
    std::fprintf(g_stats, "%s %s %d %u %d %.2f %.2f %.2f %.2f %lu %lu %lu %lu %u %u %u %u %u\n",
                 mtx.c_str(), alg, 1, f, mesh.Z, (float)sendMsg, (float)sendVol, (float)recvMsg,
                 (float)recvVol, (unsigned long)sendMsg, (unsigned long)sendVol,
                 (unsigned long)recvMsg, (unsigned long)recvVol, pt.comm1Time, pt.comm2Time,
                 pt.commcpyTime, pt.compTime, pt.totalTime);
}

// src/comm_stats.cpp:59-73
void stats_sparse(const std::string &mtx, const char *alg, const SparseComm<real_t> &c, idx_t f,
                  const parallelTiming &pt, const Mesh &mesh)
{
    const idx_large_t sv = (idx_large_t)std::accumulate(c.sendCount.begin(), c.sendCount.end(), 0.0);
    const idx_large_t rv = (idx_large_t)std::accumulate(c.recvCount.begin(), c.recvCount.end(), 0.0);
    print_line(mtx, alg, f, mesh, (idx_large_t)c.outDegree, sv, (idx_large_t)c.inDegree, rv, pt);
}

// src/comm_stats.cpp:74-92
void stats_sparse2(const std::string &mtx, const char *alg, const SparseComm<real_t> &a,
                   const SparseComm<real_t> &b, idx_t f, const parallelTiming &pt,
                   const Mesh &mesh)
{
    const idx_large_t sv =
        (idx_large_t)(std::accumulate(a.sendCount.begin(), a.sendCount.end(), 0.0) +
                      std::accumulate(b.sendCount.begin(), b.sendCount.end(), 0.0));
    const idx_large_t rv =
        (idx_large_t)(std::accumulate(a.recvCount.begin(), a.recvCount.end(), 0.0) +
                      std::accumulate(b.recvCount.begin(), b.recvCount.end(), 0.0));
    print_line(mtx, alg, f, mesh, (idx_large_t)(a.outDegree + b.outDegree), sv,
               (idx_large_t)(a.inDegree + b.inDegree), rv, pt);
}

// src/comm_stats.cpp:93-129, with this rank being rank 0 of every sub-communicator
void stats_dense(const std::string &mtx, const char *alg, const DenseComm &d, idx_t f,
                 const parallelTiming &pt, const Mesh &mesh)
{
    idx_large_t sendVol = 0, recvVol = 0, sendMsg = 1, recvMsg = 0;
    if (d.OP == 1 && d.commXflag && d.commYflag) {
        if (!d.bcastXcnt.empty()) {
            sendVol = (d.bcastXdisp.empty() ? 0 : d.bcastXdisp.back()) + d.bcastXcnt.back();
            recvVol = d.bcastXcnt[0];
        }
        recvMsg = 1;
    } else {
        idx_large_t all = 0;
        if (d.commXflag)
            all += (idx_large_t)std::accumulate(d.bcastXcnt.begin(), d.bcastXcnt.end(), 0.0);
        if (d.commYflag)
            all += (idx_large_t)std::accumulate(d.bcastYcnt.begin(), d.bcastYcnt.end(), 0.0);
        sendVol = (d.commXflag && !d.bcastXcnt.empty() ? d.bcastXcnt[0] : 0) +
                  (d.commYflag && !d.bcastYcnt.empty() ? d.bcastYcnt[0] : 0);
        recvVol = all - sendVol;
        recvMsg = (d.commXflag ? d.outDegreeX : 0) + (d.commYflag ? d.outDegreeY : 0);
    }
    print_line(mtx, alg, f, mesh, sendMsg, sendVol, recvMsg, recvVol, pt);
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
