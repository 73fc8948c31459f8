// The reference's six distributed wrappers (src/distributed_comp.cpp:17,141,194,237,285,
// 349) over operands that stay on the device.  Phase order and statistics lines as in
// distributed_comp.cpp; every phase is queued on the context's stream, device events mark
// the phase boundaries, and the call waits once, at its end, to read them.
#include "spc3d/distributed_comp_device.hpp"

#include "dist_internal.hpp"

using namespace SpKernels;
using spc3d_dist::require_single;
using spc3d_dist::stats_sparse;
using spc3d_dist::stats_sparse2;

namespace {

// Event slots of the context's timer used by these wrappers (below the two the one-shot
// host calls use).
constexpr int kSlot0 = 4070;
enum Mark { kStart = 0, kCpyA0, kCpyA1, kCpyB0, kCpyB1, kPreEnd, kCompEnd, kCpyC0, kCpyC1, kCpyD0,
            kCpyD1, kEnd };

struct Marks {
    spc3d::Context &ctx;
    bool set[kEnd + 1] = {false};
    void at(Mark m)
    {
        ctx.mark(kSlot0 + m);
        set[m] = true;
    }
    double us(Mark a, Mark b) { return set[a] && set[b] ? 1e3 * ctx.elapsed_ms(kSlot0 + a, kSlot0 + b) : 0.0; }
};

// Reads the events (this waits for the call's last kernel) and files the times: whole
// milliseconds where the reference has them, microseconds beside.
void finish(Marks &m)
{
    distTiming &g = spc3d_dist::last_timing();
    g = distTiming();
    const double total = m.us(kStart, kEnd);
    const double comm1 = m.us(kStart, kPreEnd), comp = m.us(kPreEnd, kCompEnd);
    const double comm2 = m.us(kCompEnd, kEnd);
    const double cpy = m.us(kCpyA0, kCpyA1) + m.us(kCpyB0, kCpyB1) + m.us(kCpyC0, kCpyC1) +
                       m.us(kCpyD0, kCpyD1);
    g.totalTimeUs = (idx_large_t)total;
    g.comm1TimeUs = (idx_large_t)comm1;
    g.compTimeUs = (idx_large_t)comp;
    g.comm2TimeUs = (idx_large_t)comm2;
    g.commcpyTimeUs = (idx_large_t)cpy;
    g.pt.totalTime = (idx_t)(total / 1e3);
    g.pt.comm1Time = (idx_t)(comm1 / 1e3);
    g.pt.compTime = (idx_t)(comp / 1e3);
    g.pt.comm2Time = (idx_t)(comm2 / 1e3);
    g.pt.commcpyTime = (idx_t)(cpy / 1e3);
}

spc3d_dist::DenseShape shape_of(const DeviceDenseComm &d)
{
    spc3d_dist::DenseShape s;
    s.reduce_scatter = d.OP == 1 && d.commXflag && d.commYflag;
    s.x = d.commXflag;
    s.y = d.commYflag;
    s.cnt0 = s.last_end = s.x0 = s.all_x = d.count;
    s.outDegreeX = d.count ? 1 : 0;
    return s;
}

void stats_dense(const std::string &mtx, const char *alg, const DeviceDenseComm &d, idx_t f,
                 const parallelTiming &pt, const Mesh &mesh)
{
    spc3d_dist::stats_dense(mtx, alg, shape_of(d), f, pt, mesh);
}

// The expand before a kernel as dist_spmm_spcomm and dist_sddmm_spcomm run it
// (src/distributed_comp.cpp:28-51,152-175).
// A copy is bracketed by events only when it launches something: an event costs a few
// microseconds of host time, which a call over empty exchanges need not pay.
template <typename F> void timed_copy(Marks &m, bool runs, Mark a, Mark b, F copy)
{
    if (runs)
        m.at(a);
    copy();
    if (runs)
        m.at(b);
}

void expand(Marks &m, DeviceSparseComm &pre)
{
    pre.issue_Irecvs();
    timed_copy(m, pre.packs(), kCpyA0, kCpyA1, [&] { pre.copy_to_sendbuff(); });
    pre.issue_Sends();
    pre.issue_Waitall();
    timed_copy(m, pre.unpacks(), kCpyB0, kCpyB1, [&] { pre.copy_from_recvbuff(); });
}

void sddmm_two_sided(spc3d::Context &ctx, spc3d::Panel<real_t> &A, spc3d::Panel<real_t> &B,
                     spc3d::Plan<real_t> &S, DeviceSparseComm &preA, DeviceSparseComm &preB,
                     DeviceDenseComm &comm_post, spc3d::Vals<real_t> &C, const Mesh &mesh,
                     const std::string &mtx, const char *pre_name, const char *post_name,
                     bool with_dt)
{
    require_single(mesh);
    Marks m{ctx};
    m.at(kStart);
    preA.issue_Irecvs();
    preB.issue_Irecvs();
    preA.issue_Sends(with_dt);
    preB.issue_Sends(with_dt);
    preA.issue_Waitall();
    preB.issue_Waitall();
    m.at(kPreEnd);
    spc3d::sddmm(ctx, S, A, B, C);
    m.at(kCompEnd);
    comm_post.perform_dense_comm();
    m.at(kEnd);
    finish(m);
    const parallelTiming &pt = spc3d_dist::last_timing().pt;
    stats_sparse2(mtx, pre_name, preA, preB, A.cols(), pt, mesh);
    stats_dense(mtx, post_name, comm_post, A.cols(), pt, mesh);
}

} // namespace

// src/distributed_comp.cpp:17-76.  The reference's post phase calls
// comm_pre.copy_from_recvbuff() where comm_post.copy_to_sendbuff() is evidently meant
// (:59); the call is kept as it is there.
void dist_spmm_spcomm(spc3d::Context &ctx, spc3d::Panel<real_t> &X, spc3d::Plan<real_t> &A,
                      spc3d::Panel<real_t> &Y, DeviceSparseComm &comm_pre,
                      DeviceSparseComm &comm_post, const Mesh &mesh, const std::string &mtx)
{
    require_single(mesh);
    Marks m{ctx};
    m.at(kStart);
    expand(m, comm_pre);
    m.at(kPreEnd);
    spc3d::spmm(ctx, A, X, Y);
    m.at(kCompEnd);
    comm_post.issue_Irecvs();
    timed_copy(m, comm_pre.unpacks(), kCpyC0, kCpyC1,
               [&] { comm_pre.copy_from_recvbuff(); }); // sic, as the reference (:59)
    comm_post.issue_Sends();
    comm_post.issue_Waitall();
    timed_copy(m, comm_post.unpacks(), kCpyD0, kCpyD1, [&] { comm_post.SUM_from_recvbuff(); });
    m.at(kEnd);
    finish(m);
    const parallelTiming &pt = spc3d_dist::last_timing().pt;
    stats_sparse(mtx, "sparse spmm PRE", comm_pre, X.cols(), pt, mesh);
    stats_sparse(mtx, "sparse spmm POST", comm_post, X.cols(), pt, mesh);
}

// src/distributed_comp.cpp:285-348
void dist_spmm_dcomm(spc3d::Context &ctx, spc3d::Panel<real_t> &X, spc3d::Panel<real_t> &Y,
                     spc3d::Plan<real_t> &A, DeviceDenseComm &comm_pre,
                     DeviceDenseComm &comm_post, const Mesh &mesh, const std::string &mtx)
{
    require_single(mesh);
    Marks m{ctx};
    m.at(kStart);
    comm_pre.perform_dense_comm();
    m.at(kPreEnd);
    spc3d::spmm(ctx, A, X, Y);
    m.at(kCompEnd);
    comm_post.perform_dense_comm();
    m.at(kEnd);
    finish(m);
    const parallelTiming &pt = spc3d_dist::last_timing().pt;
    stats_dense(mtx, "dense spmm PRE", comm_pre, X.cols(), pt, mesh);
    stats_dense(mtx, "dense spmm POST", comm_post, X.cols(), pt, mesh);
}

// src/distributed_comp.cpp:141-193
void dist_sddmm_spcomm(spc3d::Context &ctx, spc3d::Panel<real_t> &A, spc3d::Panel<real_t> &B,
                       spc3d::Plan<real_t> &S, DeviceSparseComm &comm_pre,
                       DeviceDenseComm &comm_post, spc3d::Vals<real_t> &C, const Mesh &mesh,
                       const std::string &mtx)
{
    require_single(mesh);
    Marks m{ctx};
    m.at(kStart);
    expand(m, comm_pre);
    m.at(kPreEnd);
    spc3d::sddmm(ctx, S, A, B, C);
    m.at(kCompEnd);
    comm_post.perform_dense_comm();
    m.at(kEnd);
    finish(m);
    const parallelTiming &pt = spc3d_dist::last_timing().pt;
    stats_sparse(mtx, "sparse sddmm PRE", comm_pre, A.cols(), pt, mesh);
    stats_dense(mtx, "sparse sddmm POST", comm_post, A.cols(), pt, mesh);
}

// src/distributed_comp.cpp:237-284
void dist_sddmm_spcomm2(spc3d::Context &ctx, spc3d::Panel<real_t> &A, spc3d::Panel<real_t> &B,
                        spc3d::Plan<real_t> &S, DeviceSparseComm &comm_preA,
                        DeviceSparseComm &comm_preB, DeviceDenseComm &comm_post,
                        spc3d::Vals<real_t> &C, const Mesh &mesh, const std::string &mtx)
{
    sddmm_two_sided(ctx, A, B, S, comm_preA, comm_preB, comm_post, C, mesh, mtx,
                    "sparseNRB sddmm PRE", "sparseNRB sddmm POST", false);
}

// src/distributed_comp.cpp:194-236
void dist_sddmm_spcomm3(spc3d::Context &ctx, spc3d::Panel<real_t> &A, spc3d::Panel<real_t> &B,
                        spc3d::Plan<real_t> &S, DeviceSparseComm &comm_preA,
                        DeviceSparseComm &comm_preB, DeviceDenseComm &comm_post,
                        spc3d::Vals<real_t> &C, const Mesh &mesh, const std::string &mtx)
{
    sddmm_two_sided(ctx, A, B, S, comm_preA, comm_preB, comm_post, C, mesh, mtx,
                    "sparseNB sddmm PRE", "sparseNB sddmm POST", true);
}

// src/distributed_comp.cpp:349-413
void dist_sddmm_dcomm(spc3d::Context &ctx, spc3d::Panel<real_t> &A, spc3d::Panel<real_t> &B,
                      spc3d::Plan<real_t> &S, DeviceDenseComm &comm_pre,
                      DeviceDenseComm &comm_post, spc3d::Vals<real_t> &C, const Mesh &mesh,
                      const std::string &mtx)
{
    require_single(mesh);
    Marks m{ctx};
    m.at(kStart);
    comm_pre.perform_dense_comm();
    m.at(kPreEnd);
    spc3d::sddmm(ctx, S, A, B, C);
    m.at(kCompEnd);
    comm_post.perform_dense_comm();
    m.at(kEnd);
    finish(m);
    const parallelTiming &pt = spc3d_dist::last_timing().pt;
    stats_dense(mtx, "dense sddmm PRE", comm_pre, A.cols(), pt, mesh);
    stats_dense(mtx, "dense sddmm POST", comm_post, A.cols(), pt, mesh);
}
