// The reference's six distributed wrappers (src/distributed_comp.hpp:11-64) over
// operands that STAY on the device: dense panels (spc3d::Panel), the sparse operand
// as a plan (spc3d::Plan), value vectors and the send / receive buffers of the
// exchanges (spc3d::Vals).  Same phase order as the reference (and as the host-memory
// wrappers of distributed_comp.hpp): pre-communication, local kernel, post-
// communication, statistics line.  Nothing crosses the host-device boundary inside a
// call; every phase is queued on the context's stream and the call waits once, at its
// end, to read the phase times off device events.
//
// One rank on one GPU: the only messages an exchange can carry are those a rank
// addresses to itself, which is enough to run the copies either side of an exchange
// as kernels (spc3d_rows_pack / _unpack / _unpack_sum for SparseComm::copy_to_sendbuff /
// copy_from_recvbuff / SUM_from_recvbuff, src/comm.hpp:90-103,166-189) and is what the
// buffers of a real exchange (RCCL send / recv of sendBuff / into recvBuff) would hold.
#pragma once

#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "basic.hpp"
#include "device.hpp"
#include "distributed_comp.hpp"

namespace SpKernels {

// Device form of SparseComm<real_t> (src/comm.hpp:33-52).  sendptr / recvptr, which in
// the reference point at rows of a dense matrix, are row numbers of a device panel; the
// buffers are device vectors; counts and displacements are in reals as in the reference.
class DeviceSparseComm {
  public:
    int inDegree = 0, outDegree = 0;
    idx_t dataUnitSize = 1;
    std::vector<int> inSet, outSet;
    std::vector<int> sendCount, recvCount;
    std::vector<int> sendDisp, recvDisp;

    DeviceSparseComm(spc3d::Context &ctx, idx_t unitSize) : dataUnitSize(unitSize), ctx_(&ctx) {}

    // The rows this plan packs (row send_rows[i] of `from` is slot i of the send buffer) and
    // the rows it unpacks into (slot i of the receive buffer goes to row recv_rows[i] of
    // `into`); either list may be empty.  The panels must outlive the plan.
    void set_rows(spc3d::Panel<real_t> *from, const std::vector<idx_t> &send_rows,
                  spc3d::Panel<real_t> *into, const std::vector<idx_t> &recv_rows)
    {
        send_panel_ = from;
        recv_panel_ = into;
        send_map_.reset();
        recv_map_.reset();
        sendBuff.reset();
        recvBuff.reset();
        if (!send_rows.empty()) {
            if (!from || from->cols() != dataUnitSize)
                throw std::runtime_error("DeviceSparseComm: the panel's rows are not dataUnitSize wide");
            send_map_.reset(new spc3d::RowMap(*ctx_, from->rows(), send_rows.size(), send_rows.data()));
            sendBuff.reset(new spc3d::Vals<real_t>(*ctx_, (uint64_t)send_rows.size() * dataUnitSize));
        }
        if (!recv_rows.empty()) {
            if (!into || into->cols() != dataUnitSize)
                throw std::runtime_error("DeviceSparseComm: the panel's rows are not dataUnitSize wide");
            recv_map_.reset(new spc3d::RowMap(*ctx_, into->rows(), recv_rows.size(), recv_rows.data()));
            recvBuff.reset(new spc3d::Vals<real_t>(*ctx_, (uint64_t)recv_rows.size() * dataUnitSize));
        }
    }
    // The plan of a host-memory SparseComm whose sendptr point into `host_from` and whose
    // recvptr point into `host_into` (the dense matrices the device panels mirror).
    void adopt(const SparseComm<real_t> &h, const denseMatrix &host_from,
               spc3d::Panel<real_t> *from, const denseMatrix &host_into, spc3d::Panel<real_t> *into)
    {
        inDegree = h.inDegree, outDegree = h.outDegree;
        dataUnitSize = h.dataUnitSize;
        inSet = h.inSet, outSet = h.outSet;
        sendCount = h.sendCount, recvCount = h.recvCount;
        sendDisp = h.sendDisp, recvDisp = h.recvDisp;
        auto rows_of = [&](const std::vector<real_t *> &ptrs, const denseMatrix &M) {
            std::vector<idx_t> rows(ptrs.size());
            for (size_t i = 0; i < ptrs.size(); ++i) {
                const std::ptrdiff_t off = ptrs[i] - M.data.data();
                if (off < 0 || (size_t)off >= M.data.size() || off % M.n != 0)
                    throw std::runtime_error("DeviceSparseComm: a row pointer does not point at a "
                                             "row of the matrix it is said to belong to");
                rows[i] = (idx_t)(off / M.n);
            }
            return rows;
        };
        set_rows(from, rows_of(h.sendptr, host_from), into, rows_of(h.recvptr, host_into));
    }

    void issue_Irecvs() { require_self(); }
    void issue_Sends(bool with_DT = false)
    {
        require_self();
        if (with_DT && outDegree != 0)
            throw std::runtime_error("DeviceSparseComm: datatype sends have no single-rank form");
        for (int i = 0; i < outDegree; ++i) {
            if (sendCount.at(i) != recvCount.at(i) || !sendBuff || !recvBuff)
                throw std::runtime_error("DeviceSparseComm: a self-addressed message must be "
                                         "received with the length it is sent with");
            spc3d::check(spc3d_vals_copy(recvBuff->get(), (uint64_t)recvDisp.at(i), sendBuff->get(),
                                         (uint64_t)sendDisp.at(i), (uint64_t)sendCount[i]),
                         "spc3d_vals_copy");
        }
    }
    void issue_Waitall() { require_self(); }
    void copy_to_sendbuff() // src/comm.hpp:90-103
    {
        require_self();
        if (send_map_)
            spc3d::rows_pack(*ctx_, *send_panel_, *send_map_, *sendBuff);
    }
    void copy_from_recvbuff() // src/comm.hpp:166-177
    {
        require_self();
        if (recv_map_)
            spc3d::rows_unpack(*ctx_, *recv_panel_, *recv_map_, *recvBuff);
    }
    void SUM_from_recvbuff() // src/comm.hpp:178-189
    {
        require_self();
        if (recv_map_)
            spc3d::rows_unpack_sum(*ctx_, *recv_panel_, *recv_map_, *recvBuff);
    }
    void perform_sparse_comm(bool sendcopyflag = true, bool recvcopyflag = true)
    {
        issue_Irecvs();
        if (sendcopyflag)
            copy_to_sendbuff();
        issue_Sends();
        issue_Waitall();
        if (recvcopyflag)
            copy_from_recvbuff();
    }

    bool packs() const { return send_map_ != nullptr; }   // copy_to_sendbuff launches a kernel
    bool unpacks() const { return recv_map_ != nullptr; } // copy_from / SUM_from_recvbuff do

    std::unique_ptr<spc3d::Vals<real_t>> sendBuff, recvBuff; // device; null while empty

  private:
    void require_self() const
    {
        bool ok = inDegree == outDegree && (size_t)inDegree == inSet.size() &&
                  (size_t)outDegree == outSet.size();
        for (int r : inSet)
            ok = ok && r == 0;
        for (int r : outSet)
            ok = ok && r == 0;
        if (!ok)
            throw std::runtime_error("DeviceSparseComm: exchanges between ranks are outside this "
                                     "single-GPU library (only messages a rank addresses to "
                                     "itself can be carried out)");
    }
    spc3d::Context *ctx_;
    spc3d::Panel<real_t> *send_panel_ = nullptr, *recv_panel_ = nullptr;
    std::unique_ptr<spc3d::RowMap> send_map_, recv_map_;
};

// Device form of DComm::DenseComm (src/denseComm.hpp:12-48) on one rank: broadcasts from
// oneself and an in-place all-reduce change nothing; the reduce-scatter of SDDMM's Z
// reduction (OP 1, both flags) delivers the send buffer: to[0 .. count) = from[0 .. count).
struct DeviceDenseComm {
    int OP = 1;
    bool commXflag = false, commYflag = false;
    spc3d::Vals<real_t> *from = nullptr, *to = nullptr; // bufferptrX, bufferptrY
    idx_large_t count = 0;                              // bcastXcnt[0]
    void perform_dense_comm()
    {
        if (OP == 1 && commXflag && commYflag && from && to && from != to && count)
            spc3d::check(spc3d_vals_copy(to->get(), 0, from->get(), 0, count), "spc3d_vals_copy");
    }
};

// Single-rank form of setup_3dsddmm_reduce_scatter (src/comm_setup.cpp:671-689) on the
// device: the Z reduction sends C.vv and receives C.ownedVals, all nnz of them.
inline void setup_sddmm_reduce_single_rank(spc3d::Vals<real_t> &Cvv, spc3d::Vals<real_t> &ownedVals,
                                           DeviceDenseComm &comm_post)
{
    comm_post.OP = 1;
    comm_post.commXflag = comm_post.commYflag = true;
    comm_post.from = &Cvv;
    comm_post.to = &ownedVals;
    comm_post.count = Cvv.size();
}

} // namespace SpKernels

// The six wrappers over resident operands.  `mtx` is the name the statistics lines carry
// (cooMat::mtxName in the reference).  Phase times of the last call: dist_last_timing(),
// whose microsecond fields come from device events (the millisecond fields of its
// parallelTiming are those rounded down, for the reference's output format).
void dist_spmm_spcomm(spc3d::Context &ctx, spc3d::Panel<SpKernels::real_t> &X,
                      spc3d::Plan<SpKernels::real_t> &A, spc3d::Panel<SpKernels::real_t> &Y,
                      SpKernels::DeviceSparseComm &comm_pre, SpKernels::DeviceSparseComm &comm_post,
                      const SpKernels::Mesh &mesh, const std::string &mtx = "");
void dist_spmm_dcomm(spc3d::Context &ctx, spc3d::Panel<SpKernels::real_t> &X,
                     spc3d::Panel<SpKernels::real_t> &Y, spc3d::Plan<SpKernels::real_t> &A,
                     SpKernels::DeviceDenseComm &comm_pre, SpKernels::DeviceDenseComm &comm_post,
                     const SpKernels::Mesh &mesh, const std::string &mtx = "");
void dist_sddmm_spcomm(spc3d::Context &ctx, spc3d::Panel<SpKernels::real_t> &A,
                       spc3d::Panel<SpKernels::real_t> &B, spc3d::Plan<SpKernels::real_t> &S,
                       SpKernels::DeviceSparseComm &comm_pre, SpKernels::DeviceDenseComm &comm_post,
                       spc3d::Vals<SpKernels::real_t> &C, const SpKernels::Mesh &mesh,
                       const std::string &mtx = "");
void dist_sddmm_spcomm2(spc3d::Context &ctx, spc3d::Panel<SpKernels::real_t> &A,
                        spc3d::Panel<SpKernels::real_t> &B, spc3d::Plan<SpKernels::real_t> &S,
                        SpKernels::DeviceSparseComm &comm_preA,
                        SpKernels::DeviceSparseComm &comm_preB,
                        SpKernels::DeviceDenseComm &comm_post, spc3d::Vals<SpKernels::real_t> &C,
                        const SpKernels::Mesh &mesh, const std::string &mtx = "");
void dist_sddmm_spcomm3(spc3d::Context &ctx, spc3d::Panel<SpKernels::real_t> &A,
                        spc3d::Panel<SpKernels::real_t> &B, spc3d::Plan<SpKernels::real_t> &S,
                        SpKernels::DeviceSparseComm &comm_preA,
                        SpKernels::DeviceSparseComm &comm_preB,
                        SpKernels::DeviceDenseComm &comm_post, spc3d::Vals<SpKernels::real_t> &C,
                        const SpKernels::Mesh &mesh, const std::string &mtx = "");
void dist_sddmm_dcomm(spc3d::Context &ctx, spc3d::Panel<SpKernels::real_t> &A,
                      spc3d::Panel<SpKernels::real_t> &B, spc3d::Plan<SpKernels::real_t> &S,
                      SpKernels::DeviceDenseComm &comm_pre, SpKernels::DeviceDenseComm &comm_post,
                      spc3d::Vals<SpKernels::real_t> &C, const SpKernels::Mesh &mesh,
                      const std::string &mtx = "");
