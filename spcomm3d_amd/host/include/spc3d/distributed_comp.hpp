// The reference's distributed kernel wrappers (src/distributed_comp.hpp:11-64),
// for ONE rank on ONE GPU: pre-communication, the local kernel, post-
// communication, and the reference's statistics line, with the reference's
// names and parameter order.  With a single rank every exchange is empty
// (inDegree = outDegree = 0, src/comm.hpp:66-70) and the Z reduction of SDDMM is
// a copy of C.vv into C.ownedVals (MPI_Reduce_scatter over one rank,
// src/denseComm.hpp:39 with the buffers of src/comm_setup.cpp:678-679), so
// this header carries single-rank stand-ins for SparseComm / DenseComm instead
// of MPI: the MPI communication layer itself is outside this library.
//
// The last parameter of every wrapper is the process mesh (the reference passes
// the Cartesian communicator and reads its dimensions back, e.g.
// src/distributed_comp.cpp:25-27); here it is the dimensions themselves and
// must be 1 x 1 x 1.
#pragma once

#include <cstdio>
#include <stdexcept>
#include <string>
#include <vector>

#include "SparseMatrix.hpp"
#include "basic.hpp"

namespace SpKernels {

struct Mesh {
    int X = 1, Y = 1, Z = 1;
};

// Sparse point-to-point plan of one rank (src/comm.hpp:33-52): who sends what
// to whom.  On one rank there is nobody to talk to; a plan that says otherwise
// cannot be executed here.
template <typename T> class SparseComm {
  public:
    int inDegree = 0, outDegree = 0;
    idx_t dataUnitSize = 1;
    std::vector<int> inSet, outSet;
    std::vector<int> sendCount, recvCount;
    std::vector<int> sendDisp, recvDisp;
    std::vector<T> sendBuff, recvBuff;
    std::vector<T *> sendptr, recvptr;

    SparseComm() = default;
    explicit SparseComm(idx_t unitSize) : dataUnitSize(unitSize) {}

    void issue_Irecvs() { require_single(); }
    void issue_Sends(bool = false) { require_single(); }
    void issue_Waitall() { require_single(); }
    void copy_to_sendbuff() { require_single(); }
    void copy_from_recvbuff() { require_single(); }
    void SUM_from_recvbuff() { require_single(); }
    void perform_sparse_comm(bool = true, bool = true) { require_single(); }

  private:
    void require_single() const
    {
        if (inDegree != 0 || outDegree != 0)
            throw std::runtime_error("SparseComm: exchanges between ranks are outside this "
                                     "single-GPU library");
    }
};

} // namespace SpKernels

namespace DComm {

using SpKernels::idx_t;
using SpKernels::real_t;

// Dense collective plan (src/denseComm.hpp:12-48).  OP 0 = broadcasts, OP 1 =
// reduction; commXflag / commYflag say which sub-communicators take part.
struct DenseComm {
    int OP = 1;
    bool commXflag = false, commYflag = false;
    real_t *bufferptrX = nullptr, *bufferptrY = nullptr;
    int outDegreeX = 0, outDegreeY = 0;
    std::vector<idx_t> bcastXcnt, bcastYcnt, bcastXdisp, bcastYdisp;
    std::vector<real_t> reduceBuffer;

    // One rank: a broadcast from oneself and an in-place all-reduce change
    // nothing; a reduce-scatter (both flags, OP 1) delivers the whole send
    // buffer: bufferptrY[0 .. bcastXcnt[0]) = bufferptrX[0 .. bcastXcnt[0]).
    void perform_dense_comm()
    {
        if (OP == 1 && commXflag && commYflag && bufferptrX && bufferptrY && !bcastXcnt.empty() &&
            bufferptrX != bufferptrY)
            for (idx_t i = 0; i < bcastXcnt[0]; ++i)
                bufferptrY[i] = bufferptrX[i];
    }
};

} // namespace DComm

// Single-rank form of setup_3dsddmm_reduce_scatter (src/comm_setup.cpp:671-689):
// the Z reduction sends C.vv and receives C.ownedVals, all nnz of them.
void setup_sddmm_reduce_single_rank(SpKernels::cooMat &C, DComm::DenseComm &comm_post);

// src/distributed_comp.hpp:11-64.  Each prints the reference's statistics lines
// (src/comm_stats.cpp:33-36,53) and returns the phase times of the call.
SpKernels::parallelTiming dist_spmm_spcomm(SpKernels::denseMatrix &X, SpKernels::cooMat &A,
                                           SpKernels::denseMatrix &Y,
                                           SpKernels::SparseComm<SpKernels::real_t> &comm_pre,
                                           SpKernels::SparseComm<SpKernels::real_t> &comm_post,
                                           const SpKernels::Mesh &mesh);
SpKernels::parallelTiming dist_spmm_dcomm(SpKernels::denseMatrix &X, SpKernels::denseMatrix &Y,
                                          SpKernels::cooMat &A, DComm::DenseComm &comm_pre,
                                          DComm::DenseComm &comm_post,
                                          const SpKernels::Mesh &mesh);
SpKernels::parallelTiming dist_sddmm_spcomm(SpKernels::denseMatrix &A, SpKernels::denseMatrix &B,
                                            SpKernels::cooMat &S,
                                            SpKernels::SparseComm<SpKernels::real_t> &comm_pre,
                                            DComm::DenseComm &comm_post, SpKernels::cooMat &C,
                                            const SpKernels::Mesh &mesh);
SpKernels::parallelTiming dist_sddmm_spcomm2(SpKernels::denseMatrix &A, SpKernels::denseMatrix &B,
                                             SpKernels::cooMat &S,
                                             SpKernels::SparseComm<SpKernels::real_t> &comm_preA,
                                             SpKernels::SparseComm<SpKernels::real_t> &comm_preB,
                                             DComm::DenseComm &comm_post, SpKernels::cooMat &C,
                                             const SpKernels::Mesh &mesh);
SpKernels::parallelTiming dist_sddmm_spcomm3(SpKernels::denseMatrix &A, SpKernels::denseMatrix &B,
                                             SpKernels::cooMat &S,
                                             SpKernels::SparseComm<SpKernels::real_t> &comm_preA,
                                             SpKernels::SparseComm<SpKernels::real_t> &comm_preB,
                                             DComm::DenseComm &comm_post, SpKernels::cooMat &C,
                                             const SpKernels::Mesh &mesh);
SpKernels::parallelTiming dist_sddmm_dcomm(SpKernels::denseMatrix &A, SpKernels::denseMatrix &B,
                                           SpKernels::cooMat &S, DComm::DenseComm &comm_pre,
                                           DComm::DenseComm &comm_post, SpKernels::cooMat &C,
                                           const SpKernels::Mesh &mesh);

// Where the statistics lines go (default stdout); nullptr silences them.
void dist_set_stats_stream(std::FILE *f);
