// The reference's distributed kernel wrappers (src/distributed_comp.hpp:11-64),
// for ONE rank on ONE GPU: pre-communication, the local kernel, post-
// communication, and the reference's statistics line, with the reference's
// names, parameter order and return type (void).  With a single rank every
// exchange is empty (inDegree = outDegree = 0, src/comm.hpp:66-70) and the Z
// reduction of SDDMM is a copy of C.vv into C.ownedVals (MPI_Reduce_scatter over
// one rank, src/denseComm.hpp:39 with the buffers of src/comm_setup.cpp:678-679),
// so this header carries single-rank stand-ins for SparseComm / DenseComm instead
// of MPI: the MPI communication layer itself is outside this library.
//
// The last parameter of every wrapper is the process mesh.  The reference passes
// the Cartesian communicator and reads its dimensions back
// (src/distributed_comp.cpp:25-27): compiled with -DSPC3D_WITH_MPI (and an mpi.h
// on the include path) this header declares exactly those signatures,
// `void dist_*(..., MPI_Comm comm)`, which read the dimensions with MPI_Cart_get
// and refuse anything but 1 x 1 x 1.  Without MPI the same wrappers take the
// dimensions themselves (`const Mesh &`).  The phase times the reference keeps in
// a local and only prints are also kept for the caller: dist_last_timing().
#pragma once

#include <cstdio>
#include <stdexcept>
#include <string>
#include <vector>

#include "SparseMatrix.hpp"
#include "basic.hpp"

#ifdef SPC3D_WITH_MPI
#include <mpi.h>
#endif

namespace SpKernels {

struct Mesh {
    int X = 1, Y = 1, Z = 1;
};

// Sparse point-to-point plan of one rank (src/comm.hpp:33-52): who sends what to
// whom.  On one rank the only possible peer is the rank itself: a plan may hold
// messages addressed to rank 0 (what MPI delivers when a rank sends to itself), which
// exercises the copies either side of an exchange (src/comm.hpp:90-103,166-189)
// exactly as the reference runs them; a plan that names any other rank cannot be
// executed here.  Counts and displacements are in reals, as in the reference; send i is
// matched with receive i (one source, one tag: MPI matches them in order).
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

    void issue_Irecvs() { require_self(); }
    // with_DT: the reference sends straight out of the dense panel through derived
    // datatypes (src/comm.hpp:113-118); no self-addressed form of that is kept here.
    void issue_Sends(bool with_DT = false)
    {
        require_self();
        if (with_DT && outDegree != 0)
            throw std::runtime_error("SparseComm: datatype sends have no single-rank form");
        for (int i = 0; i < outDegree; ++i) {
            if (sendCount.at(i) != recvCount.at(i))
                throw std::runtime_error("SparseComm: a self-addressed message must be received "
                                         "with the length it is sent with");
            for (int k = 0; k < sendCount[i]; ++k)
                recvBuff.at((size_t)recvDisp.at(i) + k) = sendBuff.at((size_t)sendDisp.at(i) + k);
        }
    }
    void issue_Waitall() { require_self(); }
    void copy_to_sendbuff() // src/comm.hpp:90-103
    {
        require_self();
        size_t idx = 0;
        for (size_t i = 0; i < sendptr.size(); ++i)
            for (size_t j = 0; j < dataUnitSize; ++j)
                sendBuff.at(idx++) = sendptr[i][j];
    }
    void copy_from_recvbuff() // src/comm.hpp:166-177
    {
        require_self();
        size_t idx = 0;
        for (size_t i = 0; i < recvptr.size(); ++i)
            for (size_t j = 0; j < dataUnitSize; ++j)
                recvptr[i][j] = recvBuff.at(idx++);
    }
    void SUM_from_recvbuff() // src/comm.hpp:178-189
    {
        require_self();
        size_t idx = 0;
        for (size_t i = 0; i < recvptr.size(); ++i)
            for (size_t j = 0; j < dataUnitSize; ++j)
                recvptr[i][j] += recvBuff.at(idx++);
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
            throw std::runtime_error("SparseComm: exchanges between ranks are outside this "
                                     "single-GPU library (only messages a rank addresses to "
                                     "itself can be carried out)");
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
// (src/comm_stats.cpp:33-36,53).
void dist_spmm_spcomm(SpKernels::denseMatrix &X, SpKernels::cooMat &A,
                      SpKernels::denseMatrix &Y,
                      SpKernels::SparseComm<SpKernels::real_t> &comm_pre,
                      SpKernels::SparseComm<SpKernels::real_t> &comm_post,
                      const SpKernels::Mesh &mesh);
void dist_spmm_dcomm(SpKernels::denseMatrix &X, SpKernels::denseMatrix &Y,
                     SpKernels::cooMat &A, DComm::DenseComm &comm_pre,
                     DComm::DenseComm &comm_post,
                     const SpKernels::Mesh &mesh);
void dist_sddmm_spcomm(SpKernels::denseMatrix &A, SpKernels::denseMatrix &B,
                       SpKernels::cooMat &S,
                       SpKernels::SparseComm<SpKernels::real_t> &comm_pre,
                       DComm::DenseComm &comm_post, SpKernels::cooMat &C,
                       const SpKernels::Mesh &mesh);
void dist_sddmm_spcomm2(SpKernels::denseMatrix &A, SpKernels::denseMatrix &B,
                        SpKernels::cooMat &S,
                        SpKernels::SparseComm<SpKernels::real_t> &comm_preA,
                        SpKernels::SparseComm<SpKernels::real_t> &comm_preB,
                        DComm::DenseComm &comm_post, SpKernels::cooMat &C,
                        const SpKernels::Mesh &mesh);
void dist_sddmm_spcomm3(SpKernels::denseMatrix &A, SpKernels::denseMatrix &B,
                        SpKernels::cooMat &S,
                        SpKernels::SparseComm<SpKernels::real_t> &comm_preA,
                        SpKernels::SparseComm<SpKernels::real_t> &comm_preB,
                        DComm::DenseComm &comm_post, SpKernels::cooMat &C,
                        const SpKernels::Mesh &mesh);
void dist_sddmm_dcomm(SpKernels::denseMatrix &A, SpKernels::denseMatrix &B,
                      SpKernels::cooMat &S, DComm::DenseComm &comm_pre,
                      DComm::DenseComm &comm_post, SpKernels::cooMat &C,
                      const SpKernels::Mesh &mesh);

// Where the statistics lines go (default stdout); nullptr silences them.
void dist_set_stats_stream(std::FILE *f);

// Phase times of the last dist_* call on this thread: the reference's five
// millisecond counters, and the compute phase again as the device measured it, in
// microseconds (a GPU kernel lasts well under the reference's 1 ms resolution).
// The device-resident wrappers (distributed_comp_device.hpp) fill every microsecond field
// from device events; the host-memory wrappers fill compTimeUs only.
struct distTiming {
    SpKernels::parallelTiming pt;
    SpKernels::idx_large_t compTimeUs = 0;
    SpKernels::idx_large_t comm1TimeUs = 0, comm2TimeUs = 0, commcpyTimeUs = 0, totalTimeUs = 0;
};
const distTiming &dist_last_timing();

#ifdef SPC3D_WITH_MPI
// The reference's own signatures (src/distributed_comp.hpp:11-64).  Inline, so
// that the library itself needs no MPI: the caller's translation unit, which has
// the communicator, links the MPI library it was made with.
namespace spc3d_detail {
inline SpKernels::Mesh mesh_of(MPI_Comm comm)
{
    int dims[3] = {0, 0, 0}, periods[3], coords[3], nd = 0, topo = MPI_UNDEFINED;
    MPI_Topo_test(comm, &topo);
    if (topo == MPI_CART)
        MPI_Cartdim_get(comm, &nd);
    if (topo != MPI_CART || nd != 3)
        throw std::runtime_error("dist_*: the communicator must be the 3D Cartesian one "
                                 "(src/distributed_comp.cpp:25-27)");
    MPI_Cart_get(comm, 3, dims, periods, coords);
    SpKernels::Mesh m;
    m.X = dims[0];
    m.Y = dims[1];
    m.Z = dims[2];
    return m;
}
} // namespace spc3d_detail

inline void dist_spmm_spcomm(SpKernels::denseMatrix &X, SpKernels::cooMat &A,
                             SpKernels::denseMatrix &Y,
                             SpKernels::SparseComm<SpKernels::real_t> &comm_pre,
                             SpKernels::SparseComm<SpKernels::real_t> &comm_post, MPI_Comm comm)
{
    dist_spmm_spcomm(X, A, Y, comm_pre, comm_post, spc3d_detail::mesh_of(comm));
}
inline void dist_spmm_dcomm(SpKernels::denseMatrix &X, SpKernels::denseMatrix &Y,
                            SpKernels::cooMat &A, DComm::DenseComm &comm_pre,
                            DComm::DenseComm &comm_post, MPI_Comm comm)
{
    dist_spmm_dcomm(X, Y, A, comm_pre, comm_post, spc3d_detail::mesh_of(comm));
}
inline void dist_sddmm_spcomm(SpKernels::denseMatrix &A, SpKernels::denseMatrix &B,
                              SpKernels::cooMat &S,
                              SpKernels::SparseComm<SpKernels::real_t> &comm_pre,
                              DComm::DenseComm &comm_post, SpKernels::cooMat &C, MPI_Comm comm)
{
    dist_sddmm_spcomm(A, B, S, comm_pre, comm_post, C, spc3d_detail::mesh_of(comm));
}
inline void dist_sddmm_spcomm2(SpKernels::denseMatrix &A, SpKernels::denseMatrix &B,
                               SpKernels::cooMat &S,
                               SpKernels::SparseComm<SpKernels::real_t> &comm_preA,
                               SpKernels::SparseComm<SpKernels::real_t> &comm_preB,
                               DComm::DenseComm &comm_post, SpKernels::cooMat &C, MPI_Comm comm)
{
    dist_sddmm_spcomm2(A, B, S, comm_preA, comm_preB, comm_post, C, spc3d_detail::mesh_of(comm));
}
inline void dist_sddmm_spcomm3(SpKernels::denseMatrix &A, SpKernels::denseMatrix &B,
                               SpKernels::cooMat &S,
                               SpKernels::SparseComm<SpKernels::real_t> &comm_preA,
                               SpKernels::SparseComm<SpKernels::real_t> &comm_preB,
                               DComm::DenseComm &comm_post, SpKernels::cooMat &C, MPI_Comm comm)
{
    dist_sddmm_spcomm3(A, B, S, comm_preA, comm_preB, comm_post, C, spc3d_detail::mesh_of(comm));
}
inline void dist_sddmm_dcomm(SpKernels::denseMatrix &A, SpKernels::denseMatrix &B,
                             SpKernels::cooMat &S, DComm::DenseComm &comm_pre,
                             DComm::DenseComm &comm_post, SpKernels::cooMat &C, MPI_Comm comm)
{
    dist_sddmm_dcomm(A, B, S, comm_pre, comm_post, C, spc3d_detail::mesh_of(comm));
}
#endif // SPC3D_WITH_MPI
