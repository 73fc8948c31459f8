// What the host-memory and the device-resident wrappers share: the statistics lines of
// src/comm_stats.cpp for one rank, and the record of the last call's phase times.
#pragma once

#include <cstdio>
#include <numeric>
#include <stdexcept>
#include <string>

#include "spc3d/distributed_comp.hpp"

namespace spc3d_dist {

using namespace SpKernels;

std::FILE *&stats_stream();   // where the lines go (nullptr: nowhere)
distTiming &last_timing();    // of the calling thread

inline void require_single(const Mesh &mesh)
{
    if (mesh.X != 1 || mesh.Y != 1 || mesh.Z != 1)
        throw std::runtime_error("dist_*: this library runs one rank on one GPU; the mesh must be "
                                 "1 x 1 x 1");
}

// "mtx alg P Kloc Z avgSendMsg avgSendVol avgRecvMsg avgRecvVol maxSendMsg
//  maxSendVol maxRecvMsg maxRecvVol comm1 comm2 commcpy comp total"
// (src/comm_stats.cpp:33-36,53,71-73) with P = 1: averages equal maxima.
inline void print_line(const std::string &mtx, const char *alg, idx_t f, const Mesh &mesh,
                       idx_large_t sendMsg, idx_large_t sendVol, idx_large_t recvMsg,
                       idx_large_t recvVol, const parallelTiming &pt)
{
    std::FILE *out = stats_stream();
    if (!out)
        return;
    std::fprintf(out, "%s %s %d %u %d %.2f %.2f %.2f %.2f %lu %lu %lu %lu %u %u %u %u %u\n",
                 mtx.c_str(), alg, 1, f, mesh.Z, (float)sendMsg, (float)sendVol, (float)recvMsg,
                 (float)recvVol, (unsigned long)sendMsg, (unsigned long)sendVol,
                 (unsigned long)recvMsg, (unsigned long)recvVol, pt.comm1Time, pt.comm2Time,
                 pt.commcpyTime, pt.compTime, pt.totalTime);
}

// src/comm_stats.cpp:59-73; Comm: SparseComm<real_t> or its device form
template <typename Comm>
void stats_sparse(const std::string &mtx, const char *alg, const Comm &c, idx_t f,
                  const parallelTiming &pt, const Mesh &mesh)
{
    const idx_large_t sv = (idx_large_t)std::accumulate(c.sendCount.begin(), c.sendCount.end(), 0.0);
    const idx_large_t rv = (idx_large_t)std::accumulate(c.recvCount.begin(), c.recvCount.end(), 0.0);
    print_line(mtx, alg, f, mesh, (idx_large_t)c.outDegree, sv, (idx_large_t)c.inDegree, rv, pt);
}

// src/comm_stats.cpp:74-92
template <typename Comm>
void stats_sparse2(const std::string &mtx, const char *alg, const Comm &a, const Comm &b, idx_t f,
                   const parallelTiming &pt, const Mesh &mesh)
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

// src/comm_stats.cpp:93-129, with this rank being rank 0 of every sub-communicator.
// reduce_scatter: OP 1 with both flags; cnt0 / last_end: bcastXcnt[0] and the end of the
// last block of the send buffer; all_x / all_y: sums of bcastXcnt / bcastYcnt; x0 / y0: this
// rank's own blocks.
struct DenseShape {
    bool reduce_scatter = false, x = false, y = false;
    idx_large_t cnt0 = 0, last_end = 0, all_x = 0, all_y = 0, x0 = 0, y0 = 0;
    int outDegreeX = 0, outDegreeY = 0;
};
inline void stats_dense(const std::string &mtx, const char *alg, const DenseShape &d, idx_t f,
                        const parallelTiming &pt, const Mesh &mesh)
{
    idx_large_t sendVol = 0, recvVol = 0, sendMsg = 1, recvMsg = 0;
    if (d.reduce_scatter) {
        sendVol = d.last_end;
        recvVol = d.cnt0;
        recvMsg = 1;
    } else {
        const idx_large_t all = (d.x ? d.all_x : 0) + (d.y ? d.all_y : 0);
        sendVol = (d.x ? d.x0 : 0) + (d.y ? d.y0 : 0);
        recvVol = all - sendVol;
        recvMsg = (d.x ? d.outDegreeX : 0) + (d.y ? d.outDegreeY : 0);
    }
    print_line(mtx, alg, f, mesh, sendMsg, sendVol, recvMsg, recvVol, pt);
}

} // namespace spc3d_dist
