// C entry point around the reference's own SparseComm::copy_to_sendbuff /
// copy_from_recvbuff / SUM_from_recvbuff (src/comm.hpp:90-103,166-189).
// TEST INFRASTRUCTURE ONLY, built like ref_shim.cpp (oracle/Makefile, target
// `ref`) where the reference tree and an mpi.h are present: comm.hpp includes
// <mpi.h> for the types of its members; the three methods used here call no MPI
// function, and nothing of MPI is linked.  fp64 only (the reference's real_t).
//
// This file contains no reference code; it includes the reference header by path.
#include <cassert>
#include <cstdint>
#include <cstring>
#include <exception>
#include <numeric>

#include "comm.hpp"

using namespace SpKernels;

extern "C" {

// op 0: buf[i,:] = panel[rows[i],:]; op 1: panel[rows[i],:] = buf[i,:];
// op 2: panel[rows[i],:] += buf[i,:]; k reals per row, nslots rows.  Returns 0,
// or -1 for a bad argument.
__attribute__((visibility("default"))) int
ref_rows_f64(int op, uint32_t panel_rows, uint32_t k, double *panel, uint64_t nslots,
             const uint32_t *rows, double *buf)
{
    if (op < 0 || op > 2 || k == 0)
        return -1;
    for (uint64_t i = 0; i < nslots; ++i)
        if (rows[i] >= panel_rows)
            return -1;
    try {
        SparseComm<double> comm(k);
        if (op == 0) {
            comm.sendCount.assign(1, (int)(nslots * k)); // the method asserts on their sum
            comm.sendBuffPtr = buf;
            for (uint64_t i = 0; i < nslots; ++i)
                comm.sendptr.push_back(panel + (size_t)rows[i] * k);
            comm.copy_to_sendbuff();
        } else {
            comm.recvBuffPtr = buf;
            for (uint64_t i = 0; i < nslots; ++i)
                comm.recvptr.push_back(panel + (size_t)rows[i] * k);
            if (op == 1)
                comm.copy_from_recvbuff();
            else
                comm.SUM_from_recvbuff();
        }
        return 0;
    } catch (const std::exception &) {
        return -1;
    }
}
}
