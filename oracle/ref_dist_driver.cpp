// Checker: drives the reference's OWN six distributed wrappers
// (/root/reference/src/distributed_comp.cpp:17,141,194,237,285,349, compiled from
// where they lie together with src/comm_stats.cpp) on one MPI rank over a small
// seeded pattern, and prints a checksum after each call.  oracle/Makefile builds it
// twice: with the reference's src/core_ops.cpp, and with ref_binding/core_ops_hip.cpp
// (the GPU library behind the same two symbols) in its place.  All six call sites of
// SpKernels::sddmm / spmm in the reference's wrappers resolve against the binding, and
// the two programs must print the same "CHK" lines.
//
// The operands are small multiples of 1/8 and 1/4, so every product and every sum is
// exact in double whatever the order of summation: the two builds agree to the bit.
//
// Test infrastructure only; includes the reference's headers by path, copies nothing.
#include <mpi.h>

#include <cstdio>
#include <cstdlib>
#include <string>
#include <vector>

#include "distributed_comp.hpp" // the reference's

namespace {

uint64_t lcg(uint64_t &s)
{
    s = s * 6364136223846793005ull + 1442695040888963407ull;
    return s >> 33;
}

void fill(denseMatrix &M, idx_t m, idx_t n, int a, int b)
{
    M.m = m;
    M.n = n;
    M.data.resize((size_t)m * n);
    for (idx_t i = 0; i < m; ++i)
        for (idx_t j = 0; j < n; ++j)
            M.data[(size_t)i * n + j] = (double)((int)((i * a + j * b) % 11) - 5) / 8.0;
}

double weighted(const std::vector<real_t> &v)
{
    double s = 0;
    for (size_t i = 0; i < v.size(); ++i)
        s += v[i] * (double)(i % 13 + 1);
    return s;
}

void report(const char *what, const std::vector<real_t> &v)
{
    double s = 0;
    for (real_t x : v)
        s += x;
    std::printf("CHK %s %.17g %.17g\n", what, s, weighted(v));
    std::fflush(stdout);
}

// Single-rank Z reduction of SDDMM: C.vv -> C.ownedVals, all nnz of them
// (what setup_3dsddmm_reduce_scatter leaves on one rank, src/comm_setup.cpp:671-689).
void reduce_plan(cooMat &C, DenseComm &d, MPI_Comm comm)
{
    d.OP = 1;
    d.commXflag = d.commYflag = true;
    d.commX = d.commY = comm;
    d.bufferptrX = C.vv.data();
    d.bufferptrY = C.ownedVals.data();
    d.bcastXcnt.assign(1, (idx_t)C.nnz);
    d.bcastXdisp.assign(1, 0);
    d.outDegreeX = 1;
}

// A dense plan that takes part in nothing.
void idle_plan(DenseComm &d, MPI_Comm comm)
{
    d.OP = 0;
    d.commXflag = d.commYflag = false;
    d.commX = d.commY = comm;
    d.bufferptrX = d.bufferptrY = nullptr;
}

} // namespace

int main(int argc, char **argv)
{
    MPI_Init(&argc, &argv);
    const idx_t K = argc > 1 ? (idx_t)std::atoi(argv[1]) : 16;
    const idx_t m = argc > 2 ? (idx_t)std::atoi(argv[2]) : 300;
    const idx_t n = argc > 3 ? (idx_t)std::atoi(argv[3]) : 200;
    const idx_large_t nnz = argc > 4 ? (idx_large_t)std::atoll(argv[4]) : 5000;
    int dims[3] = {1, 1, 1}, periods[3] = {0, 0, 0};
    MPI_Comm cart;
    MPI_Cart_create(MPI_COMM_WORLD, 3, dims, periods, 0, &cart);

    cooMat S;
    S.mtxName = "seeded";
    S.nrows = S.gnrows = m;
    S.ncols = S.gncols = n;
    S.nnz = S.gnnz = nnz;
    S.rank = S.xyrank = S.zrank = 0;
    uint64_t seed = 12345;
    for (idx_large_t e = 0; e < nnz; ++e) {
        // a few long rows, duplicates allowed, no particular order
        const idx_t r = (lcg(seed) % 4 == 0) ? (idx_t)(lcg(seed) % 3) : (idx_t)(lcg(seed) % m);
        const idx_t c = (idx_t)(lcg(seed) % n);
        const double v = (double)(lcg(seed) % 9) / 4.0;
        S.addEntry(r, c, v);
    }
    cooMat C = S;
    C.vv.assign(nnz, 0.0);
    C.ownedVals.assign(nnz, 0.0);
    C.ownedNnz = (idx_t)nnz;

    denseMatrix A, B, Y;
    fill(A, m, K, 7, 3);
    fill(B, n, K, 5, 2);
    fill(Y, m, K, 3, 1);

    SparseComm<real_t> preA(K), preB(K), post(K);
    DenseComm red, idle1, idle2;
    reduce_plan(C, red, cart);
    idle_plan(idle1, cart);
    idle_plan(idle2, cart);

    dist_sddmm_spcomm(A, B, S, preA, red, C, cart);
    report("sddmm_spcomm", C.ownedVals);
    C.vv.assign(nnz, 0.0);
    dist_sddmm_spcomm2(A, B, S, preA, preB, red, C, cart);
    report("sddmm_spcomm2", C.ownedVals);
    C.vv.assign(nnz, 0.0);
    dist_sddmm_spcomm3(A, B, S, preA, preB, red, C, cart);
    report("sddmm_spcomm3", C.ownedVals);
    C.vv.assign(nnz, 0.0);
    dist_sddmm_dcomm(A, B, S, idle1, red, C, cart);
    report("sddmm_dcomm", C.ownedVals);

    dist_spmm_spcomm(B, S, Y, preA, post, cart);
    report("spmm_spcomm", Y.data);
    dist_spmm_dcomm(B, Y, S, idle1, idle2, cart); // adds to what the call before left
    report("spmm_dcomm", Y.data);

    MPI_Finalize();
    return 0;
}
