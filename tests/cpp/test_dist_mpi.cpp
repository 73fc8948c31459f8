// The mirror's dist_* wrappers under the reference's own signatures
// (src/distributed_comp.hpp:11-64: void, last parameter MPI_Comm), the way a
// reference caller writes them (miniapp/bench_both.cpp:202-203): a 1 x 1 x 1
// Cartesian communicator, five calls, results against serial loops.  A
// communicator that is not the 3D Cartesian one is refused.
//
// Built only where an mpi.h is found (tests/cpp/Makefile); needs a GPU and the MPI
// library at run time.
#include <mpi.h>

#include <cmath>
#include <cstdio>
#include <random>
#include <stdexcept>
#include <type_traits>

#include "spc3d/distributed_comp.hpp"

using namespace SpKernels;
using namespace DComm;

static int g_fail = 0;
#define CHECK(cond)                                                                               \
    do {                                                                                          \
        if (!(cond)) {                                                                            \
            std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond);                           \
            ++g_fail;                                                                             \
        }                                                                                         \
    } while (0)

// the six symbols have the reference's types
using sp_t = SparseComm<real_t>;
static_assert(std::is_same_v<decltype(static_cast<void (*)(denseMatrix &, cooMat &, denseMatrix &, sp_t &, sp_t &, MPI_Comm)>(&dist_spmm_spcomm)),
                             void (*)(denseMatrix &, cooMat &, denseMatrix &, sp_t &, sp_t &, MPI_Comm)>);
static_assert(std::is_same_v<decltype(static_cast<void (*)(denseMatrix &, denseMatrix &, cooMat &, DenseComm &, DenseComm &, MPI_Comm)>(&dist_spmm_dcomm)),
                             void (*)(denseMatrix &, denseMatrix &, cooMat &, DenseComm &, DenseComm &, MPI_Comm)>);
static_assert(std::is_same_v<decltype(static_cast<void (*)(denseMatrix &, denseMatrix &, cooMat &, sp_t &, DenseComm &, cooMat &, MPI_Comm)>(&dist_sddmm_spcomm)),
                             void (*)(denseMatrix &, denseMatrix &, cooMat &, sp_t &, DenseComm &, cooMat &, MPI_Comm)>);
static_assert(std::is_same_v<decltype(static_cast<void (*)(denseMatrix &, denseMatrix &, cooMat &, sp_t &, sp_t &, DenseComm &, cooMat &, MPI_Comm)>(&dist_sddmm_spcomm2)),
                             void (*)(denseMatrix &, denseMatrix &, cooMat &, sp_t &, sp_t &, DenseComm &, cooMat &, MPI_Comm)>);
static_assert(std::is_same_v<decltype(static_cast<void (*)(denseMatrix &, denseMatrix &, cooMat &, sp_t &, sp_t &, DenseComm &, cooMat &, MPI_Comm)>(&dist_sddmm_spcomm3)),
                             void (*)(denseMatrix &, denseMatrix &, cooMat &, sp_t &, sp_t &, DenseComm &, cooMat &, MPI_Comm)>);
static_assert(std::is_same_v<decltype(static_cast<void (*)(denseMatrix &, denseMatrix &, cooMat &, DenseComm &, DenseComm &, cooMat &, MPI_Comm)>(&dist_sddmm_dcomm)),
                             void (*)(denseMatrix &, denseMatrix &, cooMat &, DenseComm &, DenseComm &, cooMat &, MPI_Comm)>);

static const double kTol = sizeof(real_t) == 8 ? 1e-12 : 1e-5;

int main(int argc, char **argv)
{
    MPI_Init(&argc, &argv);
    int dims[3] = {1, 1, 1}, periods[3] = {0, 0, 0};
    MPI_Comm cart;
    MPI_Cart_create(MPI_COMM_WORLD, 3, dims, periods, 0, &cart);

    const idx_t m = 500, n = 300, k = 24;
    const idx_large_t nnz = 20000;
    std::mt19937 g(5);
    cooMat S;
    S.mtxName = "mpi1";
    S.nrows = S.gnrows = m;
    S.ncols = S.gncols = n;
    for (idx_large_t e = 0; e < nnz; ++e)
        S.addEntry((idx_t)(g() % 7 == 0 ? g() % 2 : g() % m), (idx_t)(g() % n),
                   (real_t)((double)(g() % 1000) / 500.0 - 1.0));
    S.nnz = S.gnnz = nnz;
    cooMat C = S;
    denseMatrix A, B, Y;
    auto fill = [&](denseMatrix &M, idx_t rows) {
        M.m = rows;
        M.n = k;
        M.data.resize((size_t)rows * k);
        for (auto &x : M.data)
            x = (real_t)((double)(g() % 2000) / 1000.0 - 1.0);
    };
    fill(A, m);
    fill(B, n);
    fill(Y, m);
    std::vector<real_t> c_ref(nnz), y_ref = Y.data;
    for (idx_large_t e = 0; e < nnz; ++e) { // src/core_ops.cpp:11-21
        real_t s = 0;
        for (idx_t j = 0; j < k; ++j)
            s += A.at(S.ii[e], j) * B.at(S.jj[e], j);
        c_ref[e] = s * S.vv[e];
    }

    sp_t preA(k), preB(k), post(k);
    DenseComm red, idle;
    setup_sddmm_reduce_single_rank(C, red);
    idle.OP = 0;
    dist_set_stats_stream(nullptr);

    auto close = [&](const std::vector<real_t> &got, const std::vector<real_t> &want, double scale) {
        double worst = 0;
        for (size_t i = 0; i < want.size(); ++i)
            worst = std::fmax(worst, std::fabs((double)got[i] - (double)want[i]) /
                                         std::fmax(std::fabs((double)want[i]), scale));
        return worst < kTol;
    };
    for (int rep = 0; rep < 5; ++rep) { // miniapp/bench_both.cpp:202-203
        std::fill(C.vv.begin(), C.vv.end(), (real_t)0);
        dist_sddmm_spcomm(A, B, S, preA, red, C, cart);
        CHECK(close(C.ownedVals, c_ref, (double)k));
    }
    std::fill(C.vv.begin(), C.vv.end(), (real_t)0);
    dist_sddmm_spcomm2(A, B, S, preA, preB, red, C, cart);
    CHECK(close(C.ownedVals, c_ref, (double)k));
    std::fill(C.vv.begin(), C.vv.end(), (real_t)0);
    dist_sddmm_spcomm3(A, B, S, preA, preB, red, C, cart);
    CHECK(close(C.ownedVals, c_ref, (double)k));
    std::fill(C.vv.begin(), C.vv.end(), (real_t)0);
    dist_sddmm_dcomm(A, B, S, idle, red, C, cart);
    CHECK(close(C.ownedVals, c_ref, (double)k));
    CHECK(dist_last_timing().compTimeUs > 0);

    for (int rep = 0; rep < 2; ++rep) { // Y accumulates over calls (src/core_ops.cpp:32)
        for (idx_large_t e = 0; e < nnz; ++e)
            for (idx_t j = 0; j < k; ++j)
                y_ref[(size_t)S.ii[e] * k + j] += S.vv[e] * B.at(S.jj[e], j);
    }
    dist_spmm_spcomm(B, S, Y, preA, post, cart);
    dist_spmm_dcomm(B, Y, S, idle, idle, cart);
    CHECK(close(Y.data, y_ref, 200.0));

    bool threw = false;
    try {
        dist_spmm_spcomm(B, S, Y, preA, post, MPI_COMM_WORLD); // no Cartesian topology
    } catch (const std::runtime_error &) {
        threw = true;
    }
    CHECK(threw);

    MPI_Comm_free(&cart);
    MPI_Finalize();
    std::printf("%s (%d failures, real_t = %s)\n", g_fail ? "FAILED" : "PASSED", g_fail,
                sizeof(real_t) == 8 ? "double" : "float");
    return g_fail ? 1 : 0;
}
