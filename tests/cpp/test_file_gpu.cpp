// From a file to the GPU kernels through this build's own readers: MatrixMarket and
// binary files -> spc3d/io.hpp -> (block selection) -> localizeIndices -> SpKernels::sddmm
// and spmm on the GPU -> the CPU oracle.
//
//   test_file_gpu <dir with the golden files> <k>
//
// For every golden .mtx it also prints "SUM <stem> <value>" with the fill and the output
// format of the reference's sequential checker (miniapp/numCheckSeq.cpp:118-132), so that
// the caller can hold the line against what the reference's own program prints for the file.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <iostream>
#include <numeric>
#include <string>
#include <vector>

#include "spc3d/core_ops.hpp"
#include "spc3d/device.hpp"
#include "spc3d/io.hpp"

extern "C" {
int oracle_sddmm_f64(uint32_t, uint32_t, uint32_t, const double *, const double *, uint64_t,
                     const uint32_t *, const uint32_t *, const double *, double *);
int oracle_spmm_f64(uint32_t, uint32_t, uint32_t, const double *, uint64_t, const uint32_t *,
                    const uint32_t *, const double *, double *);
int oracle_sddmm_f32(uint32_t, uint32_t, uint32_t, const float *, const float *, uint64_t,
                     const uint32_t *, const uint32_t *, const float *, float *);
int oracle_spmm_f32(uint32_t, uint32_t, uint32_t, const float *, uint64_t, const uint32_t *,
                    const uint32_t *, const float *, float *);
}

using namespace SpKernels;

static int g_fail = 0;
#define CHECK(cond)                                                                               \
    do {                                                                                          \
        if (!(cond)) {                                                                            \
            std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond);                           \
            ++g_fail;                                                                             \
        }                                                                                         \
    } while (0)

static const double kTol = sizeof(real_t) == 8 ? 1e-12 : 1e-5;

// GPU SDDMM and SpMM over S (local indices) against the oracle; returns the SDDMM result.
static std::vector<real_t> run_both(const cooMat &S0, const denseMatrix &A0, const denseMatrix &B0)
{
    cooMat S = S0, C = S0;
    denseMatrix A = A0, B = B0, Y;
    Y.m = A.m;
    Y.n = A.n;
    Y.data.assign((size_t)Y.m * Y.n, (real_t)0.25);
    std::vector<real_t> c_ref(S.nnz), y_ref = Y.data;
    int rc1, rc2;
    if constexpr (sizeof(real_t) == 8) {
        rc1 = oracle_sddmm_f64(A.m, B.m, A.n, (const double *)A.data.data(), (const double *)B.data.data(),
                               S.nnz, S.ii.data(), S.jj.data(), (const double *)S.vv.data(), (double *)c_ref.data());
        rc2 = oracle_spmm_f64(B.m, Y.m, B.n, (const double *)B.data.data(), S.nnz, S.ii.data(), S.jj.data(),
                              (const double *)S.vv.data(), (double *)y_ref.data());
    } else {
        rc1 = oracle_sddmm_f32(A.m, B.m, A.n, (const float *)A.data.data(), (const float *)B.data.data(),
                               S.nnz, S.ii.data(), S.jj.data(), (const float *)S.vv.data(), (float *)c_ref.data());
        rc2 = oracle_spmm_f32(B.m, Y.m, B.n, (const float *)B.data.data(), S.nnz, S.ii.data(), S.jj.data(),
                              (const float *)S.vv.data(), (float *)y_ref.data());
    }
    CHECK(rc1 == 0 && rc2 == 0);
    std::fill(C.vv.begin(), C.vv.end(), (real_t)-7);
    sddmm(A, B, S, C);
    spmm(B, S, Y);
    double amax = 0, bmax = 0;
    for (real_t x : A.data)
        amax = std::fmax(amax, std::fabs((double)x));
    for (real_t x : B.data)
        bmax = std::fmax(bmax, std::fabs((double)x));
    for (idx_large_t e = 0; e < S.nnz; ++e) {
        const double scale = std::fabs((double)S.vv[e]) * amax * bmax * A.n;
        CHECK(std::fabs((double)C.vv[e] - (double)c_ref[e]) <= kTol * std::fmax(std::fabs((double)c_ref[e]), scale));
    }
    std::vector<double> deg(Y.m, 0.0);
    for (idx_large_t e = 0; e < S.nnz; ++e)
        deg[S.ii[e]] += std::fabs((double)S.vv[e]);
    for (size_t i = 0; i < Y.data.size(); ++i) {
        const double scale = 0.25 + deg[i / Y.n] * bmax;
        CHECK(std::fabs((double)Y.data[i] - (double)y_ref[i]) <= kTol * std::fmax(std::fabs((double)y_ref[i]), scale));
    }
    return C.vv;
}

// i / 1000 in every column of row i (miniapp/numCheckSeq.cpp:125-128); `global` names the
// global id of local row i when the rows are a block's
static denseMatrix ramp(idx_t m, idx_t k, const std::vector<idx_t> *global = nullptr)
{
    denseMatrix M;
    M.m = m;
    M.n = k;
    M.data.resize((size_t)m * k);
    for (idx_t i = 0; i < m; ++i)
        for (idx_t j = 0; j < k; ++j)
            M.data[(size_t)i * k + j] = (real_t)(global ? (*global)[i] : i) / (real_t)1000;
    return M;
}

int main(int argc, char **argv)
{
    if (argc < 3) {
        std::printf("usage: test_file_gpu <golden dir> <k>\n");
        return 2;
    }
    const std::string dir = argv[1];
    const idx_t k = (idx_t)std::atoi(argv[2]);
    try {
        for (const char *stem : {"general", "symmetric", "integer", "pattern_symmetric", "complex"}) {
            // the text file, as the reference's sequential checker reads it
            cooMat S;
            mm reader(dir + "/" + stem + ".mtx");
            reader.read_mm(dir + "/" + stem + ".mtx", S);
            const std::vector<real_t> c = run_both(S, ramp(S.gnrows, k), ramp(S.gncols, k));
            const real_t sum = std::accumulate(c.begin(), c.end(), 0.0); // :131
            std::cout << "SUM " << stem << " " << sum << std::endl;          // :132
            // the binary file: same matrix, same result, bit for bit
            cooMat R;
            read_binary(dir + "/" + stem + ".bin", R);
            CHECK(R.ii == S.ii && R.jj == S.jj && R.vv == S.vv);
            CHECK(run_both(R, ramp(R.gnrows, k), ramp(R.gncols, k)) == c); // same input, same plan
            // as one rank's blocks of a 2 x 2 mesh, localized: every block on the GPU, and the
            // block results put back at their file positions give the whole-file result
            std::vector<real_t> whole(S.nnz, (real_t)0);
            for (int gx = 0; gx < 2; ++gx)
                for (int gy = 0; gy < 2; ++gy) {
                    cooMat Bk;
                    std::vector<int> rp, cp;
                    read_binary_block(dir + "/" + stem + ".bin", Bk, 2, 2, gx, gy, 4, rp, cp);
                    Bk.localizeIndices();
                    if (Bk.nnz == 0)
                        continue;
                    const std::vector<real_t> cb =
                        run_both(Bk, ramp(Bk.nrows, k, &Bk.ltgR), ramp(Bk.ncols, k, &Bk.ltgC));
                    idx_large_t at = 0;
                    for (idx_large_t e = 0; e < S.nnz; ++e)
                        if (rp[S.ii[e]] == gx && cp[S.jj[e]] == gy)
                            whole[e] = cb[at++];
                    CHECK(at == Bk.nnz);
                }
            for (idx_large_t e = 0; e < S.nnz; ++e)
                CHECK(std::fabs((double)whole[e] - (double)c[e]) <= kTol * std::fmax(std::fabs((double)c[e]), 1.0));
        }
        // a generated file of a useful size: hub rows, repeated entries, 4 x 4 mesh
        {
            const std::string big = "/tmp/spc3d_test_file_gpu.bin";
            cooMat G;
            G.gnrows = 30000;
            G.gncols = 20000;
            unsigned long long x = 0x2545F4914F6CDD1Dull;
            const idx_large_t nnz = 400000;
            for (idx_large_t i = 0; i < nnz; ++i) {
                x ^= x << 13, x ^= x >> 7, x ^= x << 17;
                const idx_t r = (x & 7) == 0 ? (idx_t)((x >> 8) % 5) : (idx_t)((x >> 8) % G.gnrows);
                G.addEntry(r, (idx_t)((x >> 32) % G.gncols), (real_t)((double)((x >> 12) % 2001) / 1000.0 - 1.0));
            }
            G.gnnz = G.nnz = nnz;
            convert_to_binary(G, big);
            idx_large_t total = 0;
            for (int gx = 0; gx < 4; gx += 3)
                for (int gy = 1; gy < 3; ++gy) {
                    cooMat Bk;
                    std::vector<int> rp, cp;
                    read_binary_block(big, Bk, 4, 4, gx, gy, 21, rp, cp);
                    Bk.localizeIndices();
                    CHECK(Bk.nnz > nnz / 32);
                    denseMatrix A, B;
                    A.m = Bk.nrows, B.m = Bk.ncols, A.n = B.n = k;
                    A.data.resize((size_t)A.m * k);
                    B.data.resize((size_t)B.m * k);
                    for (auto &v : A.data) {
                        x ^= x << 13, x ^= x >> 7, x ^= x << 17;
                        v = (real_t)((double)(x % 2001) / 1000.0 - 1.0);
                    }
                    for (auto &v : B.data) {
                        x ^= x << 13, x ^= x >> 7, x ^= x << 17;
                        v = (real_t)((double)(x % 2001) / 1000.0 - 1.0);
                    }
                    run_both(Bk, A, B);
                    total += Bk.nnz;
                }
            CHECK(total > 0);
            std::remove(big.c_str());
        }
        hip::shutdown();
    } catch (const std::exception &e) {
        std::printf("FAIL: exception: %s\n", e.what());
        ++g_fail;
    }
    std::printf("%s (%d failures, real_t = %s)\n", g_fail ? "FAILED" : "PASSED", g_fail,
                sizeof(real_t) == 8 ? "double" : "float");
    return g_fail ? 1 : 0;
}
