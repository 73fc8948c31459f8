// Tests of the C++ host shim (spcomm3d_amd/host): the reference's call surface
// over the GPU library.  Written the way the reference checks itself: the fill
// of miniapp/numCheckSeq.cpp:125-131 with its closed-form answer, the constant
// fill of miniapp/bench_both.cpp:191-192, five repeated calls, and the index
// transforms that run before the kernels.
//
//   test_shim --host   : only what needs no GPU (types, index transforms, errors)
//   test_shim          : everything
//
// The serial loops below are the test's own checker (and the C oracle is linked
// for the random cases); the library under test never sees them.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <stdexcept>
#include <string>

#include "spc3d/core_ops.hpp"
#include "spc3d/device.hpp"
#include "spc3d/distributed_comp.hpp"

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

static void oracle_sddmm(const denseMatrix &A, const denseMatrix &B, const cooMat &S,
                         std::vector<real_t> &out)
{
    out.assign(S.nnz, 0);
    int rc;
    if constexpr (sizeof(real_t) == 8)
        rc = oracle_sddmm_f64(A.m, B.m, A.n, (const double *)A.data.data(),
                              (const double *)B.data.data(), S.nnz, S.ii.data(), S.jj.data(),
                              (const double *)S.vv.data(), (double *)out.data());
    else
        rc = oracle_sddmm_f32(A.m, B.m, A.n, (const float *)A.data.data(),
                              (const float *)B.data.data(), S.nnz, S.ii.data(), S.jj.data(),
                              (const float *)S.vv.data(), (float *)out.data());
    CHECK(rc == 0);
}

static void oracle_spmm(const denseMatrix &X, const cooMat &A, std::vector<real_t> &Y, idx_t rows)
{
    int rc;
    if constexpr (sizeof(real_t) == 8)
        rc = oracle_spmm_f64(X.m, rows, X.n, (const double *)X.data.data(), A.nnz, A.ii.data(),
                             A.jj.data(), (const double *)A.vv.data(), (double *)Y.data());
    else
        rc = oracle_spmm_f32(X.m, rows, X.n, (const float *)X.data.data(), A.nnz, A.ii.data(),
                             A.jj.data(), (const float *)A.vv.data(), (float *)Y.data());
    CHECK(rc == 0);
}

static cooMat random_coo(idx_t m, idx_t n, idx_large_t nnz, unsigned seed)
{
    std::mt19937 g(seed);
    cooMat S;
    S.gnrows = S.nrows = m;
    S.gncols = S.ncols = n;
    S.nnz = S.gnnz = nnz;
    for (idx_large_t i = 0; i < nnz; ++i)
        S.addEntry(g() % m, g() % n, (real_t)((g() % 1000) / 1000.0));
    S.mtxName = "rand";
    return S;
}

static denseMatrix random_panel(idx_t m, idx_t n, unsigned seed)
{
    std::mt19937 g(seed);
    denseMatrix P;
    P.m = m;
    P.n = n;
    P.data.resize((size_t)m * n);
    for (auto &v : P.data)
        v = (real_t)((int)(g() % 2001) - 1000) / (real_t)1000;
    return P;
}

static double max_rel(const std::vector<real_t> &got, const std::vector<real_t> &ref, double scale)
{
    double e = 0;
    for (size_t i = 0; i < ref.size(); ++i)
        e = std::max(e, std::fabs((double)got[i] - (double)ref[i]) /
                            std::max(scale, std::fabs((double)ref[i])));
    return e;
}

// ---- host only ------------------------------------------------------------------
static void test_types_and_index_transforms()
{
    denseMatrix D;
    D.m = 3;
    D.n = 2;
    D.data = {0, 1, 2, 3, 4, 5};
    CHECK(D.at(2, 1) == 5 && D.at(1, 0) == 2); // row-major, src/basic.hpp:32,36
    bool threw = false;
    try {
        D.at(3, 0);
    } catch (const std::out_of_range &) {
        threw = true;
    }
    CHECK(threw);

    // localizeIndices: ids in first-appearance order of the entry stream; only
    // touched rows / columns get one (src/SparseMatrix.hpp:69-99)
    cooMat S;
    const idx_t gi[] = {70, 5, 70, 9, 5, 1000};
    const idx_t gj[] = {3, 3, 8, 1, 8, 3};
    for (int i = 0; i < 6; ++i)
        S.addEntry(gi[i], gj[i], (real_t)(i + 1));
    S.nnz = 6;
    S.localizeIndices();
    const idx_t li[] = {0, 1, 0, 2, 1, 3}, lj[] = {0, 0, 1, 2, 1, 0};
    CHECK(S.nrows == 4 && S.ncols == 3);
    for (int i = 0; i < 6; ++i)
        CHECK(S.ii[i] == li[i] && S.jj[i] == lj[i]);
    CHECK(S.ltgR[0] == 70 && S.ltgR[1] == 5 && S.ltgR[2] == 9 && S.ltgR[3] == 1000);
    CHECK(S.ltgC[0] == 3 && S.ltgC[1] == 8 && S.ltgC[2] == 1);
    // ReMapIndices (src/SparseMatrix.hpp:100-106)
    S.ReMapIndices({3, 2, 1, 0}, {2, 0, 1});
    CHECK(S.ii[0] == 3 && S.ii[3] == 1 && S.jj[0] == 2 && S.jj[2] == 0);
    cooMat Cc = S; // the benches copy S into C (miniapp/bench_both.cpp:160)
    CHECK(Cc.vv == S.vv && Cc.nnz == S.nnz);
}

static void test_random_pattern_generator()
{
    cooMat S;
    S.gnrows = 37;
    S.gncols = 11;
    S.self_generate_random(300, 5);
    CHECK(S.ii.size() == 300 && S.jj.size() == 300 && S.vv.size() == 300);
    std::vector<char> seen(37 * 11, 0);
    bool ok = true;
    for (size_t i = 0; i < 300; ++i) {
        ok = ok && S.ii[i] < 37 && S.jj[i] < 11 && S.vv[i] == (real_t)1;
        ok = ok && !seen[S.ii[i] * 11 + S.jj[i]];
        seen[S.ii[i] * 11 + S.jj[i]] = 1;
    }
    CHECK(ok); // in range, value 1, no position twice
    cooMat T;
    T.gnrows = 37;
    T.gncols = 11;
    T.self_generate_random(300, 5);
    CHECK(T.ii == S.ii && T.jj == S.jj); // same seed, same pattern
    // every cell may be asked for; one more than that may not
    cooMat U;
    U.gnrows = 2;
    U.gncols = 2;
    U.self_generate_random(4, 1);
    CHECK(U.ii.size() == 4);
    bool threw = false;
    try {
        U.self_generate_random(5, 1);
    } catch (const std::out_of_range &) {
        threw = true;
    }
    CHECK(threw);
}

static void test_errors_without_touching_the_gpu()
{
    // C.vv too short: the reference's C.vv.at(i) throws (core_ops.cpp:18)
    cooMat S = random_coo(4, 4, 8, 1), C = S;
    C.vv.resize(3);
    denseMatrix A = random_panel(4, 2, 2), B = random_panel(4, 2, 3);
    bool threw = false;
    try {
        sddmm(A, B, S, C);
    } catch (const std::out_of_range &) {
        threw = true;
    }
    CHECK(threw);
    // panel shorter than m*n
    A.data.resize(5);
    threw = false;
    try {
        cooMat C2 = S;
        sddmm(A, B, S, C2);
    } catch (const std::out_of_range &) {
        threw = true;
    }
    CHECK(threw);
    // a mesh other than 1x1x1 is refused by the wrappers
    SparseComm<real_t> pre, post;
    denseMatrix X = random_panel(4, 2, 4), Y = random_panel(4, 2, 5);
    threw = false;
    try {
        Mesh m;
        m.Z = 2;
        dist_spmm_spcomm(X, S, Y, pre, post, m);
    } catch (const std::runtime_error &) {
        threw = true;
    }
    CHECK(threw);
    // a plan that wants to talk to another rank cannot run here
    pre.outDegree = 1;
    threw = false;
    try {
        dist_spmm_spcomm(X, S, Y, pre, post, Mesh{});
    } catch (const std::runtime_error &) {
        threw = true;
    }
    CHECK(threw);
    // nnz == 0 is a no-op and needs no device
    cooMat E;
    denseMatrix Y0 = Y;
    spmm(X, E, Y);
    CHECK(Y.data == Y0.data);
}

// ---- GPU ------------------------------------------------------------------------------
static void test_numcheck_closed_form()
{
    // miniapp/numCheckSeq.cpp:125-131
    const idx_t m = 300, n = 200, k = 8;
    cooMat S = random_coo(m, n, 5000, 7), C = S;
    denseMatrix A, B;
    A.m = m; A.n = k; B.m = n; B.n = k;
    A.data.resize((size_t)m * k);
    B.data.resize((size_t)n * k);
    for (idx_t i = 0; i < m; ++i)
        for (idx_t j = 0; j < k; ++j)
            A.at(i, j) = i / (real_t)1000;
    for (idx_t i = 0; i < n; ++i)
        for (idx_t j = 0; j < k; ++j)
            B.at(i, j) = i / (real_t)1000;
    std::fill(C.vv.begin(), C.vv.end(), (real_t)-1);
    sddmm(A, B, S, C);
    double sum = 0, want = 0, err = 0;
    for (idx_large_t e = 0; e < S.nnz; ++e) {
        const double w = (double)S.vv[e] * k * ((double)S.ii[e] / 1000.0) * ((double)S.jj[e] / 1000.0);
        sum += C.vv[e];
        want += w;
        err = std::max(err, std::fabs(C.vv[e] - w) / std::max(std::fabs(w), 1e-30));
    }
    CHECK(err < (sizeof(real_t) == 8 ? 1e-12 : 2e-6));
    CHECK(std::fabs(sum - want) <= 1e-6 * std::fabs(want));
}

static void test_bench_fill_and_five_calls()
{
    // miniapp/bench_both.cpp:180-203: constant panels, C zeroed once, five calls
    const idx_t m = 500, n = 400, k = 64;
    cooMat S = random_coo(m, n, 20000, 11), C = S;
    denseMatrix A, B;
    A.m = m; A.n = k; B.m = n; B.n = k;
    A.data.assign((size_t)m * k, (real_t)3);
    B.data.assign((size_t)n * k, (real_t)3);
    std::fill(C.vv.begin(), C.vv.end(), (real_t)0);
    for (int it = 0; it < 5; ++it)
        sddmm(A, B, S, C);
    for (idx_large_t e = 0; e < S.nnz; ++e)
        CHECK(C.vv[e] == (real_t)(9 * k) * S.vv[e]); // exact: 9k is a small integer
    CHECK(hip::last_kernel_us() > 0);

    // bench_spmm.cpp:185-186: Y is not reset between the five calls
    denseMatrix X, Y;
    X.m = n; X.n = k; Y.m = m; Y.n = k;
    X.data.assign((size_t)n * k, (real_t)1);
    Y.data.assign((size_t)m * k, (real_t)0);
    for (int it = 0; it < 5; ++it)
        spmm(X, S, Y);
    std::vector<double> rowsum(m, 0.0);
    for (idx_large_t e = 0; e < S.nnz; ++e)
        rowsum[S.ii[e]] += S.vv[e];
    double err = 0;
    for (idx_t r = 0; r < m; ++r)
        for (idx_t j = 0; j < k; ++j)
            err = std::max(err, std::fabs(Y.at(r, j) - 5 * rowsum[r]) / std::max(1.0, 5 * rowsum[r]));
    CHECK(err < (sizeof(real_t) == 8 ? 1e-12 : 1e-5));
}

static void test_random_against_oracle_and_remap()
{
    const idx_t m = 700, n = 900, k = 32;
    cooMat S = random_coo(m, n, 60000, 21), C = S;
    for (idx_large_t e = 0; e < 3000; ++e)
        S.ii[e] = 17; // a long row
    denseMatrix A = random_panel(m, k, 22), B = random_panel(n, k, 23);
    std::vector<real_t> ref;
    sddmm(A, B, S, C);
    oracle_sddmm(A, B, S, ref);
    CHECK(max_rel(C.vv, ref, k * 1.0) < kTol);

    // ReMapIndices rewrites ii / jj in place at the same addresses
    // (miniapp/bench_both.cpp:200-205): the cached plan must not be reused
    std::vector<idx_t> mapR(m), mapC(n);
    for (idx_t i = 0; i < m; ++i)
        mapR[i] = m - 1 - i;
    for (idx_t j = 0; j < n; ++j)
        mapC[j] = (j * 7) % n; // 7 and 900 are coprime
    S.ReMapIndices(mapR, mapC);
    sddmm(A, B, S, C);
    oracle_sddmm(A, B, S, ref);
    CHECK(max_rel(C.vv, ref, k * 1.0) < kTol);

    // one index changed in place, the last one included (the tail of the key's last
    // 32-byte block): a new pattern again
    for (idx_large_t at : {(idx_large_t)7, S.nnz - 1}) {
        S.jj[at] = (S.jj[at] + 1) % n;
        sddmm(A, B, S, C);
        oracle_sddmm(A, B, S, ref);
        CHECK(max_rel(C.vv, ref, k * 1.0) < kTol);
    }

    // new values on the same pattern
    for (auto &v : S.vv)
        v = (real_t)1 - v;
    denseMatrix Y = random_panel(m, k, 24);
    std::vector<real_t> yref = Y.data;
    spmm(B, S, Y);
    oracle_spmm(B, S, yref, m);
    CHECK(max_rel(Y.data, yref, 3000.0) < kTol);

    // an index outside the panels: std::out_of_range, as from .at() (core_ops.cpp:16)
    S.jj[5] = n;
    bool threw = false;
    try {
        sddmm(A, B, S, C);
    } catch (const std::out_of_range &) {
        threw = true;
    }
    CHECK(threw);
}

static void test_dist_wrappers_single_rank()
{
    const idx_t m = 200, n = 150, k = 16;
    cooMat S = random_coo(m, n, 4000, 31), C = S;
    S.mtxName = C.mtxName = "r200";
    denseMatrix A = random_panel(m, k, 32), B = random_panel(n, k, 33);
    SparseComm<real_t> preA, preB;
    DComm::DenseComm post;
    setup_sddmm_reduce_single_rank(C, post);
    std::FILE *f = std::tmpfile();
    dist_set_stats_stream(f);
    std::fill(C.vv.begin(), C.vv.end(), (real_t)0);
    static_assert(sizeof(parallelTiming) == 5 * sizeof(idx_t), "the reference's layout");
    dist_sddmm_spcomm3(A, B, S, preA, preB, post, C, Mesh{});
    const distTiming tm = dist_last_timing();
    std::vector<real_t> ref;
    oracle_sddmm(A, B, S, ref);
    CHECK(max_rel(C.vv, ref, k * 1.0) < kTol);
    CHECK(C.ownedVals == C.vv); // the Z reduce-scatter over one rank
    CHECK(tm.compTimeUs > 0 && tm.pt.totalTime >= tm.pt.compTime);
    dist_sddmm_spcomm(A, B, S, preA, post, C, Mesh{});
    dist_sddmm_spcomm2(A, B, S, preA, preB, post, C, Mesh{});
    DComm::DenseComm dpre;
    dpre.OP = 0;
    dist_sddmm_dcomm(A, B, S, dpre, post, C, Mesh{});
    denseMatrix Y = random_panel(m, k, 34);
    std::vector<real_t> yref = Y.data;
    SparseComm<real_t> spre, spost;
    dist_spmm_spcomm(B, S, Y, spre, spost, Mesh{});
    oracle_spmm(B, S, yref, m);
    DComm::DenseComm dpost;
    dpost.OP = 1;
    dpost.commYflag = true;
    dist_spmm_dcomm(B, Y, S, dpre, dpost, Mesh{});
    oracle_spmm(B, S, yref, m);
    CHECK(max_rel(Y.data, yref, 100.0) < kTol);
    // the statistics lines: "mtx alg P Kloc Z 4 x avg 4 x max comm1 comm2 commcpy comp total"
    std::rewind(f);
    char line[512];
    int lines = 0;
    bool first_ok = false;
    while (std::fgets(line, sizeof line, f)) {
        if (lines == 0) {
            const char *want = "r200 sparseNB sddmm PRE 1 16 1 0.00 0.00 0.00 0.00 0 0 0 0 ";
            first_ok = std::strncmp(line, want, std::strlen(want)) == 0;
        }
        if (lines == 1) {
            char want[128];
            std::snprintf(want, sizeof want, "r200 sparseNB sddmm POST 1 16 1 1.00 %.2f 1.00 %.2f 1 %lu 1 %lu ",
                          4000.0, 4000.0, 4000ul, 4000ul);
            CHECK(std::strncmp(line, want, std::strlen(want)) == 0);
        }
        ++lines;
    }
    CHECK(first_ok);
    CHECK(lines == 12); // two lines per wrapper call
    dist_set_stats_stream(stdout);
    std::fclose(f);
}

// The resident-operand handles: SDDMM whose result feeds SpMM without leaving the
// device, a plan made from a pattern that is already there, and the pack /
// sum-unpack pair either side of a sparse exchange (src/comm.hpp:90-103,178-189),
// here sending every partial Y row back onto itself twice.
static void test_resident_handles_and_row_exchange()
{
    const idx_t m = 300, n = 257, k = 24;
    cooMat S = random_coo(m, n, 5000, 41);
    denseMatrix A = random_panel(m, k, 42), B = random_panel(n, k, 43), Y0 = random_panel(m, k, 44);
    spc3d::Context ctx(0);
    spc3d::Panel<real_t> dA(ctx, m, k), dB(ctx, n, k), dY(ctx, m, k);
    dA.upload(A.data.data());
    dB.upload(B.data.data());
    dY.upload(Y0.data.data());
    // the pattern goes up as 32-bit words and is planned where it lies
    static_assert(sizeof(float) == sizeof(idx_t), "index words travel as 32-bit values");
    spc3d::Vals<float> dii(ctx, S.nnz), djj(ctx, S.nnz);
    dii.upload(reinterpret_cast<const float *>(S.ii.data()));
    djj.upload(reinterpret_cast<const float *>(S.jj.data()));
    spc3d::Plan<real_t> P(spc3d::Plan<real_t>::FromDevice{}, ctx, m, n, S.nnz, dii.device_ptr(),
                          djj.device_ptr());
    P.set_values(S.vv.data());
    spc3d::Vals<real_t> dC(ctx, S.nnz);
    spc3d::sddmm(ctx, P, dA, dB, dC);
    std::vector<real_t> c(S.nnz), cref;
    dC.download(c.data());
    oracle_sddmm(A, B, S, cref);
    CHECK(max_rel(c, cref, k * 1.0) < kTol);
    // C becomes the sparse operand of SpMM on the device
    P.set_values(dC);
    spc3d::spmm(ctx, P, dB, dY);
    cooMat S2 = S;
    S2.vv = cref;
    std::vector<real_t> yref = Y0.data;
    oracle_spmm(B, S2, yref, m);
    std::vector<real_t> y((size_t)m * k);
    dY.download(y.data());
    CHECK(max_rel(y, yref, 100.0) < 10 * kTol);

    // the same two results from the one-pass call, chained: Y0 += C B
    {
        spc3d::Panel<real_t> dY2(ctx, m, k);
        spc3d::Vals<real_t> dC2(ctx, S.nnz);
        dY2.upload(Y0.data.data());
        P.set_values(S.vv.data());
        spc3d::sddmm_spmm(ctx, P, dA, dB, dC2, dY2, true);
        std::vector<real_t> c2(S.nnz), y2((size_t)m * k);
        dC2.download(c2.data());
        dY2.download(y2.data());
        CHECK(max_rel(c2, cref, k * 1.0) < kTol);
        CHECK(max_rel(y2, yref, 100.0) < 10 * kTol);
    }

    // pack rows (with repeats), then sum them back: Y[r] += (times r is listed) * Y[r]
    std::vector<idx_t> rows;
    for (idx_t r = 0; r < m; r += 3) {
        rows.push_back(r);
        if (r % 2 == 0)
            rows.push_back(r);
    }
    spc3d::RowMap map(ctx, m, rows.size(), rows.data());
    spc3d::Vals<real_t> buf(ctx, rows.size() * (uint64_t)k);
    spc3d::rows_pack(ctx, dY, map, buf);
    spc3d::rows_unpack_sum(ctx, dY, map, buf);
    std::vector<real_t> y2((size_t)m * k), want = y;
    dY.download(y2.data());
    for (idx_t r : rows)
        for (idx_t j = 0; j < k; ++j)
            want[(size_t)r * k + j] += y[(size_t)r * k + j]; // sequential, slot order
    CHECK(y2 == want); // copies and ordered adds: bit for bit
    bool threw = false;
    try {
        idx_t bad = m;
        spc3d::RowMap nope(ctx, m, 1, &bad);
    } catch (const std::out_of_range &) {
        threw = true;
    }
    CHECK(threw);
}

int main(int argc, char **argv)
{
    const bool host_only = argc > 1 && std::strcmp(argv[1], "--host") == 0;
    test_types_and_index_transforms();
    test_random_pattern_generator();
    test_errors_without_touching_the_gpu();
    if (!host_only) {
        try {
            test_numcheck_closed_form();
            test_bench_fill_and_five_calls();
            test_random_against_oracle_and_remap();
            test_dist_wrappers_single_rank();
            test_resident_handles_and_row_exchange();
            hip::shutdown();
        } catch (const std::exception &e) {
            std::printf("FAIL: exception: %s\n", e.what());
            ++g_fail;
        }
    }
    std::printf("%s (%d failures, real_t = %s)\n", g_fail ? "FAILED" : "PASSED", g_fail,
                sizeof(real_t) == 8 ? "double" : "float");
    return g_fail ? 1 : 0;
}
