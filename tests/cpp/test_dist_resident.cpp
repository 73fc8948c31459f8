// The six distributed wrappers over device-resident operands
// (spc3d/distributed_comp_device.hpp) against the same wrappers over host memory
// (spc3d/distributed_comp.hpp) and against the CPU oracle, on one GPU.
//
// The exchanges carry messages the rank addresses to itself, so that the copies either
// side of an exchange run (on the device: spc3d_rows_pack / _unpack / _unpack_sum; on the
// host: the loops of src/comm.hpp:90-103,166-189): rows of the dense operand are packed,
// "sent", and unpacked over other rows before the kernel, and for SpMM a receive buffer is
// summed into rows of Y after it.  The reference's slip at src/distributed_comp.cpp:59
// (the post phase unpacks comm_pre again instead of packing comm_post) is part of what both
// forms must reproduce: comm_post's send buffer goes out as it was set up.
//
// Every result of the resident form must equal the host-memory form's bit for bit (same
// kernels, exact copies), and both are held to the oracle run over operands that went
// through the same row copies on the CPU.
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <numeric>
#include <random>
#include <string>
#include <vector>

#include "spc3d/core_ops.hpp"
#include "spc3d/distributed_comp_device.hpp"

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

static cooMat random_coo(idx_t m, idx_t n, idx_large_t nnz, unsigned seed, idx_t hub)
{
    std::mt19937 g(seed);
    cooMat S;
    S.gnrows = S.nrows = m;
    S.gncols = S.ncols = n;
    S.nnz = S.gnnz = nnz;
    for (idx_large_t i = 0; i < nnz; ++i)
        S.addEntry(i < hub ? m / 3 : g() % m, g() % n, (real_t)((g() % 1000) / 1000.0));
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

// A self-addressed exchange over rows of M: nsend rows (distinct) are packed and arrive in
// nrecv = nsend receive slots that go to other rows, some of them twice (two messages).
struct Rows {
    std::vector<idx_t> send, recv;
};
static Rows pick_rows(idx_t m, idx_t n, unsigned seed)
{
    std::mt19937 g(seed);
    std::vector<idx_t> all(m);
    std::iota(all.begin(), all.end(), 0);
    std::shuffle(all.begin(), all.end(), g);
    Rows r;
    r.send.assign(all.begin(), all.begin() + n);
    r.recv.assign(all.begin() + n, all.begin() + 2 * n); // disjoint from the senders
    for (idx_t i = 0; i + 1 < n; i += 7)
        r.recv[i + 1] = r.recv[i]; // a row that receives two slots
    return r;
}
static void host_plan(SparseComm<real_t> &c, denseMatrix &from, denseMatrix &into, const Rows &r)
{
    const idx_t K = c.dataUnitSize;
    const int n = (int)r.send.size(), half = n / 2;
    c.inDegree = c.outDegree = 2; // two messages to oneself
    c.inSet = c.outSet = {0, 0};
    c.sendCount = c.recvCount = {(int)(half * K), (int)((n - half) * K)};
    c.sendDisp = c.recvDisp = {0, (int)(half * K), (int)(n * K)};
    c.sendBuff.assign((size_t)n * K, 0);
    c.recvBuff.assign((size_t)n * K, 0);
    c.sendptr.clear();
    c.recvptr.clear();
    for (idx_t row : r.send)
        c.sendptr.push_back(&from.at(row, 0));
    for (idx_t row : r.recv)
        c.recvptr.push_back(&into.at(row, 0));
}

static void spmm_case(spc3d::Context &ctx, idx_t m, idx_t n, idx_t K, idx_large_t nnz, unsigned seed)
{
    cooMat A = random_coo(m, n, nnz, seed, (idx_t)(nnz / 5));
    denseMatrix X = random_panel(n, K, seed + 1), Y = random_panel(m, K, seed + 2);
    const denseMatrix X0 = X, Y0 = Y;
    const Rows rx = pick_rows(n, n / 4, seed + 3), ry = pick_rows(m, m / 5, seed + 4);
    // the post exchange's send buffer is never packed (src/distributed_comp.cpp:59): it goes
    // out as it was set up
    std::vector<real_t> post_send = random_panel((idx_t)ry.send.size(), K, seed + 5).data;

    // ---- host memory ----
    SparseComm<real_t> pre(K), post(K);
    host_plan(pre, X, X, rx);
    host_plan(post, Y, Y, ry);
    post.sendBuff = post_send;
    dist_spmm_spcomm(X, A, Y, pre, post, Mesh{});

    // ---- resident ----
    spc3d::Panel<real_t> dX(ctx, n, K), dY(ctx, m, K);
    dX.upload(X0.data.data());
    dY.upload(Y0.data.data());
    spc3d::Plan<real_t> dA(ctx, m, n, A.nnz, A.ii.data(), A.jj.data(), A.vv.data());
    denseMatrix X1 = X0, Y1 = Y0; // what the pointers of the host plans below point into
    SparseComm<real_t> hpre(K), hpost(K);
    host_plan(hpre, X1, X1, rx);
    host_plan(hpost, Y1, Y1, ry);
    DeviceSparseComm dpre(ctx, K), dpost(ctx, K);
    dpre.adopt(hpre, X1, &dX, X1, &dX);
    dpost.adopt(hpost, Y1, &dY, Y1, &dY);
    dpost.sendBuff->upload(post_send.data());
    dist_spmm_spcomm(ctx, dX, dA, dY, dpre, dpost, Mesh{}, A.mtxName);
    const distTiming t = dist_last_timing();
    std::vector<real_t> gX(X.data.size()), gY(Y.data.size());
    dX.download(gX.data());
    dY.download(gY.data());
    CHECK(gX == X.data); // bit for bit
    CHECK(gY == Y.data);
    CHECK(t.compTimeUs > 0 && t.totalTimeUs >= t.compTimeUs + t.comm1TimeUs);
    CHECK(t.commcpyTimeUs > 0 && t.commcpyTimeUs <= t.comm1TimeUs + t.comm2TimeUs);

    // ---- oracle over the same copies ----
    denseMatrix Xe = X0;
    for (size_t i = 0; i < rx.recv.size(); ++i) // expand: slot i = row send[i], lands in row recv[i]
        for (idx_t j = 0; j < K; ++j)
            Xe.at(rx.recv[i], j) = X0.at(rx.send[i], j);
    CHECK(Xe.data == X.data);
    std::vector<real_t> Ye = Y0.data;
    int rc;
    if constexpr (sizeof(real_t) == 8)
        rc = oracle_spmm_f64(n, m, K, (const double *)Xe.data.data(), A.nnz, A.ii.data(), A.jj.data(),
                             (const double *)A.vv.data(), (double *)Ye.data());
    else
        rc = oracle_spmm_f32(n, m, K, (const float *)Xe.data.data(), A.nnz, A.ii.data(), A.jj.data(),
                             (const float *)A.vv.data(), (float *)Ye.data());
    CHECK(rc == 0);
    // post: the :59 slip unpacks comm_pre's receive buffer over X once more (no change), then
    // the unpacked send buffer is summed into the rows of Y
    for (size_t i = 0; i < ry.recv.size(); ++i)
        for (idx_t j = 0; j < K; ++j)
            Ye[(size_t)ry.recv[i] * K + j] += post_send[i * K + j];
    CHECK(max_rel(Y.data, Ye, 1.0) <= kTol * 50);
}

static void sddmm_case(spc3d::Context &ctx, idx_t m, idx_t n, idx_t K, idx_large_t nnz, unsigned seed)
{
    cooMat S = random_coo(m, n, nnz, seed, (idx_t)(nnz / 5)), C = S;
    denseMatrix A = random_panel(m, K, seed + 1), B = random_panel(n, K, seed + 2);
    const denseMatrix A0 = A;
    const Rows ra = pick_rows(m, m / 4, seed + 3);
    std::fill(C.vv.begin(), C.vv.end(), (real_t)-7);

    SparseComm<real_t> pre(K);
    host_plan(pre, A, A, ra);
    DComm::DenseComm post;
    setup_sddmm_reduce_single_rank(C, post);
    dist_sddmm_spcomm(A, B, S, pre, post, C, Mesh{});

    spc3d::Panel<real_t> dA(ctx, m, K), dB(ctx, n, K);
    dA.upload(A0.data.data());
    dB.upload(B.data.data());
    spc3d::Plan<real_t> dS(ctx, m, n, S.nnz, S.ii.data(), S.jj.data(), S.vv.data());
    spc3d::Vals<real_t> dC(ctx, S.nnz), dOwned(ctx, S.nnz);
    dC.fill(-7);
    dOwned.fill(0);
    denseMatrix A1 = A0;
    SparseComm<real_t> hpre(K);
    host_plan(hpre, A1, A1, ra);
    DeviceSparseComm dpre(ctx, K);
    dpre.adopt(hpre, A1, &dA, A1, &dA);
    DeviceDenseComm dpost;
    setup_sddmm_reduce_single_rank(dC, dOwned, dpost);
    dist_sddmm_spcomm(ctx, dA, dB, dS, dpre, dpost, dC, Mesh{}, S.mtxName);
    std::vector<real_t> gC(S.nnz), gO(S.nnz), gA(A.data.size());
    dC.download(gC.data());
    dOwned.download(gO.data());
    dA.download(gA.data());
    CHECK(gA == A.data);
    CHECK(gC == C.vv);        // bit for bit
    CHECK(gO == C.ownedVals); // the Z reduction over one rank
    CHECK(gO == gC);

    denseMatrix Ae = A0;
    for (size_t i = 0; i < ra.recv.size(); ++i)
        for (idx_t j = 0; j < K; ++j)
            Ae.at(ra.recv[i], j) = A0.at(ra.send[i], j);
    std::vector<real_t> want(S.nnz);
    int rc;
    if constexpr (sizeof(real_t) == 8)
        rc = oracle_sddmm_f64(m, n, K, (const double *)Ae.data.data(), (const double *)B.data.data(),
                              S.nnz, S.ii.data(), S.jj.data(), (const double *)S.vv.data(),
                              (double *)want.data());
    else
        rc = oracle_sddmm_f32(m, n, K, (const float *)Ae.data.data(), (const float *)B.data.data(),
                              S.nnz, S.ii.data(), S.jj.data(), (const float *)S.vv.data(),
                              (float *)want.data());
    CHECK(rc == 0);
    CHECK(max_rel(C.vv, want, (double)K) <= kTol);

    // the other four wrappers: dense pre phases and empty two-sided expands change nothing,
    // and every one of them leaves the host form's bits
    auto same = [&](const char *what) {
        dC.download(gC.data());
        dOwned.download(gO.data());
        if (!(gC == C.vv && gO == C.ownedVals)) {
            std::printf("FAIL resident %s differs from its host form\n", what);
            ++g_fail;
        }
    };
    SparseComm<real_t> e1(K), e2(K);
    DeviceSparseComm d1(ctx, K), d2(ctx, K);
    DComm::DenseComm hdpre;
    DeviceDenseComm ddpre;
    dist_sddmm_spcomm2(A, B, S, e1, e2, post, C, Mesh{});
    dist_sddmm_spcomm2(ctx, dA, dB, dS, d1, d2, dpost, dC, Mesh{}, S.mtxName);
    same("dist_sddmm_spcomm2");
    dist_sddmm_spcomm3(A, B, S, e1, e2, post, C, Mesh{});
    dist_sddmm_spcomm3(ctx, dA, dB, dS, d1, d2, dpost, dC, Mesh{}, S.mtxName);
    same("dist_sddmm_spcomm3");
    dist_sddmm_dcomm(A, B, S, hdpre, post, C, Mesh{});
    dist_sddmm_dcomm(ctx, dA, dB, dS, ddpre, dpost, dC, Mesh{}, S.mtxName);
    same("dist_sddmm_dcomm");
    denseMatrix Y = random_panel(m, K, seed + 9);
    spc3d::Panel<real_t> dY(ctx, m, K);
    dY.upload(Y.data.data());
    DComm::DenseComm hpost2;
    DeviceDenseComm dpost2;
    dist_spmm_dcomm(B, Y, S, hdpre, hpost2, Mesh{});
    dist_spmm_dcomm(ctx, dB, dY, dS, ddpre, dpost2, Mesh{}, S.mtxName);
    std::vector<real_t> gY(Y.data.size());
    dY.download(gY.data());
    CHECK(gY == Y.data);

    // refusals: another mesh, a peer that is not this rank
    bool threw = false;
    try {
        Mesh bad;
        bad.X = 2;
        dist_sddmm_dcomm(ctx, dA, dB, dS, ddpre, dpost, dC, bad, "x");
    } catch (const std::runtime_error &) {
        threw = true;
    }
    CHECK(threw);
    d1.inDegree = d1.outDegree = 1;
    d1.inSet = d1.outSet = {1};
    threw = false;
    try {
        dist_sddmm_spcomm2(ctx, dA, dB, dS, d1, d2, dpost, dC, Mesh{}, "x");
    } catch (const std::runtime_error &) {
        threw = true;
    }
    CHECK(threw);
}

int main()
{
    dist_set_stats_stream(nullptr);
    try {
        spc3d::Context ctx(0);
        spmm_case(ctx, 900, 700, 16, 20000, 11);
        spmm_case(ctx, 5000, 4000, 64, 300000, 12);
        sddmm_case(ctx, 900, 700, 16, 20000, 21);
        sddmm_case(ctx, 5000, 4000, 64, 300000, 22);
        // the statistics lines: the resident form prints what the host form prints but for the
        // times (volumes: two self-addressed messages, their reals)
        std::FILE *f = std::tmpfile();
        dist_set_stats_stream(f);
        spmm_case(ctx, 300, 200, 8, 3000, 31);
        dist_set_stats_stream(nullptr);
        std::rewind(f);
        char line[512];
        std::vector<std::string> lines;
        while (std::fgets(line, sizeof line, f))
            lines.push_back(line);
        std::fclose(f);
        CHECK(lines.size() == 4); // PRE + POST of the host form, PRE + POST of the resident form
        auto head = [](const std::string &s) { // everything before the five times
            size_t pos = s.size();
            for (int k = 0; k < 5; ++k)
                pos = s.find_last_of(' ', pos - 1);
            return s.substr(0, pos);
        };
        if (lines.size() == 4) {
            CHECK(head(lines[0]) == head(lines[2]));
            CHECK(head(lines[1]) == head(lines[3]));
            CHECK(lines[0].rfind("rand sparse spmm PRE 1 8 1 2.00 400.00 2.00 400.00 2 400 2 400", 0) == 0);
        }
    } catch (const std::exception &e) {
        std::printf("FAIL exception: %s\n", e.what());
        ++g_fail;
    }
    SpKernels::hip::shutdown();
    std::printf(g_fail ? "FAILED (%d)\n" : "PASSED\n", g_fail);
    return g_fail != 0;
}
