// The one-shot entry points over host memory (spc3d_sddmm_host / spc3d_spmm_host) called
// the way the reference's drivers call SpKernels::sddmm / spmm: five times over one
// pattern and the same panels (miniapp/bench_both.cpp:202-203, bench_spmm.cpp:185-186),
// with indices rewritten in place between groups of calls (:200-205).  What the context
// keeps between calls must never show in a result: every variation below changes an
// operand in the smallest way and holds the result to the CPU oracle.
//
//   test_host_calls [rows [nnz [k]]]      (defaults 300000 3000000 64)
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include "../../include/spcomm3d_hip.h"

extern "C" {
int oracle_sddmm_f64(uint32_t, uint32_t, uint32_t, const double *, const double *, uint64_t,
                     const uint32_t *, const uint32_t *, const double *, double *);
int oracle_spmm_f64(uint32_t, uint32_t, uint32_t, const double *, uint64_t, const uint32_t *,
                    const uint32_t *, const double *, double *);
}

static int g_fail = 0;
#define CHECK(cond)                                                                               \
    do {                                                                                          \
        if (!(cond)) {                                                                            \
            std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond);                           \
            ++g_fail;                                                                             \
        }                                                                                         \
    } while (0)
#define OK(call) CHECK((call) == SPC3D_OK)

using clk = std::chrono::steady_clock;
static double ms_since(clk::time_point t0)
{
    return std::chrono::duration<double, std::milli>(clk::now() - t0).count();
}

struct Problem {
    uint32_t m, n, k;
    uint64_t nnz;
    std::vector<uint32_t> ii, jj;
    std::vector<double> vv, A, B, Y;
};

static bool sddmm_matches(const Problem &p, const std::vector<double> &c)
{
    std::vector<double> ref(p.nnz);
    if (oracle_sddmm_f64(p.m, p.n, p.k, p.A.data(), p.B.data(), p.nnz, p.ii.data(), p.jj.data(),
                         p.vv.data(), ref.data()) != 0)
        return false;
    for (uint64_t e = 0; e < p.nnz; ++e)
        if (std::fabs(c[e] - ref[e]) > 1e-12 * std::fmax(std::fabs(ref[e]), (double)p.k))
            return false;
    return true;
}

int main(int argc, char **argv)
{
    Problem p;
    p.m = p.n = argc > 1 ? (uint32_t)std::atoi(argv[1]) : 300000u; // square: A and B share a shape
    p.nnz = argc > 2 ? (uint64_t)std::atoll(argv[2]) : 3000000ull;
    p.k = argc > 3 ? (uint32_t)std::atoi(argv[3]) : 64u;
    std::mt19937_64 g(99);
    p.ii.resize(p.nnz), p.jj.resize(p.nnz), p.vv.resize(p.nnz);
    for (uint64_t e = 0; e < p.nnz; ++e) {
        p.ii[e] = (uint32_t)(g() % 16 == 0 ? g() % 8 : g() % p.m); // a few hub rows
        p.jj[e] = (uint32_t)(g() % p.n);
        p.vv[e] = (double)(g() % 2001) / 1000.0 - 1.0;
    }
    auto fill = [&](std::vector<double> &v, size_t count) {
        v.resize(count);
        for (auto &x : v)
            x = (double)(g() % 2001) / 1000.0 - 1.0;
    };
    fill(p.A, (size_t)p.m * p.k);
    fill(p.B, (size_t)p.n * p.k);
    fill(p.Y, (size_t)p.m * p.k);
    const uint64_t panel_bytes = (uint64_t)p.m * p.k * 8, val_bytes = p.nnz * 8;

    spc3d_ctx *ctx = nullptr;
    if (spc3d_ctx_create(0, &ctx) != SPC3D_OK) {
        std::printf("FAIL: no context: %s\n", spc3d_last_error());
        return 1;
    }
    std::vector<double> c(p.nnz), c1;
    uint64_t sent = 0, kept = 0;
    int reused = -1;
    auto sddmm = [&]() {
        const auto t0 = clk::now();
        OK(spc3d_sddmm_host(ctx, SPC3D_F64, p.m, p.n, p.k, p.A.data(), p.B.data(), p.nnz,
                            p.ii.data(), p.jj.data(), p.vv.data(), c.data()));
        const double ms = ms_since(t0);
        OK(spc3d_host_call_stats(ctx, &sent, &kept, &reused));
        return ms;
    };

    // ---- five identical calls ---------------------------------------------------------
    double first = sddmm(), later = 0;
    CHECK(reused == 0 && kept == 0 && sent >= 2 * panel_bytes + val_bytes);
    CHECK(sddmm_matches(p, c));
    c1 = c;
    for (int rep = 1; rep < 5; ++rep) {
        std::fill(c.begin(), c.end(), -1.0);
        later += sddmm() / 4;
        CHECK(reused == 1 && kept == 2 * panel_bytes && sent == val_bytes);
        CHECK(c == c1); // the same plan over the same operands: the same bits
    }
    float kernel_ms = 0;
    OK(spc3d_timer_elapsed_ms(ctx, SPC3D_TIMER_HOST_CALL_BEGIN, SPC3D_TIMER_HOST_CALL_END, &kernel_ms));
    std::printf("TIMING sddmm_host m=n=%u nnz=%llu k=%u: first call %.1f ms, calls 2..5 %.1f ms each "
                "(kernel %.3f ms; %.0f MB of panels left in place, %.0f MB of values sent, %.0f MB of "
                "results fetched)\n",
                p.m, (unsigned long long)p.nnz, p.k, first, later, kernel_ms, 2 * panel_bytes / 1e6,
                val_bytes / 1e6, val_bytes / 1e6);

    // ---- one element of A changes: one block goes up, the result follows ----------------
    p.A[(size_t)p.ii[5] * p.k + 3] += 0.5;
    sddmm();
    CHECK(reused == 1 && sent <= val_bytes + ((uint64_t)4 << 20) && sent > val_bytes);
    CHECK(c != c1 && sddmm_matches(p, c));
    // the last element of B (a short last block)
    p.B.back() = -p.B.back() + 0.125;
    sddmm();
    CHECK(reused == 1 && sent <= val_bytes + ((uint64_t)4 << 20) && sent > val_bytes);
    CHECK(sddmm_matches(p, c));
    // A and B trade places (same shape, same addresses, other content)
    p.A.swap(p.B); // the vectors trade buffers: each content now sits at the other's address
    sddmm();
    CHECK(reused == 1 && kept == 2 * panel_bytes); // found by content, wherever it lies
    CHECK(sddmm_matches(p, c));
    std::vector<double> tmp = p.A; // now the contents move and the addresses stay
    std::memcpy(p.A.data(), p.B.data(), panel_bytes);
    std::memcpy(p.B.data(), tmp.data(), panel_bytes);
    sddmm();
    CHECK(reused == 1 && kept == 2 * panel_bytes);
    CHECK(sddmm_matches(p, c));

    // ---- two panels used in turn for one operand: both stay ----------------------------
    {
        std::vector<double> other(p.A.size());
        for (auto &x : other)
            x = (double)(g() % 2001) / 1000.0 - 1.0;
        p.A.swap(other);
        sddmm();
        CHECK(reused == 1 && kept == panel_bytes && sent == val_bytes + panel_bytes); // B stays, the new A goes up
        CHECK(sddmm_matches(p, c));
        p.A.swap(other);
        sddmm();
        CHECK(kept == 2 * panel_bytes && sddmm_matches(p, c)); // the first A was not pushed out
        p.A.swap(other);
        sddmm();
        CHECK(kept == 2 * panel_bytes && sddmm_matches(p, c)); // nor the second
        p.A.swap(other);
    }

    // ---- values change: always sent ---------------------------------------------------
    p.vv[p.nnz / 2] = 7.25;
    sddmm();
    CHECK(reused == 1 && sddmm_matches(p, c));

    // ---- one index changes, in place: a new plan ----------------------------------------
    const uint32_t old_j = p.jj[p.nnz - 1];
    p.jj[p.nnz - 1] = (old_j + 1) % p.n;
    sddmm();
    CHECK(reused == 0 && kept == 2 * panel_bytes && sddmm_matches(p, c));
    // two entries trade their rows (the sum of the words stays, their places do not)
    std::swap(p.ii[10], p.ii[11 + 4 * 1024]);
    sddmm();
    CHECK(reused == 0 && sddmm_matches(p, c));
    std::swap(p.ii[10], p.ii[11 + 4 * 1024]);
    p.jj[p.nnz - 1] = old_j; // back to the first pattern: its plan is still kept
    sddmm();
    CHECK(reused == 1 && sddmm_matches(p, c));
    // a bad index is reported as always, and nothing stale answers for it
    p.ii[7] = p.m;
    CHECK(spc3d_sddmm_host(ctx, SPC3D_F64, p.m, p.n, p.k, p.A.data(), p.B.data(), p.nnz, p.ii.data(),
                           p.jj.data(), p.vv.data(), c.data()) == SPC3D_ERR_BAD_INDEX);
    p.ii[7] = 0;
    sddmm();
    CHECK(sddmm_matches(p, c));

    // ---- the index maps of a driver: rewritten in place, run, mapped back ----------------
    {
        std::vector<uint32_t> mapR(p.m), mapC(p.n), invR(p.m), invC(p.n);
        for (uint32_t i = 0; i < p.m; ++i)
            mapR[i] = (uint32_t)(((uint64_t)i * 7919u + 13u) % p.m);
        for (uint32_t i = 0; i < p.n; ++i)
            mapC[i] = (uint32_t)(((uint64_t)i * 104729u + 5u) % p.n);
        bool bijection = true;
        std::vector<char> hit(p.m, 0);
        for (uint32_t i = 0; i < p.m; ++i) {
            if (hit[mapR[i]])
                bijection = false;
            hit[mapR[i]] = 1;
            invR[mapR[i]] = i;
        }
        for (uint32_t i = 0; i < p.n; ++i)
            invC[mapC[i]] = i;
        if (bijection) {
            for (uint64_t e = 0; e < p.nnz; ++e)
                p.ii[e] = mapR[p.ii[e]], p.jj[e] = mapC[p.jj[e]];
            sddmm();
            CHECK(reused == 0 && sddmm_matches(p, c));
            sddmm();
            CHECK(reused == 1);
            for (uint64_t e = 0; e < p.nnz; ++e)
                p.ii[e] = invR[p.ii[e]], p.jj[e] = invC[p.jj[e]];
            sddmm();
            CHECK(reused == 1 && sddmm_matches(p, c)); // the pattern from before the maps
        }
    }

    // ---- SpMM: X kept; Y accumulates over the calls and goes up again only where the caller
    //      touched it since the last result came back ------------------------------------------
    {
        std::vector<double> y_ref = p.Y;
        double t_first = 0, t_later = 0;
        auto spmm = [&]() {
            const auto t0 = clk::now();
            OK(spc3d_spmm_host(ctx, SPC3D_F64, p.n, p.m, p.k, p.B.data(), p.nnz, p.ii.data(),
                               p.jj.data(), p.vv.data(), p.Y.data()));
            const double ms = ms_since(t0);
            OK(spc3d_host_call_stats(ctx, &sent, &kept, &reused));
            CHECK(oracle_spmm_f64(p.n, p.m, p.k, p.B.data(), p.nnz, p.ii.data(), p.jj.data(),
                                  p.vv.data(), y_ref.data()) == 0);
            return ms;
        };
        auto y_matches = [&]() {
            double worst = 0;
            for (size_t i = 0; i < y_ref.size(); ++i)
                worst = std::fmax(worst, std::fabs(p.Y[i] - y_ref[i]) / std::fmax(std::fabs(y_ref[i]), 100.0));
            return worst < 1e-12;
        };
        for (int rep = 0; rep < 5; ++rep) {
            (rep ? t_later : t_first) += spmm() / (rep ? 4 : 1);
            CHECK(reused == 1); // the SDDMM calls planned this pattern at this k
            if (rep == 0)       // X is SDDMM's B, already there; Y goes up whole the first time
                CHECK(kept == panel_bytes && sent == val_bytes + panel_bytes);
            else                // then the result that came back is what the device holds
                CHECK(kept == 2 * panel_bytes && sent == val_bytes);
        }
        CHECK(y_matches());
        std::printf("TIMING spmm_host: first call %.1f ms, calls 2..5 %.1f ms each\n", t_first, t_later);
        // one element of Y changes on the host: its block goes up, the rest stays
        p.Y[p.Y.size() / 2] += 3.0;
        y_ref[p.Y.size() / 2] += 3.0;
        spmm();
        CHECK(sent > val_bytes && sent <= val_bytes + ((uint64_t)4 << 20) && y_matches());
        // the caller rewrites all of Y before every call: the first time it is read in vain,
        // then it goes up unread for a stretch, and the results are right throughout
        for (int rep = 0; rep < 5; ++rep) {
            for (size_t i = 0; i < p.Y.size(); ++i)
                p.Y[i] = y_ref[i] = 0.5 + (double)((i + rep) % 7);
            spmm();
            CHECK(sent == val_bytes + panel_bytes && kept == panel_bytes && y_matches());
        }
        // and a Y left alone again is found again (after the stretch has run out)
        for (int rep = 0; rep < 4; ++rep)
            spmm();
        CHECK(kept == 2 * panel_bytes && sent == val_bytes && y_matches());
        // the result of one call as the dense operand of the next: found by content
        {
            std::vector<double> x2 = p.Y, y2((size_t)p.m * p.k, 0.0), y2_ref = y2;
            OK(spc3d_spmm_host(ctx, SPC3D_F64, p.n, p.m, p.k, x2.data(), p.nnz, p.ii.data(),
                               p.jj.data(), p.vv.data(), y2.data()));
            OK(spc3d_host_call_stats(ctx, &sent, &kept, &reused));
            CHECK(kept >= panel_bytes); // x2 is a copy of the Y that was just fetched
            CHECK(oracle_spmm_f64(p.n, p.m, p.k, x2.data(), p.nnz, p.ii.data(), p.jj.data(),
                                  p.vv.data(), y2_ref.data()) == 0);
            double worst = 0;
            for (size_t i = 0; i < y2.size(); ++i)
                worst = std::fmax(worst, std::fabs(y2[i] - y2_ref[i]) / std::fmax(std::fabs(y2_ref[i]), 1e4));
            CHECK(worst < 1e-12);
        }
        // SDDMM still finds A and B after SpMM used panels for Y
        sddmm();
        CHECK(reused == 1 && sddmm_matches(p, c));
    }

    // ---- dropping what is kept changes nothing but the work ------------------------------
    OK(spc3d_host_cache_clear(ctx));
    sddmm();
    CHECK(reused == 0 && kept == 0 && sddmm_matches(p, c));
    OK(spc3d_ctx_destroy(ctx));
    std::printf("%s (%d failures)\n", g_fail ? "FAILED" : "PASSED", g_fail);
    return g_fail ? 1 : 0;
}
