// Times one step of the reference's distributed wrappers over device-resident operands:
// dist_sddmm_spcomm then dist_spmm_spcomm (src/distributed_comp.cpp:141-193,17-76) on one
// rank, whose exchanges are empty, over a pattern read from a .bin file
// (tools/read_convert_mm.cpp:81-94).  Per call it reports the wall-clock time of the whole
// wrapper (queueing, the one wait at its end, the statistics bookkeeping) beside the device
// time of the kernel inside it, as JSON on stdout.
//
//   dist_step <file.bin> <K> <reps>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <string>
#include <vector>

#include "spc3d/distributed_comp_device.hpp"
#include "spc3d/io.hpp"

using namespace SpKernels;

int main(int argc, char **argv)
{
    if (argc < 4) {
        std::fprintf(stderr, "usage: %s <file.bin> <K> <reps>\n", argv[0]);
        return 2;
    }
    try {
        const idx_t K = (idx_t)std::atoi(argv[2]);
        const int reps = std::atoi(argv[3]);
        cooMat S;
        read_binary(argv[1], S);
        const idx_t m = S.gnrows, n = S.gncols;
        std::mt19937 g(1);
        std::vector<real_t> hA((size_t)m * K), hB((size_t)n * K), hY((size_t)m * K);
        for (auto *v : {&hA, &hB, &hY})
            for (auto &x : *v)
                x = (real_t)((int)(g() % 2001) - 1000) / (real_t)1000;
        dist_set_stats_stream(nullptr);
        spc3d::Context ctx(0);
        spc3d::Panel<real_t> A(ctx, m, K), B(ctx, n, K), Y(ctx, m, K);
        A.upload(hA.data());
        B.upload(hB.data());
        Y.upload(hY.data());
        spc3d::Plan<real_t> P(ctx, m, n, S.nnz, S.ii.data(), S.jj.data(), S.vv.data());
        spc3d::Vals<real_t> C(ctx, S.nnz), owned(ctx, S.nnz);
        DeviceSparseComm pre(ctx, K), post(ctx, K);
        DeviceDenseComm zred;
        setup_sddmm_reduce_single_rank(C, owned, zred);
        const Mesh mesh;
        using clk = std::chrono::steady_clock;
        auto run = [&](bool sddmm_call, double &call_us, double &kernel_us, double &post_us) {
            for (int i = 0; i < 3; ++i) {
                if (sddmm_call)
                    dist_sddmm_spcomm(ctx, A, B, P, pre, zred, C, mesh, "bench");
                else
                    dist_spmm_spcomm(ctx, B, P, Y, pre, post, mesh, "bench");
            }
            double k = 0, c2 = 0;
            const auto t0 = clk::now();
            for (int i = 0; i < reps; ++i) {
                if (sddmm_call)
                    dist_sddmm_spcomm(ctx, A, B, P, pre, zred, C, mesh, "bench");
                else
                    dist_spmm_spcomm(ctx, B, P, Y, pre, post, mesh, "bench");
                k += (double)dist_last_timing().compTimeUs;
                c2 += (double)dist_last_timing().comm2TimeUs;
            }
            call_us = std::chrono::duration<double, std::micro>(clk::now() - t0).count() / reps;
            kernel_us = k / reps;
            post_us = c2 / reps;
        };
        double sc, sk, sp, pc, pk, pp;
        run(true, sc, sk, sp);
        run(false, pc, pk, pp);
        std::printf("{\"wrappers\": \"dist_sddmm_spcomm, dist_spmm_spcomm (device-resident, one rank)\", "
                    "\"real\": \"%s\", \"nnz\": %llu, \"k\": %u, \"reps\": %d, "
                    "\"sddmm_call_us\": %.1f, \"sddmm_kernel_us\": %.1f, \"sddmm_z_reduce_us\": %.1f, "
                    "\"spmm_call_us\": %.1f, \"spmm_kernel_us\": %.1f, "
                    "\"sddmm_host_overhead_us\": %.1f, \"spmm_host_overhead_us\": %.1f, "
                    "\"sddmm_call_over_device_work\": %.4f, \"spmm_call_over_device_work\": %.4f}\n",
                    sizeof(real_t) == 8 ? "f64" : "f32", (unsigned long long)S.nnz, K, reps, sc, sk,
                    sp, pc, pk, sc - sk - sp, pc - pk - pp, sc / (sk + sp), pc / (pk + pp));
    } catch (const std::exception &e) {
        std::fprintf(stderr, "dist_step: %s\n", e.what());
        return 1;
    }
    return 0;
}
