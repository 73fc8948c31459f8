// Times one step of the reference's distributed wrappers over device-resident operands:
// dist_sddmm_spcomm then dist_spmm_spcomm (src/distributed_comp.cpp:141-193,17-76) on one
// rank, whose exchanges are empty, over a pattern read from a .bin file
// (tools/read_convert_mm.cpp:81-94).  Per call it reports the wall-clock time of the whole
// wrapper (queueing, the one wait at its end, the statistics bookkeeping) beside the device
// time of the kernel inside it, as JSON on stdout.
//
//   dist_step <file.bin> <K> <reps>
#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <memory>
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
        // The reference's loop around its kernels on resident operands (miniapp/bench_both.cpp:
        // 196-205): ReMapIndices over the pattern, NUM_ITER = 5 calls of the wrapper over the
        // remapped pattern, ReMapIndices back.  The pattern lives on the device; the plan is made
        // from it there after the remap (a plan is tied to the indices it was made from).
        double loop_us = 0, loop_plan_us = 0, loop_calls_us = 0;
        {
            std::vector<idx_t> mapA(m), mapB(n), mapAI(m), mapBI(n);
            for (idx_t i = 0; i < m; ++i) mapA[i] = i;
            for (idx_t i = 0; i < n; ++i) mapB[i] = i;
            std::shuffle(mapA.begin(), mapA.end(), g);
            std::shuffle(mapB.begin(), mapB.end(), g);
            for (idx_t i = 0; i < m; ++i) mapAI[mapA[i]] = i;
            for (idx_t i = 0; i < n; ++i) mapBI[mapB[i]] = i;
            // 32-bit words on the device: index arrays and maps travel as value vectors of floats
            auto words = [&](const std::vector<idx_t> &v) {
                auto *d = new spc3d::Vals<float>(ctx, v.size());
                d->upload(reinterpret_cast<const float *>(v.data()));
                return std::unique_ptr<spc3d::Vals<float>>(d);
            };
            auto dii = words(S.ii), djj = words(S.jj), dA = words(mapA), dB = words(mapB),
                 dAI = words(mapAI), dBI = words(mapBI);
            spc3d::Vals<real_t> vv(ctx, S.nnz);
            vv.upload(S.vv.data());
            auto remap = [&](spc3d::Vals<float> &idx, spc3d::Vals<float> &map, idx_t len) {
                spc3d::check(spc3d_remap_device(ctx.get(), S.nnz, idx.device_ptr(), map.device_ptr(), len),
                             "spc3d_remap_device");
            };
            const int loops = 3;
            for (int it = 0; it < loops + 1; ++it) { // the first pass warms up
                ctx.sync();
                const auto t0 = clk::now();
                remap(*dii, *dA, m);
                remap(*djj, *dB, n);
                const auto t1 = clk::now();
                spc3d::Plan<real_t> Q(spc3d::Plan<real_t>::FromDevice{}, ctx, m, n, S.nnz,
                                      dii->device_ptr(), djj->device_ptr());
                Q.set_values(vv);
                ctx.sync();
                const auto t2 = clk::now();
                for (int i = 0; i < 5; ++i)
                    dist_sddmm_spcomm(ctx, A, B, Q, pre, zred, C, mesh, "bench");
                const auto t3 = clk::now();
                remap(*dii, *dAI, m);
                remap(*djj, *dBI, n);
                ctx.sync();
                const auto t4 = clk::now();
                if (it == 0)
                    continue;
                loop_us += std::chrono::duration<double, std::micro>(t4 - t0).count() / loops;
                loop_plan_us += std::chrono::duration<double, std::micro>(t2 - t1).count() / loops;
                loop_calls_us += std::chrono::duration<double, std::micro>(t3 - t2).count() / loops;
            }
        }
        std::printf("{\"reference_loop\": {\"what\": \"ReMapIndices, plan from the device, 5 x "
                    "dist_sddmm_spcomm, ReMapIndices back; all operands resident "
                    "(miniapp/bench_both.cpp:196-205)\", \"total_us\": %.1f, \"plan_us\": %.1f, "
                    "\"five_calls_us\": %.1f, \"remaps_us\": %.1f}, ",
                    loop_us, loop_plan_us, loop_calls_us, loop_us - loop_plan_us - loop_calls_us);
        std::printf("\"wrappers\": \"dist_sddmm_spcomm, dist_spmm_spcomm (device-resident, one rank)\", "
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
