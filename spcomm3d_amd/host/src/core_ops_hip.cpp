// SpKernels::sddmm / SpKernels::spmm over host vectors, executed on the GPU.
// Replaces the reference's src/core_ops.cpp at link time (same two symbols,
// src/core_ops.hpp:9-12).  See spc3d/core_ops.hpp for the contract.
#include "spc3d/core_ops.hpp"

#include <cstring>
#if defined(__x86_64__)
#include <nmmintrin.h>
#endif
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "spc3d/device.hpp"

namespace SpKernels {
namespace {

using spc3d::Context;
using spc3d::Panel;
using spc3d::Plan;
using spc3d::Vals;

// 128-bit key of a pattern: every byte of ii and jj goes in (ReMapIndices rewrites
// them in place, at the same addresses, and the cached plan must not survive that).
// Four interleaved CRC-32C streams run at the speed one core reads memory (128 MiB
// in 18 ms where a multiply-xorshift chain over 8-byte words took 45 ms); without
// SSE 4.2 the chain is the fallback.
struct PatternKey {
    uint64_t a = 0, b = 0;
    bool operator==(const PatternKey &o) const { return a == o.a && b == o.b; }
};

void mix_words(const void *data, size_t bytes, uint64_t (&h)[4])
{
    const unsigned char *p = static_cast<const unsigned char *>(data);
    size_t i = 0;
    for (; i + 32 <= bytes; i += 32) {
        uint64_t w[4];
        std::memcpy(w, p + i, 32);
        for (int l = 0; l < 4; ++l) {
            h[l] = (h[l] ^ w[l]) * 0xBF58476D1CE4E5B9ull;
            h[l] ^= h[l] >> 29;
        }
    }
    uint64_t tail[4] = {0, 0, 0, 0};
    std::memcpy(tail, p + i, bytes - i);
    for (int l = 0; l < 4; ++l)
        h[l] = (h[l] ^ tail[l]) * 0x94D049BB133111EBull;
}

#if defined(__x86_64__)
__attribute__((target("sse4.2"))) void crc_words(const void *data, size_t bytes, uint64_t (&h)[4])
{
    const unsigned char *p = static_cast<const unsigned char *>(data);
    size_t i = 0;
    for (; i + 32 <= bytes; i += 32) {
        uint64_t w[4];
        std::memcpy(w, p + i, 32);
        for (int l = 0; l < 4; ++l)
            h[l] = _mm_crc32_u64(h[l], w[l]);
    }
    uint64_t tail[4] = {0, 0, 0, 0};
    std::memcpy(tail, p + i, bytes - i);
    for (int l = 0; l < 4; ++l)
        h[l] = _mm_crc32_u64(h[l], tail[l]);
}
#endif

PatternKey pattern_key(const idx_t *ii, const idx_t *jj, uint64_t nnz)
{
    uint64_t h[4] = {nnz, ~nnz, 0x9E3779B97F4A7C15ull, 0xD6E8FEB86659FD93ull};
#if defined(__x86_64__)
    static const bool crc = __builtin_cpu_supports("sse4.2");
    if (crc) {
        crc_words(ii, nnz * sizeof(idx_t), h);
        static const uint64_t boundary[4] = {0x1F3D5B79u, 0x2E4C6A80u, 0x3D5B798Fu, 0x4C6A809Eu};
        crc_words(boundary, sizeof boundary, h); // ii | jj
        crc_words(jj, nnz * sizeof(idx_t), h);
        return {h[0] | (h[1] << 32), h[2] | (h[3] << 32)};
    }
#endif
    mix_words(ii, nnz * sizeof(idx_t), h);
    mix_words(jj, nnz * sizeof(idx_t), h);
    return {h[0] ^ (h[1] >> 31), h[2] ^ (h[3] >> 31)};
}

struct CachedPlan {
    PatternKey pattern;
    uint64_t nnz = 0;
    uint32_t nrows = 0, ncols = 0, k = 0;
    uint64_t last_use = 0;
    std::unique_ptr<Plan<real_t>> plan;
};

struct Shim {
    int device = 0;
    std::unique_ptr<Context> ctx;
    std::vector<CachedPlan> plans; // a handful: S, and C's pattern copy, per driver
    uint64_t clock = 0;
    // Device operands are kept between calls and reused while their shape holds.
    std::unique_ptr<Panel<real_t>> a, b, y;
    std::unique_ptr<Vals<real_t>> c;
    double last_us = 0;

    Context &context()
    {
        if (!ctx)
            ctx.reset(new Context(device));
        return *ctx;
    }

    Panel<real_t> &panel(std::unique_ptr<Panel<real_t>> &slot, uint32_t m, uint32_t n)
    {
        if (!slot || slot->rows() != m || slot->cols() != n) {
            slot.reset();
            slot.reset(new Panel<real_t>(context(), m, n));
        }
        return *slot;
    }

    Vals<real_t> &vals(uint64_t n)
    {
        if (!c || c->size() != n) {
            c.reset();
            c.reset(new Vals<real_t>(context(), n));
        }
        return *c;
    }

    // k: the row width the plan will run with (it sizes the set of dense rows planned
    // for L2); a pattern used with another width is planned again.
    Plan<real_t> &plan_for(const cooMat &S, uint32_t nrows, uint32_t ncols, uint32_t k)
    {
        const uint64_t nnz = S.nnz;
        if (S.ii.size() < nnz || S.jj.size() < nnz || S.vv.size() < nnz)
            throw std::out_of_range("cooMat: ii / jj / vv hold fewer than nnz entries");
        const PatternKey key = pattern_key(S.ii.data(), S.jj.data(), nnz);
        ++clock;
        for (CachedPlan &e : plans) {
            if (e.pattern == key && e.nnz == nnz && e.nrows == nrows && e.ncols == ncols &&
                e.k == k) {
                // The values go up on every call: sending them (4 ms for 16 M doubles)
                // is cheaper than reading them once more to see whether they changed.
                e.plan->set_values(S.vv.data());
                e.last_use = clock;
                return *e.plan;
            }
        }
        constexpr size_t kMaxPlans = 4;
        if (plans.size() >= kMaxPlans) {
            size_t oldest = 0;
            for (size_t i = 1; i < plans.size(); ++i)
                if (plans[i].last_use < plans[oldest].last_use)
                    oldest = i;
            plans.erase(plans.begin() + (std::ptrdiff_t)oldest);
        }
        CachedPlan e;
        e.pattern = key;
        e.nnz = nnz;
        e.nrows = nrows;
        e.ncols = ncols;
        e.k = k;
        e.last_use = clock;
        // Validates every index against the panel heights: a bad one throws
        // std::out_of_range here, as the reference's .at() would at that entry.
        spc3d_plan_opts opts = {};
        opts.k_hint = k;
        e.plan.reset(new Plan<real_t>(context(), nrows, ncols, nnz, S.ii.data(), S.jj.data(),
                                      S.vv.data(), &opts));
        plans.push_back(std::move(e));
        return *plans.back().plan;
    }
};

// Never destroyed: at process exit the HIP runtime may already be gone, and
// freeing device memory then is not safe.  hip::shutdown() releases everything.
Shim &shim()
{
    static Shim *s = new Shim;
    return *s;
}

void require_panel(const denseMatrix &M, const char *name)
{
    if (M.data.size() < static_cast<size_t>(M.m) * M.n)
        throw std::out_of_range(std::string("denseMatrix ") + name +
                                ": data holds fewer than m*n values");
}

} // namespace

void sddmm(denseMatrix &A, denseMatrix &B, cooMat &S, cooMat &C)
{
    if (S.nnz == 0)
        return;
    require_panel(A, "A");
    require_panel(B, "B");
    if (C.vv.size() < S.nnz)
        throw std::out_of_range("sddmm: C.vv holds fewer than S.nnz values");
    if (B.n != A.n)
        throw std::runtime_error("sddmm: B.n != A.n is not supported");
    Shim &s = shim();
    Plan<real_t> &plan = s.plan_for(S, A.m, B.m, A.n);
    Panel<real_t> &a = s.panel(s.a, A.m, A.n);
    Panel<real_t> &b = s.panel(s.b, B.m, B.n);
    Vals<real_t> &c = s.vals(S.nnz);
    a.upload(A.data.data());
    b.upload(B.data.data());
    Context &ctx = s.context();
    ctx.mark(0);
    spc3d::sddmm(ctx, plan, a, b, c);
    ctx.mark(1);
    if (C.vv.size() == S.nnz) {
        c.download(C.vv.data());
    } else { // only the first S.nnz values of a longer C.vv are written
        std::vector<real_t> tmp(S.nnz);
        c.download(tmp.data());
        std::memcpy(C.vv.data(), tmp.data(), S.nnz * sizeof(real_t));
    }
    s.last_us = 1e3 * ctx.elapsed_ms(0, 1);
}

void spmm(denseMatrix &X, cooMat &A, denseMatrix &Y)
{
    if (A.nnz == 0)
        return;
    require_panel(X, "X");
    require_panel(Y, "Y");
    if (Y.n != X.n)
        throw std::runtime_error("spmm: Y.n != X.n is not supported");
    Shim &s = shim();
    Plan<real_t> &plan = s.plan_for(A, Y.m, X.m, X.n);
    Panel<real_t> &x = s.panel(s.b, X.m, X.n);
    Panel<real_t> &y = s.panel(s.y, Y.m, Y.n);
    x.upload(X.data.data());
    y.upload(Y.data.data());
    Context &ctx = s.context();
    ctx.mark(0);
    spc3d::spmm(ctx, plan, x, y);
    ctx.mark(1);
    y.download(Y.data.data());
    s.last_us = 1e3 * ctx.elapsed_ms(0, 1);
}

namespace hip {

void set_device(int device)
{
    Shim &s = shim();
    if (s.ctx && s.device != device)
        shutdown();
    s.device = device;
}

void invalidate(const cooMat *)
{
    // Plans are keyed by content, not by address: dropping all of them is
    // always enough and costs one re-plan per matrix.
    shim().plans.clear();
}

double last_kernel_us() { return shim().last_us; }

void shutdown()
{
    Shim &s = shim();
    s.plans.clear();
    s.a.reset();
    s.b.reset();
    s.y.reset();
    s.c.reset();
    s.ctx.reset();
}

} // namespace hip
} // namespace SpKernels
