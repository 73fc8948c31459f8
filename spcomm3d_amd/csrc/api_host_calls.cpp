// C ABI, the one-shot calls over host memory (spc3d_sddmm_host, spc3d_spmm_host) and what a
// context keeps between them (see include/spcomm3d_hip.h and api_internal.h).
#include "api_internal.h"

extern "C" {

namespace {

bool host_cache_enabled(const spc3d_ctx *ctx) { return ctx->use_host_cache; }

HostCallCache *cache_of(spc3d_ctx *ctx)
{
    if (!ctx->host_cache)
        ctx->host_cache = new (std::nothrow) HostCallCache();
    return ctx->host_cache;
}

void sample_indices(const uint32_t *ii, const uint32_t *jj, uint64_t nnz, std::vector<uint32_t> &out)
{
    out.clear();
    for (size_t s = 0; s < HostCallCache::kSamples && nnz; ++s) {
        const uint64_t e = (uint64_t)((unsigned __int128)s * nnz / HostCallCache::kSamples);
        out.push_back(ii[e]);
        out.push_back(jj[e]);
    }
}

// The plan for this pattern at this row width: the cached one when the pattern's
// content is what it was planned from, else a new one (which validates every index, so
// a bad one is reported as the one-shot calls always reported it).  The values are
// sent on every call: that costs less than reading them to see whether they changed.
int host_plan(spc3d_ctx *ctx, HostCallCache *hc, int dtype, uint32_t nrows, uint32_t ncols,
              uint32_t k, uint64_t nnz, const uint32_t *ii, const uint32_t *jj, const void *vv,
              spc3d_plan **out)
{
    *out = nullptr;
    if (nnz && (!ii || !jj))
        return fail(SPC3D_ERR_INVALID_ARG, "ii or jj is NULL");
    std::vector<BlockKey> kii, kjj;
    std::vector<uint32_t> sample;
    keys_of(ii, (size_t)nnz * 4, kii, ctx->host_threads);
    keys_of(jj, (size_t)nnz * 4, kjj, ctx->host_threads);
    sample_indices(ii, jj, nnz, sample);
    ++hc->clock;
    for (CachedHostPlan &e : hc->plans) {
        if (e.dtype == dtype && e.nrows == nrows && e.ncols == ncols && e.k == k && e.nnz == nnz &&
            e.key_ii == kii && e.key_jj == kjj && e.sample == sample) {
            int rc = spc3d_plan_set_values(e.plan, vv);
            if (rc)
                return rc;
            e.last_use = hc->clock;
            hc->plan_reused = 1;
            hc->bytes_sent += (uint64_t)nnz * elem_size(dtype);
            *out = e.plan;
            return SPC3D_OK;
        }
    }
    hc->plan_reused = 0;
    if (hc->plans.size() >= HostCallCache::kMaxPlans) {
        size_t oldest = 0;
        for (size_t i = 1; i < hc->plans.size(); ++i)
            if (hc->plans[i].last_use < hc->plans[oldest].last_use)
                oldest = i;
        (void)spc3d_plan_destroy(hc->plans[oldest].plan);
        hc->plans.erase(hc->plans.begin() + (std::ptrdiff_t)oldest);
    }
    spc3d_plan_opts o = opts_from_env();
    if (!o.k_hint)
        o.k_hint = k; // the one width this plan will run with; sizes the partial-sum rows too
    spc3d_plan *plan = nullptr;
    int rc = spc3d_plan_create_ex(ctx, dtype, nrows, ncols, nnz, ii, jj, vv, &o, &plan);
    if (rc)
        return rc;
    hc->bytes_sent += (uint64_t)nnz * (8 + elem_size(dtype));
    CachedHostPlan e;
    e.plan = plan;
    e.dtype = dtype;
    e.nrows = nrows;
    e.ncols = ncols;
    e.k = k;
    e.nnz = nnz;
    e.key_ii.swap(kii);
    e.key_jj.swap(kjj);
    e.sample.swap(sample);
    e.last_use = hc->clock;
    hc->plans.push_back(std::move(e));
    *out = plan;
    return SPC3D_OK;
}

// A kept device panel of this shape for the operand at `host`, or a new one.  keys: those
// of the operand's blocks, or empty when they were not computed.  Among the panels that this
// call does not use yet: the one that holds most of the operand already; failing that, for
// an output, the one this memory's last result was fetched from; failing that one that
// mirrors nothing;
// failing that a new one while there is room, so that a second operand of the same shape
// (A and B of a square pattern, two panels used in turn) does not push the first one out;
// only then the one unused for longest.
int pick_panel(spc3d_ctx *ctx, HostCallCache *hc, int dtype, uint32_t m, uint32_t n,
               const std::vector<BlockKey> &keys, bool output, const void *host, uint64_t stamp,
               CachedHostPanel **out)
{
    *out = nullptr;
    CachedHostPanel *hit = nullptr, *was_output = nullptr, *other_output = nullptr, *blank = nullptr,
                    *oldest = nullptr;
    size_t best = 0; // blocks that would stay
    for (auto &up : hc->panels) {
        CachedHostPanel &e = *up;
        if (e.last_use == stamp || e.panel->dtype != dtype || e.panel->m != m || e.panel->n != n)
            continue;
        if (output && e.output) {
            if (e.host == host)
                was_output = &e; // this memory's own result panel
            else if (!other_output || e.last_use < other_output->last_use)
                other_output = &e; // another result, which a later call may want as an input
        }
        if (e.keys.empty()) {
            if (!blank || e.host == host)
                blank = &e;
            continue;
        }
        size_t same = 0;
        if (!keys.empty() && e.keys.size() == keys.size())
            for (size_t b = 0; b < keys.size(); ++b)
                same += e.keys[b] == keys[b];
        if (same > best || (same == best && same > 0 && e.host == host)) {
            hit = &e;
            best = same;
        }
        if (!e.output && (!oldest || e.last_use < oldest->last_use))
            oldest = &e;
    }
    if (!hit)
        hit = was_output;
    if (!hit)
        hit = blank;
    if (!hit && hc->panels.size() >= HostCallCache::kMaxPanels)
        hit = output ? other_output : oldest; // same shape, other content: sent in full
    if (!hit) {
        if (hc->panels.size() >= HostCallCache::kMaxPanels) {
            size_t lru = hc->panels.size();
            for (size_t i = 0; i < hc->panels.size(); ++i)
                if (hc->panels[i]->last_use != stamp &&
                    (lru == hc->panels.size() || hc->panels[i]->last_use < hc->panels[lru]->last_use))
                    lru = i;
            if (lru < hc->panels.size()) {
                (void)spc3d_panel_destroy(hc->panels[lru]->panel);
                hc->panels.erase(hc->panels.begin() + (std::ptrdiff_t)lru);
            }
        }
        std::unique_ptr<CachedHostPanel> e(new (std::nothrow) CachedHostPanel());
        if (!e)
            return fail(SPC3D_ERR_ALLOC, "host allocation failed");
        int rc = spc3d_panel_create(ctx, dtype, m, n, &e->panel);
        if (rc)
            return rc;
        hc->panels.push_back(std::move(e));
        hit = hc->panels.back().get();
    }
    hit->last_use = stamp;
    *out = hit;
    return SPC3D_OK;
}

// What one operand's transfer did; merged into the cache's figures by the calling thread.
struct Moved {
    uint64_t sent = 0, kept = 0;
    int rc = SPC3D_OK;
    std::string err; // the failing thread's message (the error text is per thread)
};

// Brings `slot`'s panel to the content of `host`.  keys (of host's blocks): the blocks whose
// key is the slot's stay as they are, the others are sent, neighbouring ones in one copy;
// no keys: everything is sent and the slot mirrors nothing known afterwards.  May run on a
// thread of its own (it touches this slot only).
void send_panel(spc3d_ctx *ctx, CachedHostPanel *slot, const void *host,
                std::vector<BlockKey> &keys, Moved &mv)
{
    const spc3d_panel *P = slot->panel;
    const size_t bytes = (size_t)P->m * P->n * elem_size(P->dtype);
    const bool known = !keys.empty() && slot->keys.size() == keys.size();
    const size_t nblocks = (bytes + kKeyBlockBytes - 1) / kKeyBlockBytes;
    const char *src = static_cast<const char *>(host);
    char *dst = static_cast<char *>(P->dev);
    hipError_t err = hipSetDevice(ctx->device);
    for (size_t b = 0; err == hipSuccess && b < nblocks;) {
        if (known && slot->keys[b] == keys[b]) {
            mv.kept += std::min(kKeyBlockBytes, bytes - b * kKeyBlockBytes);
            ++b;
            continue;
        }
        size_t e = b + 1;
        while (e < nblocks && !(known && slot->keys[e] == keys[e]))
            ++e;
        const size_t off = b * kKeyBlockBytes, len = std::min(bytes, e * kKeyBlockBytes) - off;
        err = hipMemcpyAsync(dst + off, src + off, len, hipMemcpyHostToDevice, ctx->stream);
        mv.sent += len;
        b = e;
    }
    if (err == hipSuccess)
        err = hipStreamSynchronize(ctx->stream);
    if (err != hipSuccess) {
        slot->keys.clear(); // the panel's content is no longer known
        mv.rc = fail_hip(err, "upload of a dense operand");
        mv.err = g_err;
        return;
    }
    slot->keys.swap(keys); // empty when none were given
    slot->host = host;
}

// An input operand: keys of every block (threads), the kept panel that matches best, the
// changed blocks sent.
int host_input(spc3d_ctx *ctx, HostCallCache *hc, int dtype, uint32_t m, uint32_t n,
               const void *host, uint64_t stamp, spc3d_panel **out)
{
    *out = nullptr;
    const size_t bytes = (size_t)m * n * elem_size(dtype);
    if (bytes && !host)
        return fail(SPC3D_ERR_INVALID_ARG, "a dense operand is NULL");
    std::vector<BlockKey> keys;
    keys_of(host, bytes, keys, ctx->host_threads);
    CachedHostPanel *slot = nullptr;
    int rc = pick_panel(ctx, hc, dtype, m, n, keys, false, host, stamp, &slot);
    if (rc)
        return rc;
    slot->output = false;
    Moved mv;
    send_panel(ctx, slot, host, keys, mv);
    hc->bytes_sent += mv.sent;
    hc->bytes_kept += mv.kept;
    if (mv.rc)
        return fail(mv.rc, mv.err);
    *out = slot->panel;
    return SPC3D_OK;
}

// The operand the kernel changes, before the call: what the caller left untouched since the
// last result was fetched into this memory stays on the device (see CachedHostPanel).
// Runs beside the inputs' transfers, on a thread of its own.
void send_output_operand(spc3d_ctx *ctx, CachedHostPanel *slot, const void *host, Moved &mv)
{
    const size_t bytes = (size_t)slot->panel->m * slot->panel->n * elem_size(slot->panel->dtype);
    std::vector<BlockKey> keys;
    const bool read_first = !slot->keys.empty() && slot->skip == 0;
    try { // runs as a thread's function: nothing may leave it
        if (read_first) // beside the thread that reads X: half of the context's threads each
            keys_of(host, bytes, keys, std::max(1u, ctx->host_threads / 2));
        else if (slot->skip)
            --slot->skip;
    } catch (const std::exception &) {
        keys.clear(); // no keys: everything is sent
    }
    send_panel(ctx, slot, host, keys, mv);
    if (mv.rc || !read_first)
        return;
    if (mv.sent > mv.kept) { // mostly rewritten: do not read it first for a while
        slot->backoff = std::min<uint32_t>(16, slot->backoff ? 2 * slot->backoff : 1);
        slot->skip = slot->backoff;
    } else {
        slot->backoff = 0;
    }
}

// The changed operand, after the call: fetched into the caller's memory in pieces, each
// piece keyed by worker threads while the next one is on its way.
int fetch_output_operand(spc3d_ctx *ctx, CachedHostPanel *slot, void *host)
{
    const spc3d_panel *P = slot->panel;
    const size_t bytes = (size_t)P->m * P->n * elem_size(P->dtype);
    const size_t nblocks = (bytes + kKeyBlockBytes - 1) / kKeyBlockBytes;
    std::vector<BlockKey> keys(nblocks);
    // `ready` blocks have arrived; the workers sleep on the condition until theirs has.
    std::mutex mu;
    std::condition_variable cv;
    size_t ready = 0;
    std::atomic<size_t> next{0};
    char *dst = static_cast<char *>(host);
    auto publish = [&](size_t upto) {
        {
            std::lock_guard<std::mutex> lock(mu);
            ready = upto;
        }
        cv.notify_all();
    };
    auto work = [&]() {
        for (;;) {
            const size_t b = next.fetch_add(1, std::memory_order_relaxed);
            if (b >= nblocks)
                return;
            {
                std::unique_lock<std::mutex> lock(mu);
                cv.wait(lock, [&] { return ready > b; });
            }
            const size_t off = b * kKeyBlockBytes;
            keys[b] = key_of_block(dst + off, std::min(kKeyBlockBytes, bytes - off));
        }
    };
    // Workers beside the copying thread: what the context allows, at most 4 (a 16 MiB piece is
    // keyed faster than the next one arrives).  None: this thread keys everything at the end.
    const unsigned nthreads =
        (unsigned)std::min<size_t>(std::min(4u, ctx->host_threads > 1 ? ctx->host_threads - 1 : 0u),
                                   nblocks);
    // Joined on every way out, after the workers have been let run out.
    struct Pool {
        std::vector<std::thread> threads;
        std::function<void()> release;
        ~Pool()
        {
            release();
            for (std::thread &t : threads)
                if (t.joinable())
                    t.join();
        }
    } workers{{}, [&] { publish(nblocks); }};
    std::vector<std::thread> &pool = workers.threads;
    try {
        pool.reserve(nthreads);
        for (unsigned t = 0; t < nthreads; ++t)
            pool.emplace_back(work);
    } catch (const std::exception &) {
        // fewer workers, or none: what is left over is keyed by this thread at the end
    }
    constexpr size_t kPiece = 4; // blocks per copy: 16 MiB
    hipError_t err = hipSuccess;
    const char *src = static_cast<const char *>(P->dev);
    for (size_t b = 0; b < nblocks && err == hipSuccess; b += kPiece) {
        const size_t off = b * kKeyBlockBytes;
        const size_t len = std::min(bytes, (b + kPiece) * kKeyBlockBytes) - off;
        err = hipMemcpyAsync(dst + off, src + off, len, hipMemcpyDeviceToHost, ctx->stream);
        if (err == hipSuccess)
            err = hipStreamSynchronize(ctx->stream);
        if (err == hipSuccess)
            publish(std::min(nblocks, b + kPiece));
    }
    publish(nblocks); // lets the workers run out also after a failure
    work(); // whatever no worker has taken
    for (std::thread &t : pool)
        t.join();
    if (err != hipSuccess) {
        slot->keys.clear();
        return fail_hip(err, "download of a dense operand");
    }
    slot->keys.swap(keys);
    slot->host = host;
    slot->output = true;
    return SPC3D_OK;
}

int host_call_begin(spc3d_ctx *ctx, HostCallCache **hc)
{
    if (!live(ctx))
        return fail(SPC3D_ERR_INVALID_ARG, "context is NULL or destroyed");
    if (int rc = use_device(ctx))
        return rc;
    *hc = cache_of(ctx);
    if (!*hc)
        return fail(SPC3D_ERR_ALLOC, "host allocation failed");
    (*hc)->bytes_sent = (*hc)->bytes_kept = 0;
    (*hc)->plan_reused = 0;
    return SPC3D_OK;
}

} // namespace

int spc3d_host_cache_clear(spc3d_ctx *ctx)
{
    if (!live(ctx))
        return fail(SPC3D_ERR_INVALID_ARG, "context is NULL or destroyed");
    std::lock_guard<std::mutex> lock(ctx->host_mutex);
    HostCallCache *hc = ctx->host_cache;
    if (!hc)
        return SPC3D_OK;
    (void)hipSetDevice(ctx->device);
    for (CachedHostPlan &e : hc->plans)
        (void)spc3d_plan_destroy(e.plan);
    for (auto &e : hc->panels)
        (void)spc3d_panel_destroy(e->panel);
    if (hc->c)
        (void)spc3d_vals_destroy(hc->c);
    delete hc;
    ctx->host_cache = nullptr;
    return SPC3D_OK;
}

int spc3d_host_call_stats(spc3d_ctx *ctx, uint64_t *bytes_sent, uint64_t *bytes_kept,
                          int *plan_reused)
{
    if (!live(ctx))
        return fail(SPC3D_ERR_INVALID_ARG, "context is NULL or destroyed");
    std::lock_guard<std::mutex> lock(ctx->host_mutex);
    const HostCallCache *hc = ctx->host_cache;
    if (bytes_sent) *bytes_sent = hc ? hc->bytes_sent : 0;
    if (bytes_kept) *bytes_kept = hc ? hc->bytes_kept : 0;
    if (plan_reused) *plan_reused = hc ? hc->plan_reused : 0;
    return SPC3D_OK;
}

// One-shot SDDMM without the cache (SPC3D_HOST_CACHE=0): plan, upload, run, download, free.
static int sddmm_host_uncached(spc3d_ctx *ctx, int dtype, uint32_t m, uint32_t n, uint32_t k,
                               const void *A, const void *B, uint64_t nnz, const uint32_t *ii,
                               const uint32_t *jj, const void *svv, void *cvv)
{
    spc3d_plan *S = nullptr;
    spc3d_panel *a = nullptr, *b = nullptr;
    spc3d_vals *c = nullptr;
    spc3d_plan_opts o = opts_from_env();
    if (!o.k_hint)
        o.k_hint = k; // the one width this plan will ever run with
    int rc = spc3d_plan_create_ex(ctx, dtype, m, n, nnz, ii, jj, svv, &o, &S);
    if (!rc) rc = spc3d_panel_create(ctx, dtype, m, k, &a);
    if (!rc) rc = spc3d_panel_create(ctx, dtype, n, k, &b);
    if (!rc) rc = spc3d_vals_create(ctx, dtype, nnz, &c);
    if (!rc) rc = spc3d_panel_upload(a, A);
    if (!rc) rc = spc3d_panel_upload(b, B);
    if (!rc) rc = spc3d_timer_mark(ctx, SPC3D_TIMER_HOST_CALL_BEGIN);
    if (!rc) rc = spc3d_sddmm(ctx, S, a, b, c);
    if (!rc) rc = spc3d_timer_mark(ctx, SPC3D_TIMER_HOST_CALL_END);
    if (!rc) rc = spc3d_vals_download(c, cvv);
    const std::string keep = g_err;
    if (c) spc3d_vals_destroy(c);
    if (b) spc3d_panel_destroy(b);
    if (a) spc3d_panel_destroy(a);
    if (S) spc3d_plan_destroy(S);
    return rc ? fail(rc, keep) : SPC3D_OK;
}

static int sddmm_host_call(spc3d_ctx *ctx, int dtype, uint32_t m, uint32_t n, uint32_t k,
                           const void *A, const void *B, uint64_t nnz, const uint32_t *ii,
                           const uint32_t *jj, const void *svv, void *cvv)
{
    if (nnz && (!svv || !cvv))
        return fail(SPC3D_ERR_INVALID_ARG, "svv or cvv is NULL");
    if (!live(ctx) || !dtype_ok(dtype)) // reported as plan creation reports it (bad pattern first)
        return sddmm_host_uncached(ctx, dtype, m, n, k, A, B, nnz, ii, jj, svv, cvv);
    std::lock_guard<std::mutex> lock(ctx->host_mutex);
    if (!live(ctx))
        return fail(SPC3D_ERR_INVALID_ARG, "context is NULL or destroyed");
    if (!host_cache_enabled(ctx))
        return sddmm_host_uncached(ctx, dtype, m, n, k, A, B, nnz, ii, jj, svv, cvv);
    HostCallCache *hc = nullptr;
    int rc = host_call_begin(ctx, &hc);
    if (rc)
        return rc;
    spc3d_plan *S = nullptr;
    spc3d_panel *a = nullptr, *b = nullptr;
    rc = host_plan(ctx, hc, dtype, m, n, k, nnz, ii, jj, svv, &S);
    const uint64_t stamp = hc->clock; // host_plan advanced it: unique to this call
    if (!rc) rc = host_input(ctx, hc, dtype, m, k, A, stamp, &a);
    if (!rc) rc = host_input(ctx, hc, dtype, n, k, B, stamp, &b);
    if (!rc && (!hc->c || hc->c->dtype != dtype || hc->c->n != nnz)) {
        if (hc->c)
            (void)spc3d_vals_destroy(hc->c);
        hc->c = nullptr;
        rc = spc3d_vals_create(ctx, dtype, nnz, &hc->c);
    }
    if (!rc) rc = spc3d_timer_mark(ctx, SPC3D_TIMER_HOST_CALL_BEGIN);
    if (!rc) rc = spc3d_sddmm(ctx, S, a, b, hc->c);
    if (!rc) rc = spc3d_timer_mark(ctx, SPC3D_TIMER_HOST_CALL_END);
    if (!rc) rc = spc3d_vals_download(hc->c, cvv);
    return rc;
}

int spc3d_sddmm_host(spc3d_ctx *ctx, int dtype, uint32_t m, uint32_t n, uint32_t k, const void *A,
                     const void *B, uint64_t nnz, const uint32_t *ii, const uint32_t *jj,
                     const void *svv, void *cvv)
{
    try {
        return sddmm_host_call(ctx, dtype, m, n, k, A, B, nnz, ii, jj, svv, cvv);
    } catch (const std::bad_alloc &) {
        return fail(SPC3D_ERR_ALLOC, "host allocation failed");
    }
}

static int spmm_host_uncached(spc3d_ctx *ctx, int dtype, uint32_t ncols, uint32_t nrows, uint32_t k,
                              const void *X, uint64_t nnz, const uint32_t *ii, const uint32_t *jj,
                              const void *avv, void *Y)
{
    spc3d_plan *S = nullptr;
    spc3d_panel *x = nullptr, *y = nullptr;
    spc3d_plan_opts o = opts_from_env();
    if (!o.k_hint)
        o.k_hint = k;
    int rc = spc3d_plan_create_ex(ctx, dtype, nrows, ncols, nnz, ii, jj, avv, &o, &S);
    if (!rc) rc = spc3d_panel_create(ctx, dtype, ncols, k, &x);
    if (!rc) rc = spc3d_panel_create(ctx, dtype, nrows, k, &y);
    if (!rc) rc = spc3d_panel_upload(x, X);
    if (!rc) rc = spc3d_panel_upload(y, Y);
    if (!rc) rc = spc3d_timer_mark(ctx, SPC3D_TIMER_HOST_CALL_BEGIN);
    if (!rc) rc = spc3d_spmm(ctx, S, x, y);
    if (!rc) rc = spc3d_timer_mark(ctx, SPC3D_TIMER_HOST_CALL_END);
    if (!rc) rc = spc3d_panel_download(y, Y);
    const std::string keep = g_err;
    if (y) spc3d_panel_destroy(y);
    if (x) spc3d_panel_destroy(x);
    if (S) spc3d_plan_destroy(S);
    return rc ? fail(rc, keep) : SPC3D_OK;
}

static int spmm_host_call(spc3d_ctx *ctx, int dtype, uint32_t ncols, uint32_t nrows, uint32_t k,
                          const void *X, uint64_t nnz, const uint32_t *ii, const uint32_t *jj,
                          const void *avv, void *Y)
{
    if (nnz && !avv)
        return fail(SPC3D_ERR_INVALID_ARG, "avv is NULL");
    if (!live(ctx) || !dtype_ok(dtype))
        return spmm_host_uncached(ctx, dtype, ncols, nrows, k, X, nnz, ii, jj, avv, Y);
    std::lock_guard<std::mutex> lock(ctx->host_mutex);
    if (!live(ctx))
        return fail(SPC3D_ERR_INVALID_ARG, "context is NULL or destroyed");
    if (!host_cache_enabled(ctx))
        return spmm_host_uncached(ctx, dtype, ncols, nrows, k, X, nnz, ii, jj, avv, Y);
    HostCallCache *hc = nullptr;
    int rc = host_call_begin(ctx, &hc);
    if (rc)
        return rc;
    const size_t ybytes = (size_t)nrows * k * elem_size(dtype);
    if (ybytes && !Y)
        return fail(SPC3D_ERR_INVALID_ARG, "Y is NULL");
    spc3d_plan *S = nullptr;
    spc3d_panel *x = nullptr;
    rc = host_plan(ctx, hc, dtype, nrows, ncols, k, nnz, ii, jj, avv, &S);
    if (rc)
        return rc;
    const uint64_t stamp = hc->clock;
    // Y first: its panel is chosen here, then brought up to date on a thread of its own
    // while this one reads X for its keys and sends what changed of it.
    CachedHostPanel *yslot = nullptr;
    {
        std::vector<BlockKey> none;
        rc = pick_panel(ctx, hc, dtype, nrows, k, none, true, Y, stamp, &yslot);
        if (rc)
            return rc;
        if (!yslot->output || yslot->host != Y) { // another operand's panel, or other memory:
            yslot->keys.clear();                  // nothing of it is known to be Y's
            yslot->skip = yslot->backoff = 0;
        }
        yslot->output = true;
    }
    Moved ymv;
    std::thread ythread;
    struct Joined { // on every way out
        std::thread &t;
        ~Joined()
        {
            if (t.joinable())
                t.join();
        }
    } joined{ythread};
    if (ctx->host_threads < 2) {
        send_output_operand(ctx, yslot, Y, ymv); // one thread: one after the other
    } else {
        try {
            ythread = std::thread(send_output_operand, ctx, yslot, (const void *)Y, std::ref(ymv));
        } catch (const std::system_error &) {
            send_output_operand(ctx, yslot, Y, ymv); // no thread to be had: one after the other
        }
    }
    rc = host_input(ctx, hc, dtype, ncols, k, X, stamp, &x);
    if (ythread.joinable())
        ythread.join();
    hc->bytes_sent += ymv.sent;
    hc->bytes_kept += ymv.kept;
    if (!rc && ymv.rc)
        rc = fail(ymv.rc, ymv.err);
    if (!rc) rc = spc3d_timer_mark(ctx, SPC3D_TIMER_HOST_CALL_BEGIN);
    if (!rc) rc = spc3d_spmm(ctx, S, x, yslot->panel);
    if (!rc) rc = spc3d_timer_mark(ctx, SPC3D_TIMER_HOST_CALL_END);
    if (!rc)
        rc = fetch_output_operand(ctx, yslot, Y);
    else
        yslot->keys.clear(); // whatever the panel holds now, it is not known to be Y
    return rc;
}

int spc3d_spmm_host(spc3d_ctx *ctx, int dtype, uint32_t ncols, uint32_t nrows, uint32_t k,
                    const void *X, uint64_t nnz, const uint32_t *ii, const uint32_t *jj,
                    const void *avv, void *Y)
{
    try {
        return spmm_host_call(ctx, dtype, ncols, nrows, k, X, nnz, ii, jj, avv, Y);
    } catch (const std::bad_alloc &) {
        return fail(SPC3D_ERR_ALLOC, "host allocation failed");
    }
}

} // extern "C"
