// C ABI of the local SDDMM / SpMM library (see include/spcomm3d_hip.h): contexts, recorded
// sequences, timers, dense panels, value vectors, and the hot path (spc3d_sddmm, spc3d_spmm,
// the one-pass call, the row copies).  Plans are in api_plan.cpp, the one-shot calls over
// host memory in api_host_calls.cpp.  No CPU compute fallback: without a device every
// device call fails.
#include "api_internal.h"

// ---- partial-sum rows for the SpMM entry point that allocates nothing ---------------
// spc3d_spmm_noalloc keeps the partial sums of cut rows here instead of in memory the
// plan allocated.  Every GPU the library is used on holds its own copy of the array
// until the process ends; its address on a device is looked up once, with that device
// current, when the first context on it is created, and host code uses that address,
// never the array's name.
constexpr size_t kStaticScratchBytes = (size_t)SPC3D_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices]; // per device; null until looked up

// Address of `scratch` on `device`, which must be current.
int scratch_of(int device, void **out)
{
    *out = nullptr;
    if (device < 0 || device >= kMaxDevices)
        return fail(SPC3D_ERR_NO_DEVICE, "device id beyond the library's per-device table");
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[device]) {
        void *ptr = nullptr;
        HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        if (!ptr)
            return fail(SPC3D_ERR_HIP, "hipGetSymbolAddress gave no address for the scratch array");
        g_scratch_ptr[device] = ptr;
    }
    *out = g_scratch_ptr[device];
    return SPC3D_OK;
}
} // namespace


extern "C" {

const char *spc3d_version(void) { return "spcomm3d_hip 0.1 (gfx950)"; }

const char *spc3d_last_error(void) { return g_err.c_str(); }

const char *spc3d_kernel_variant(int dtype, uint32_t k)
{
    return dtype_ok(dtype) ? kernel_variant(dtype, k) : nullptr;
}

const char *spc3d_status_name(int status)
{
    switch (status) {
    case SPC3D_OK: return "SPC3D_OK";
    case SPC3D_ERR_INVALID_ARG: return "SPC3D_ERR_INVALID_ARG";
    case SPC3D_ERR_BAD_INDEX: return "SPC3D_ERR_BAD_INDEX";
    case SPC3D_ERR_SIZE_MISMATCH: return "SPC3D_ERR_SIZE_MISMATCH";
    case SPC3D_ERR_TOO_LARGE: return "SPC3D_ERR_TOO_LARGE";
    case SPC3D_ERR_NO_DEVICE: return "SPC3D_ERR_NO_DEVICE";
    case SPC3D_ERR_HIP: return "SPC3D_ERR_HIP";
    case SPC3D_ERR_ALLOC: return "SPC3D_ERR_ALLOC";
    default: return "SPC3D_ERR_UNKNOWN";
    }
}

int spc3d_device_count(int *count)
{
    if (!count)
        return fail(SPC3D_ERR_INVALID_ARG, "count is NULL");
    *count = 0;
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n <= 0) {
        (void)hipGetLastError();
        return fail(SPC3D_ERR_NO_DEVICE,
                    std::string("no HIP device: ") +
                        (e != hipSuccess ? hipGetErrorString(e) : "device count is 0"));
    }
    *count = n;
    return SPC3D_OK;
}

/* ---- context ------------------------------------------------------------- */

// The defaults of spc3d_ctx_create: the library's, each overridable from the environment.
static spc3d_ctx_opts ctx_opts_from_env()
{
    spc3d_ctx_opts o;
    std::memset(&o, 0, sizeof o);
    unsigned long long v = 0;
    if (env_number("SPC3D_HOST_THREADS", &v) && v >= 1 && v <= 256)
        o.host_threads = (uint32_t)v;
    if (env_number("SPC3D_AUX_STREAM", &v) && v == 0)
        o.flags |= SPC3D_CTX_NO_AUX_STREAM;
    if (env_number("SPC3D_HOST_CACHE", &v) && v == 0)
        o.flags |= SPC3D_CTX_NO_HOST_CACHE;
    return o;
}

int spc3d_ctx_create(int device, spc3d_ctx **out)
{
    const spc3d_ctx_opts o = ctx_opts_from_env();
    return spc3d_ctx_create_ex(device, &o, out);
}

int spc3d_ctx_create_ex(int device, const spc3d_ctx_opts *opts, spc3d_ctx **out)
{
    spc3d_ctx_opts o;
    std::memset(&o, 0, sizeof o);
    if (opts)
        o = *opts;
    if ((o.flags & ~(uint32_t)(SPC3D_CTX_NO_AUX_STREAM | SPC3D_CTX_NO_HOST_CACHE)) || o.reserved[0] ||
        o.reserved[1] || o.reserved[2] || o.reserved[3] || o.reserved[4] || o.reserved[5])
        return fail(SPC3D_ERR_INVALID_ARG, "spc3d_ctx_opts has unknown flags or reserved words set");
    if (o.host_threads > 256)
        return fail(SPC3D_ERR_INVALID_ARG, "spc3d_ctx_opts.host_threads must be at most 256");
    if (!out)
        return fail(SPC3D_ERR_INVALID_ARG, "out is NULL");
    *out = nullptr;
    int n = 0;
    int rc = spc3d_device_count(&n);
    if (rc != SPC3D_OK)
        return rc;
    if (device < 0 || device >= n)
        return fail(SPC3D_ERR_NO_DEVICE, "device id out of range");
    HIP_TRY(hipSetDevice(device));
    spc3d_ctx *c = new (std::nothrow) spc3d_ctx();
    if (!c)
        return fail(SPC3D_ERR_ALLOC, "host allocation failed");
    c->device = device;
    rc = scratch_of(device, &c->scratch);
    if (rc != SPC3D_OK) {
        delete c;
        return rc;
    }
    hipError_t e = hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking);
    if (e != hipSuccess) {
        delete c;
        return fail_hip(e, "hipStreamCreateWithFlags");
    }
    // Same (default) priority as the main stream.  SPC3D_CTX_NO_AUX_STREAM keeps every
    // launch on the main stream.
    c->aux_stream = nullptr;
    c->fork_event = c->join_event = nullptr;
    c->use_host_cache = !(o.flags & SPC3D_CTX_NO_HOST_CACHE);
    c->host_threads = o.host_threads ? o.host_threads : 1;
    c->cu_count = 0;
    if (hipDeviceGetAttribute(&c->cu_count, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess ||
        c->cu_count < 1) {
        (void)hipGetLastError();
        c->cu_count = 256;
    }
    if (!(o.flags & SPC3D_CTX_NO_AUX_STREAM)) {
        e = hipStreamCreateWithFlags(&c->aux_stream, hipStreamNonBlocking);
        if (e == hipSuccess)
            e = hipEventCreateWithFlags(&c->fork_event, hipEventDisableTiming);
        if (e == hipSuccess)
            e = hipEventCreateWithFlags(&c->join_event, hipEventDisableTiming);
        if (e != hipSuccess) {
            if (c->join_event) (void)hipEventDestroy(c->join_event);
            if (c->fork_event) (void)hipEventDestroy(c->fork_event);
            if (c->aux_stream) (void)hipStreamDestroy(c->aux_stream);
            (void)hipStreamDestroy(c->stream);
            delete c;
            return fail_hip(e, "auxiliary stream");
        }
    }
    // Each hardware queue starts its round-robin over the XCDs at its own XCD:
    // measure where workgroup 0 lands on either stream.
    c->aux_rot = 0;
    c->capturing = false;
    if (c->aux_stream) {
        uint32_t *probe = nullptr, host[2] = {0, 0};
        e = hipMalloc((void **)&probe, 2 * sizeof(uint32_t));
        if (e == hipSuccess)
            e = launch_xcc_probe(probe, 1, c->stream);
        if (e == hipSuccess)
            e = launch_xcc_probe(probe + 1, 1, c->aux_stream);
        if (e == hipSuccess)
            e = hipStreamSynchronize(c->stream);
        if (e == hipSuccess)
            e = hipStreamSynchronize(c->aux_stream);
        if (e == hipSuccess)
            e = hipMemcpy(host, probe, sizeof host, hipMemcpyDeviceToHost);
        if (probe)
            (void)hipFree(probe);
        if (e == hipSuccess)
            c->aux_rot = (host[1] - host[0]) & 7u;
        else
            (void)hipGetLastError(); // the rotation only affects speed
    }
    for (int i = 0; i < kTimerSlots; ++i) {
        c->timers[i] = nullptr;
        c->timer_set[i] = false;
    }
    c->host_cache = nullptr;
    c->magic = kMagicCtx;
    *out = c;
    return SPC3D_OK;
}

int spc3d_ctx_destroy(spc3d_ctx *ctx)
{
    if (!live(ctx))
        return fail(SPC3D_ERR_INVALID_ARG, "context is NULL or destroyed");
    if (ctx->capturing) { // drop the unfinished recording
        hipGraph_t g = nullptr;
        (void)hipStreamEndCapture(ctx->stream, &g);
        if (g)
            (void)hipGraphDestroy(g);
        (void)hipGetLastError();
        ctx->capturing = false;
    }
    (void)hipSetDevice(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);
    (void)spc3d_host_cache_clear(ctx);
    for (int i = 0; i < kTimerSlots; ++i)
        if (ctx->timers[i])
            (void)hipEventDestroy(ctx->timers[i]);
    if (ctx->aux_stream) {
        (void)hipStreamSynchronize(ctx->aux_stream);
        (void)hipEventDestroy(ctx->fork_event);
        (void)hipEventDestroy(ctx->join_event);
        (void)hipStreamDestroy(ctx->aux_stream);
    }
    (void)hipStreamDestroy(ctx->stream);
    ctx->magic = 0;
    delete ctx;
    return SPC3D_OK;
}


int spc3d_ctx_sync(spc3d_ctx *ctx)
{
    if (!live(ctx))
        return fail(SPC3D_ERR_INVALID_ARG, "context is NULL or destroyed");
    if (int rc = refuse_while_capturing(ctx))
        return rc;
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    return SPC3D_OK;
}

/* ---- recorded sequences of calls ------------------------------------------- */
int spc3d_capture_begin(spc3d_ctx *ctx)
{
    if (!live(ctx))
        return fail(SPC3D_ERR_INVALID_ARG, "context is NULL or destroyed");
    if (ctx->capturing)
        return fail(SPC3D_ERR_INVALID_ARG, "the context is recording already");
    int rc = use_device(ctx);
    if (rc)
        return rc;
    HIP_TRY(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
    ctx->capturing = true;
    return SPC3D_OK;
}

int spc3d_capture_end(spc3d_ctx *ctx, spc3d_graph **out)
{
    if (!out)
        return fail(SPC3D_ERR_INVALID_ARG, "out is NULL");
    *out = nullptr;
    if (!live(ctx))
        return fail(SPC3D_ERR_INVALID_ARG, "context is NULL or destroyed");
    if (!ctx->capturing)
        return fail(SPC3D_ERR_INVALID_ARG, "the context is not recording");
    ctx->capturing = false;
    hipGraph_t graph = nullptr;
    hipError_t e = hipStreamEndCapture(ctx->stream, &graph);
    if (e != hipSuccess || !graph) {
        (void)hipGetLastError();
        if (graph)
            (void)hipGraphDestroy(graph);
        return fail_hip(e != hipSuccess ? e : hipErrorUnknown, "hipStreamEndCapture");
    }
    hipGraphExec_t exec = nullptr;
    e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGraphDestroy(graph);
        return fail_hip(e, "hipGraphInstantiate");
    }
    spc3d_graph *g = new (std::nothrow) spc3d_graph();
    if (!g) {
        (void)hipGraphExecDestroy(exec);
        (void)hipGraphDestroy(graph);
        return fail(SPC3D_ERR_ALLOC, "host allocation failed");
    }
    g->ctx = ctx;
    g->graph = graph;
    g->exec = exec;
    g->magic = kMagicGraph;
    *out = g;
    return SPC3D_OK;
}

int spc3d_graph_launch(spc3d_graph *g)
{
    if (!live(g))
        return fail(SPC3D_ERR_INVALID_ARG, "graph is NULL or destroyed");
    if (g->ctx->capturing)
        return fail(SPC3D_ERR_INVALID_ARG, "the context is recording");
    int rc = use_device(g->ctx);
    if (rc)
        return rc;
    HIP_TRY(hipGraphLaunch(g->exec, g->ctx->stream));
    return SPC3D_OK;
}

int spc3d_graph_destroy(spc3d_graph *g)
{
    if (!live(g))
        return fail(SPC3D_ERR_INVALID_ARG, "graph is NULL or destroyed");
    if (int rc = refuse_while_capturing(g->ctx))
        return rc;
    (void)hipSetDevice(g->ctx->device);
    (void)hipStreamSynchronize(g->ctx->stream);
    (void)hipGraphExecDestroy(g->exec);
    (void)hipGraphDestroy(g->graph);
    g->magic = 0;
    delete g;
    return SPC3D_OK;
}

int spc3d_ctx_stream(spc3d_ctx *ctx, void **hip_stream)
{
    if (!live(ctx) || !hip_stream)
        return fail(SPC3D_ERR_INVALID_ARG, "context or out pointer is NULL");
    *hip_stream = (void *)ctx->stream;
    return SPC3D_OK;
}

int spc3d_ctx_probe_xcd(spc3d_ctx *ctx, uint32_t nblocks, uint32_t *xcd)
{
    if (!live(ctx) || (nblocks && !xcd))
        return fail(SPC3D_ERR_INVALID_ARG, "context or output is NULL");
    if (nblocks == 0)
        return SPC3D_OK;
    int rc = use_device(ctx);
    if (rc)
        return rc;
    uint32_t *dev = nullptr;
    rc = dev_alloc(&dev, (size_t)nblocks);
    if (rc)
        return rc;
    hipError_t e = launch_xcc_probe(dev, nblocks, ctx->stream);
    if (e != hipSuccess) {
        (void)hipFree(dev);
        return fail_hip(e, "xcc probe");
    }
    rc = copy_d2h(ctx, xcd, dev, (size_t)nblocks * sizeof(uint32_t));
    (void)hipFree(dev);
    return rc;
}

int spc3d_timer_mark(spc3d_ctx *ctx, int slot)
{
    if (!live(ctx))
        return fail(SPC3D_ERR_INVALID_ARG, "context is NULL or destroyed");
    if (slot < 0 || slot >= kTimerSlots)
        return fail(SPC3D_ERR_INVALID_ARG, "timer slot out of range");
    if (int rc = refuse_while_capturing(ctx))
        return rc;
    if (!ctx->timers[slot])
        HIP_TRY(hipEventCreate(&ctx->timers[slot]));
    HIP_TRY(hipEventRecord(ctx->timers[slot], ctx->stream));
    ctx->timer_set[slot] = true;
    return SPC3D_OK;
}

int spc3d_timer_elapsed_ms(spc3d_ctx *ctx, int start, int stop, float *ms)
{
    if (!live(ctx) || !ms)
        return fail(SPC3D_ERR_INVALID_ARG, "context or ms is NULL");
    if (start < 0 || start >= kTimerSlots || stop < 0 || stop >= kTimerSlots ||
        !ctx->timer_set[start] || !ctx->timer_set[stop])
        return fail(SPC3D_ERR_INVALID_ARG, "timer slot not marked");
    HIP_TRY(hipEventSynchronize(ctx->timers[stop]));
    HIP_TRY(hipEventElapsedTime(ms, ctx->timers[start], ctx->timers[stop]));
    return SPC3D_OK;
}

/* ---- panels -------------------------------------------------------------- */
int spc3d_panel_create(spc3d_ctx *ctx, int dtype, uint32_t m, uint32_t n, spc3d_panel **out)
{
    if (!out)
        return fail(SPC3D_ERR_INVALID_ARG, "out is NULL");
    *out = nullptr;
    if (!live(ctx))
        return fail(SPC3D_ERR_INVALID_ARG, "context is NULL or destroyed");
    if (!dtype_ok(dtype))
        return fail(SPC3D_ERR_INVALID_ARG, "unknown dtype");
    int rc = use_device(ctx);
    if (rc)
        return rc;
    spc3d_panel *p = new (std::nothrow) spc3d_panel();
    if (!p)
        return fail(SPC3D_ERR_ALLOC, "host allocation failed");
    p->ctx = ctx;
    p->dtype = dtype;
    p->m = m;
    p->n = n;
    rc = dev_alloc_bytes(&p->dev, (size_t)m * n * elem_size(dtype));
    if (rc) {
        delete p;
        return rc;
    }
    p->magic = kMagicPanel;
    *out = p;
    return SPC3D_OK;
}

namespace {
// `dev` must be `bytes` of device memory of ctx's GPU, 16-byte aligned (the copy and
// pack kernels move 16-byte vectors from the start of a buffer).
int check_wrapped(spc3d_ctx *ctx, const void *dev, size_t bytes)
{
    if (bytes == 0)
        return SPC3D_OK;
    if (!dev)
        return fail(SPC3D_ERR_INVALID_ARG, "device pointer is NULL");
    if (reinterpret_cast<uintptr_t>(dev) % 16)
        return fail(SPC3D_ERR_INVALID_ARG, "device pointer is not 16-byte aligned");
    hipPointerAttribute_t at;
    std::memset(&at, 0, sizeof at);
    if (hipPointerGetAttributes(&at, dev) != hipSuccess) {
        (void)hipGetLastError();
        return fail(SPC3D_ERR_INVALID_ARG, "pointer is not known to the HIP runtime");
    }
    if (at.type != hipMemoryTypeDevice || at.device != ctx->device)
        return fail(SPC3D_ERR_INVALID_ARG, "pointer is not device memory of the context's GPU");
    return SPC3D_OK;
}
} // namespace

int spc3d_panel_wrap(spc3d_ctx *ctx, int dtype, uint32_t m, uint32_t n, void *dev,
                     spc3d_panel **out)
{
    if (!out)
        return fail(SPC3D_ERR_INVALID_ARG, "out is NULL");
    *out = nullptr;
    if (!live(ctx))
        return fail(SPC3D_ERR_INVALID_ARG, "context is NULL or destroyed");
    if (!dtype_ok(dtype))
        return fail(SPC3D_ERR_INVALID_ARG, "unknown dtype");
    int rc = use_device(ctx);
    if (rc)
        return rc;
    rc = check_wrapped(ctx, dev, (size_t)m * n * elem_size(dtype));
    if (rc)
        return rc;
    spc3d_panel *p = new (std::nothrow) spc3d_panel();
    if (!p)
        return fail(SPC3D_ERR_ALLOC, "host allocation failed");
    p->ctx = ctx;
    p->dtype = dtype;
    p->m = m;
    p->n = n;
    p->dev = (size_t)m * n ? dev : nullptr;
    p->owned = false;
    p->magic = kMagicPanel;
    *out = p;
    return SPC3D_OK;
}

int spc3d_panel_destroy(spc3d_panel *p)
{
    if (!live(p))
        return fail(SPC3D_ERR_INVALID_ARG, "panel is NULL or destroyed");
    if (int rc = refuse_while_capturing(p->ctx))
        return rc;
    (void)hipSetDevice(p->ctx->device);
    (void)hipStreamSynchronize(p->ctx->stream);
    if (p->dev && p->owned)
        (void)hipFree(p->dev);
    p->magic = 0;
    delete p;
    return SPC3D_OK;
}

int spc3d_panel_upload(spc3d_panel *p, const void *host)
{
    if (!live(p))
        return fail(SPC3D_ERR_INVALID_ARG, "panel is NULL or destroyed");
    const size_t bytes = (size_t)p->m * p->n * elem_size(p->dtype);
    if (bytes && !host)
        return fail(SPC3D_ERR_INVALID_ARG, "host pointer is NULL");
    int rc = use_device(p->ctx);
    return rc ? rc : copy_h2d(p->ctx, p->dev, host, bytes);
}

int spc3d_panel_download(spc3d_panel *p, void *host)
{
    if (!live(p))
        return fail(SPC3D_ERR_INVALID_ARG, "panel is NULL or destroyed");
    const size_t bytes = (size_t)p->m * p->n * elem_size(p->dtype);
    if (bytes && !host)
        return fail(SPC3D_ERR_INVALID_ARG, "host pointer is NULL");
    int rc = use_device(p->ctx);
    return rc ? rc : copy_d2h(p->ctx, host, p->dev, bytes);
}

int spc3d_panel_fill(spc3d_panel *p, double value)
{
    if (!live(p))
        return fail(SPC3D_ERR_INVALID_ARG, "panel is NULL or destroyed");
    int rc = use_device(p->ctx, true);
    if (rc)
        return rc;
    HIP_TRY(launch_fill(p->dtype, p->dev, (uint64_t)p->m * p->n, value, p->ctx->stream));
    return SPC3D_OK;
}

int spc3d_panel_copy(spc3d_panel *dst, const spc3d_panel *src)
{
    if (!live(dst) || !live(src))
        return fail(SPC3D_ERR_INVALID_ARG, "panel is NULL or destroyed");
    if (dst->ctx != src->ctx)
        return fail(SPC3D_ERR_INVALID_ARG, "panels belong to different contexts");
    if (dst->dtype != src->dtype || dst->m != src->m || dst->n != src->n)
        return fail(SPC3D_ERR_SIZE_MISMATCH, "panels differ in shape or dtype");
    if (dst->dev == src->dev)
        return SPC3D_OK;
    int rc = use_device(dst->ctx, true);
    if (rc)
        return rc;
    HIP_TRY(launch_copy(dst->dev, src->dev, (uint64_t)dst->m * dst->n * elem_size(dst->dtype),
                        dst->ctx->stream));
    return SPC3D_OK;
}

int spc3d_panel_device_ptr(spc3d_panel *p, void **dev)
{
    if (!live(p) || !dev)
        return fail(SPC3D_ERR_INVALID_ARG, "panel or out pointer is NULL");
    *dev = p->dev;
    return SPC3D_OK;
}

int spc3d_panel_shape(spc3d_panel *p, uint32_t *m, uint32_t *n, int *dtype)
{
    if (!live(p))
        return fail(SPC3D_ERR_INVALID_ARG, "panel is NULL or destroyed");
    if (m) *m = p->m;
    if (n) *n = p->n;
    if (dtype) *dtype = p->dtype;
    return SPC3D_OK;
}

/* ---- value vectors ------------------------------------------------------- */
int spc3d_vals_create(spc3d_ctx *ctx, int dtype, uint64_t n, spc3d_vals **out)
{
    if (!out)
        return fail(SPC3D_ERR_INVALID_ARG, "out is NULL");
    *out = nullptr;
    if (!live(ctx))
        return fail(SPC3D_ERR_INVALID_ARG, "context is NULL or destroyed");
    if (!dtype_ok(dtype))
        return fail(SPC3D_ERR_INVALID_ARG, "unknown dtype");
    if (n >= (1ull << 32))
        return fail(SPC3D_ERR_TOO_LARGE, "value vector longer than 2^32 - 1");
    int rc = use_device(ctx);
    if (rc)
        return rc;
    spc3d_vals *v = new (std::nothrow) spc3d_vals();
    if (!v)
        return fail(SPC3D_ERR_ALLOC, "host allocation failed");
    v->ctx = ctx;
    v->dtype = dtype;
    v->n = n;
    rc = dev_alloc_bytes(&v->dev, (size_t)n * elem_size(dtype));
    if (rc) {
        delete v;
        return rc;
    }
    v->magic = kMagicVals;
    *out = v;
    return SPC3D_OK;
}

int spc3d_vals_wrap(spc3d_ctx *ctx, int dtype, uint64_t n, void *dev, spc3d_vals **out)
{
    if (!out)
        return fail(SPC3D_ERR_INVALID_ARG, "out is NULL");
    *out = nullptr;
    if (!live(ctx))
        return fail(SPC3D_ERR_INVALID_ARG, "context is NULL or destroyed");
    if (!dtype_ok(dtype))
        return fail(SPC3D_ERR_INVALID_ARG, "unknown dtype");
    if (n >= (1ull << 32))
        return fail(SPC3D_ERR_TOO_LARGE, "value vector longer than 2^32 - 1");
    int rc = use_device(ctx);
    if (rc)
        return rc;
    rc = check_wrapped(ctx, dev, (size_t)n * elem_size(dtype));
    if (rc)
        return rc;
    spc3d_vals *v = new (std::nothrow) spc3d_vals();
    if (!v)
        return fail(SPC3D_ERR_ALLOC, "host allocation failed");
    v->ctx = ctx;
    v->dtype = dtype;
    v->n = n;
    v->dev = n ? dev : nullptr;
    v->owned = false;
    v->magic = kMagicVals;
    *out = v;
    return SPC3D_OK;
}

int spc3d_vals_destroy(spc3d_vals *v)
{
    if (!live(v))
        return fail(SPC3D_ERR_INVALID_ARG, "value vector is NULL or destroyed");
    if (int rc = refuse_while_capturing(v->ctx))
        return rc;
    (void)hipSetDevice(v->ctx->device);
    (void)hipStreamSynchronize(v->ctx->stream);
    if (v->dev && v->owned)
        (void)hipFree(v->dev);
    v->magic = 0;
    delete v;
    return SPC3D_OK;
}

int spc3d_vals_upload(spc3d_vals *v, const void *host)
{
    if (!live(v))
        return fail(SPC3D_ERR_INVALID_ARG, "value vector is NULL or destroyed");
    if (v->n && !host)
        return fail(SPC3D_ERR_INVALID_ARG, "host pointer is NULL");
    int rc = use_device(v->ctx);
    return rc ? rc : copy_h2d(v->ctx, v->dev, host, (size_t)v->n * elem_size(v->dtype));
}

int spc3d_vals_download(spc3d_vals *v, void *host)
{
    if (!live(v))
        return fail(SPC3D_ERR_INVALID_ARG, "value vector is NULL or destroyed");
    if (v->n && !host)
        return fail(SPC3D_ERR_INVALID_ARG, "host pointer is NULL");
    int rc = use_device(v->ctx);
    return rc ? rc : copy_d2h(v->ctx, host, v->dev, (size_t)v->n * elem_size(v->dtype));
}

int spc3d_vals_fill(spc3d_vals *v, double value)
{
    if (!live(v))
        return fail(SPC3D_ERR_INVALID_ARG, "value vector is NULL or destroyed");
    int rc = use_device(v->ctx, true);
    if (rc)
        return rc;
    HIP_TRY(launch_fill(v->dtype, v->dev, v->n, value, v->ctx->stream));
    return SPC3D_OK;
}

int spc3d_vals_device_ptr(spc3d_vals *v, void **dev)
{
    if (!live(v) || !dev)
        return fail(SPC3D_ERR_INVALID_ARG, "value vector or out pointer is NULL");
    *dev = v->dev;
    return SPC3D_OK;
}


int spc3d_vals_copy(spc3d_vals *dst, uint64_t dst_off, const spc3d_vals *src, uint64_t src_off,
                    uint64_t n)
{
    if (!live(dst) || !live(src))
        return fail(SPC3D_ERR_INVALID_ARG, "a value vector is NULL or destroyed");
    if (dst->ctx != src->ctx)
        return fail(SPC3D_ERR_INVALID_ARG, "operands belong to different contexts");
    if (dst->dtype != src->dtype)
        return fail(SPC3D_ERR_SIZE_MISMATCH, "value vectors of different types");
    if (dst_off > dst->n || n > dst->n - dst_off || src_off > src->n || n > src->n - src_off)
        return fail(SPC3D_ERR_SIZE_MISMATCH, "the range leaves a value vector");
    if (n == 0)
        return SPC3D_OK;
    int rc = use_device(dst->ctx, true);
    if (rc)
        return rc;
    const size_t w = elem_size(dst->dtype);
    char *d = static_cast<char *>(dst->dev) + dst_off * w;
    const char *s = static_cast<const char *>(src->dev) + src_off * w;
    if (ranges_overlap(d, n * w, s, n * w))
        return fail(SPC3D_ERR_INVALID_ARG, "source and destination ranges overlap");
    if ((((uintptr_t)d | (uintptr_t)s) & 15u) == 0)
        HIP_TRY(launch_copy(d, s, n * w, dst->ctx->stream));
    else
        HIP_TRY(hipMemcpyAsync(d, s, n * w, hipMemcpyDeviceToDevice, dst->ctx->stream));
    return SPC3D_OK;
}

/* ---- where the SDDMM results of a plan go ------------------------------------ */
// The staged results of a single plan to their places in C; queued after the launches.
static hipError_t unstage_stores(const spc3d_plan *S, void *C)
{
    if (!S->store.n)
        return hipSuccess;
    return launch_unstage_pairs(S->dtype, S->c_stage, S->store.src, S->store.dst, C, S->store.n,
                                S->ctx->stream);
}

// Where a single plan's SDDMM kernels write: C, or the plan's staging vector when the two
// passes bring the results home afterwards.
static void *sddmm_out(const spc3d_plan *S, void *C) { return S->two.n ? S->c_stage : C; }
static hipError_t finish_sddmm(const spc3d_plan *S, void *C)
{
    if (S->two.n)
        return launch_unpermute_two_pass(S->dtype, S->c_stage, S->c_mid, S->two.l1, S->two.dst1,
                                         S->two.l2, C, S->two.n, S->ctx->stream);
    return unstage_stores(S, C);
}

// A block's view for SDDMM: results at their places in the parent's staging vector.
static DevPlanView staged_view(const spc3d_plan *parent, const spc3d_plan *block)
{
    DevPlanView v = view_of(block);
    // beside a sweep: the plan of the rest, its results in its own kernel order
    v.perm = parent->sweep.n ? nullptr : parent->stage_of + block->stage_off;
    v.stream_c = true;
    return v;
}
// C[e] = c_stage[stage_pos[e]]; a caller's C that is not 16-byte aligned (a wrapped
// vector) goes the element-wise way.
static hipError_t unstage(const spc3d_plan *S, spc3d_vals *C)
{
    if (((uintptr_t)C->dev & 15u) == 0)
        return launch_unstage(S->dtype, S->c_stage, S->stage_pos, C->dev, S->info.nnz,
                              S->ctx->stream);
    return launch_gather_vals(S->dtype, S->c_stage, S->stage_pos, C->dev, S->info.nnz,
                              S->ctx->stream);
}
static void *staged_out(const spc3d_plan *parent, const spc3d_plan *)
{
    return static_cast<char *>(parent->c_stage) + parent->rest_off * elem_size(parent->dtype);
}

/* ---- hot path ------------------------------------------------------------ */
int spc3d_sddmm(spc3d_ctx *ctx, spc3d_plan *S, const spc3d_panel *A, const spc3d_panel *B,
                spc3d_vals *C)
{
    if (!live(ctx) || !live(S) || !live(A) || !live(B) || !live(C))
        return fail(SPC3D_ERR_INVALID_ARG, "a handle is NULL or destroyed");
    if (S->ctx != ctx || A->ctx != ctx || B->ctx != ctx || C->ctx != ctx)
        return fail(SPC3D_ERR_INVALID_ARG, "operands belong to different contexts");
    if (A->dtype != S->dtype || B->dtype != S->dtype || C->dtype != S->dtype)
        return fail(SPC3D_ERR_SIZE_MISMATCH, "operand dtypes differ from the plan's");
    const uint32_t K = A->n; // core_ops.cpp:6
    if (B->n != K)
        return fail(SPC3D_ERR_SIZE_MISMATCH, "A.n != B.n");
    if (S->info.nnz == 0)
        return SPC3D_OK;
    if (A->m < S->info.nrows || B->m < S->info.ncols)
        return fail(SPC3D_ERR_SIZE_MISMATCH, "panel has fewer rows than the pattern addresses");
    if (C->n < S->info.nnz)
        return fail(SPC3D_ERR_SIZE_MISMATCH, "C.vv is shorter than nnz");
    if (!S->has_values)
        return fail(SPC3D_ERR_INVALID_ARG, "plan has no values (spc3d_plan_set_values)");
    if (K == 0) { // empty dot product: every result is 0 * S.vv = 0
        int rc = use_device(ctx, true);
        if (rc)
            return rc;
        HIP_TRY(launch_fill(C->dtype, C->dev, S->info.nnz, 0.0, ctx->stream));
        return SPC3D_OK;
    }
    int rc = use_device(ctx, true);
    if (rc)
        return rc;
    rc = plan_for_k(S, K, true, &S); // a plan in row tiles at another K: its ordinary twin
    if (rc)
        return rc;
    if (S->by_col) { // the same entries with rows and columns, and so A and B, exchanged
        const spc3d_plan *T = S->by_col;
        HIP_TRY(launch_sddmm(S->dtype, view_of(T), B->dev, A->dev, C->dev, K, streams_of(ctx)));
        HIP_TRY(unstage_stores(T, C->dev));
        return SPC3D_OK;
    }
    if (S->blocks.empty() && !S->sweep.n) {
        HIP_TRY(launch_sddmm(S->dtype, view_of(S), A->dev, B->dev, sddmm_out(S, C->dev), K,
                             streams_of(ctx)));
        HIP_TRY(finish_sddmm(S, C->dev));
        return SPC3D_OK;
    }
    if (S->sweep.n && !S->c_stage) { // the tiles and the rest store at the caller's positions
        for (spc3d_plan *part : S->blocks)
            HIP_TRY(launch_sddmm(S->dtype, view_of(part), A->dev, B->dev, C->dev, K, streams_of(ctx)));
        SweepView v = sweep_view_of(S);
        v.pos = S->sweep.perm;
        HIP_TRY(launch_sweep_sddmm(S->dtype, v, A->dev, B->dev, C->dev, ctx->stream));
        return SPC3D_OK;
    }
    for (spc3d_plan *part : S->blocks)
        HIP_TRY(launch_sddmm(S->dtype, staged_view(S, part), A->dev, B->dev, staged_out(S, part), K,
                             streams_of(ctx)));
    if (S->sweep.n)
        HIP_TRY(launch_sweep_sddmm(S->dtype, sweep_view_of(S), A->dev, B->dev, S->c_stage,
                                   ctx->stream));
    HIP_TRY(unstage(S, C));
    return SPC3D_OK;
}

// Checks shared by the SpMM entry points; *K = 0 when there is nothing to do.
static int spmm_check(spc3d_ctx *ctx, spc3d_plan *Ap, const spc3d_panel *X, spc3d_panel *Y,
                      uint32_t *K)
{
    *K = 0;
    if (!live(ctx) || !live(Ap) || !live(X) || !live(Y))
        return fail(SPC3D_ERR_INVALID_ARG, "a handle is NULL or destroyed");
    if (Ap->ctx != ctx || X->ctx != ctx || Y->ctx != ctx)
        return fail(SPC3D_ERR_INVALID_ARG, "operands belong to different contexts");
    if (X->dtype != Ap->dtype || Y->dtype != Ap->dtype)
        return fail(SPC3D_ERR_SIZE_MISMATCH, "operand dtypes differ from the plan's");
    const uint32_t k = X->n; // core_ops.cpp:25
    if (Y->n != k)
        return fail(SPC3D_ERR_SIZE_MISMATCH, "X.n != Y.n");
    if (Ap->info.nnz == 0 || k == 0)
        return SPC3D_OK;
    if (X->m < Ap->info.ncols || Y->m < Ap->info.nrows)
        return fail(SPC3D_ERR_SIZE_MISMATCH, "panel has fewer rows than the pattern addresses");
    if (ranges_overlap(X->dev, panel_bytes(X), Y->dev, panel_bytes(Y)))
        return fail(SPC3D_ERR_INVALID_ARG, "X and Y must not overlap");
    if (!Ap->has_values)
        return fail(SPC3D_ERR_INVALID_ARG, "plan has no values (spc3d_plan_set_values)");
    *K = k;
    return SPC3D_OK;
}

int spc3d_spmm(spc3d_ctx *ctx, spc3d_plan *Ap, const spc3d_panel *X, spc3d_panel *Y)
{
    uint32_t K = 0;
    int rc = spmm_check(ctx, Ap, X, Y, &K);
    if (rc || K == 0)
        return rc;
    rc = use_device(ctx, true);
    if (rc)
        return rc;
    rc = plan_for_k(Ap, K, true, &Ap);
    if (rc)
        return rc;
    std::vector<spc3d_plan *> self;
    for (spc3d_plan *part : parts_of(Ap, self)) {
        rc = ensure_partial(part, K);
        if (rc)
            return rc;
    }
    // The blocks add into Y one after the other on the stream: a fixed order.
    for (spc3d_plan *part : parts_of(Ap, self))
        HIP_TRY(launch_spmm(Ap->dtype, view_of(part), X->dev, Y->dev, K, streams_of(ctx)));
    if (Ap->sweep.n) // rows of their own: none of them is in the plan of the rest
        HIP_TRY(launch_sweep_spmm(Ap->dtype, sweep_view_of(Ap), X->dev, Y->dev, ctx->stream));
    return SPC3D_OK;
}

int spc3d_spmm_noalloc(spc3d_ctx *ctx, spc3d_plan *Ap, const spc3d_panel *X, spc3d_panel *Y)
{
    uint32_t K = 0;
    int rc = spmm_check(ctx, Ap, X, Y, &K);
    if (rc || K == 0)
        return rc;
    rc = plan_for_k(Ap, K, false, &Ap); // (this call builds nothing)
    if (rc)
        return rc;
    const uint64_t need = (uint64_t)Ap->info.npartial_slots * K * elem_size(Ap->dtype);
    if (need > kStaticScratchBytes) {
        char msg[200];
        std::snprintf(msg, sizeof msg,
                      "the partial sums of this plan's cut rows take %llu bytes at K = %u; "
                      "spc3d_spmm_noalloc has %llu (SPC3D_NOALLOC_SCRATCH_BYTES): use spc3d_spmm",
                      (unsigned long long)need, K, (unsigned long long)kStaticScratchBytes);
        return fail(SPC3D_ERR_TOO_LARGE, msg);
    }
    rc = use_device(ctx, true);
    if (rc)
        return rc;
    // Every partial-sum row the fix-up reads is written by exactly one segment of this
    // call first, so what an earlier call left in the array needs no clearing.  (The
    // blocks of a plan kept in column blocks use the array one after the other;
    // npartial_slots is the largest block's.)
    // no container: no host heap either
    const size_t nparts = Ap->blocks.empty() ? (Ap->sweep.n ? 0 : 1) : Ap->blocks.size();
    for (size_t i = 0; i < nparts; ++i) {
        DevPlanView view = view_of(Ap->blocks.empty() ? Ap : Ap->blocks[i]);
        view.partial = ctx->scratch;
        HIP_TRY(launch_spmm(Ap->dtype, view, X->dev, Y->dev, K, streams_of(ctx)));
    }
    if (Ap->sweep.n) // the tiles' sums live in LDS: nothing to allocate either
        HIP_TRY(launch_sweep_spmm(Ap->dtype, sweep_view_of(Ap), X->dev, Y->dev, ctx->stream));
    return SPC3D_OK;
}

int spc3d_sddmm_spmm(spc3d_ctx *ctx, spc3d_plan *S, const spc3d_panel *A, const spc3d_panel *B,
                     spc3d_vals *C, spc3d_panel *Y, int chained)
{
    if (!live(ctx) || !live(S) || !live(A) || !live(B) || !live(C) || !live(Y))
        return fail(SPC3D_ERR_INVALID_ARG, "a handle is NULL or destroyed");
    if (S->ctx != ctx || A->ctx != ctx || B->ctx != ctx || C->ctx != ctx || Y->ctx != ctx)
        return fail(SPC3D_ERR_INVALID_ARG, "operands belong to different contexts");
    if (A->dtype != S->dtype || B->dtype != S->dtype || C->dtype != S->dtype ||
        Y->dtype != S->dtype)
        return fail(SPC3D_ERR_SIZE_MISMATCH, "operand dtypes differ from the plan's");
    const uint32_t K = A->n;
    if (B->n != K || Y->n != K)
        return fail(SPC3D_ERR_SIZE_MISMATCH, "A.n, B.n and Y.n differ");
    if (S->info.nnz == 0)
        return SPC3D_OK;
    if (A->m < S->info.nrows || B->m < S->info.ncols || Y->m < S->info.nrows)
        return fail(SPC3D_ERR_SIZE_MISMATCH, "panel has fewer rows than the pattern addresses");
    if (C->n < S->info.nnz)
        return fail(SPC3D_ERR_SIZE_MISMATCH, "C.vv is shorter than nnz");
    if (ranges_overlap(Y->dev, panel_bytes(Y), A->dev, panel_bytes(A)) ||
        ranges_overlap(Y->dev, panel_bytes(Y), B->dev, panel_bytes(B)))
        return fail(SPC3D_ERR_INVALID_ARG, "Y must not overlap A or B");
    if (!S->has_values)
        return fail(SPC3D_ERR_INVALID_ARG, "plan has no values (spc3d_plan_set_values)");
    int rc = use_device(ctx, true);
    if (rc)
        return rc;
    if (K == 0) { // empty dot products, nothing to add
        HIP_TRY(launch_fill(C->dtype, C->dev, S->info.nnz, 0.0, ctx->stream));
        return SPC3D_OK;
    }
    rc = plan_for_k(S, K, true, &S);
    if (rc)
        return rc;
    std::vector<spc3d_plan *> self;
    for (spc3d_plan *part : parts_of(S, self)) {
        rc = ensure_partial(part, K);
        if (rc)
            return rc;
    }
    const bool direct = S->sweep.n && !S->c_stage; // results straight to the caller's positions
    const bool staged = (!S->blocks.empty() || S->sweep.n) && !direct;
    for (spc3d_plan *part : parts_of(S, self)) {
        const DevPlanView view = staged ? staged_view(S, part) : view_of(part);
        void *out = staged ? staged_out(S, part) : sddmm_out(S, C->dev);
        hipError_t e = launch_sddmm_spmm(S->dtype, chained != 0, view, A->dev, B->dev, out, Y->dev,
                                         K, streams_of(ctx));
        if (e == hipErrorNotSupported) {
            (void)hipGetLastError();
            if (chained)
                return fail(SPC3D_ERR_INVALID_ARG,
                            "the chained form needs dense rows of at most 4096 bytes "
                            "(K * sizeof(real))");
            // No vector kernel for this K: the two calls one after the other.
            HIP_TRY(launch_sddmm(S->dtype, view, A->dev, B->dev, out, K, streams_of(ctx)));
            HIP_TRY(launch_spmm(S->dtype, view, B->dev, Y->dev, K, streams_of(ctx)));
            continue;
        }
        HIP_TRY(e);
    }
    if (S->sweep.n) { // the tiles: SDDMM, then SpMM over the same entries (with the results
                      // just written as its values when chained)
        SweepView v = sweep_view_of(S);
        if (direct)
            v.pos = S->sweep.perm;
        HIP_TRY(launch_sweep_sddmm(S->dtype, v, A->dev, B->dev, direct ? C->dev : S->c_stage,
                                   ctx->stream));
        if (chained)
            v.sval = direct ? C->dev : S->c_stage; // (through v.pos when direct)
        else
            v.pos = nullptr;
        HIP_TRY(launch_sweep_spmm(S->dtype, v, B->dev, Y->dev, ctx->stream));
    }
    if (direct)
        return SPC3D_OK;
    if (staged)
        HIP_TRY(unstage(S, C));
    else
        HIP_TRY(finish_sddmm(S, C->dev));
    return SPC3D_OK;
}

/* ---- row maps and the pack / unpack copies ------------------------------------ */
int spc3d_rowmap_create(spc3d_ctx *ctx, uint32_t panel_rows, uint64_t n, const uint32_t *rows,
                        spc3d_rowmap **out)
{
    if (!out)
        return fail(SPC3D_ERR_INVALID_ARG, "out is NULL");
    *out = nullptr;
    if (n && !rows)
        return fail(SPC3D_ERR_INVALID_ARG, "rows is NULL");
    if (n >= (1ull << 32))
        return fail(SPC3D_ERR_TOO_LARGE, "more than 2^32 - 1 slots");
    for (uint64_t i = 0; i < n; ++i)
        if (rows[i] >= panel_rows) {
            char buf[128];
            std::snprintf(buf, sizeof buf, "slot %llu names row %u of a panel with %u rows",
                          (unsigned long long)i, rows[i], panel_rows);
            return fail(SPC3D_ERR_BAD_INDEX, buf);
        }
    if (!live(ctx))
        return fail(SPC3D_ERR_INVALID_ARG, "context is NULL or destroyed");
    // Group the slots by row, ascending inside a row (stable counting sort).
    std::vector<uint32_t> cnt, urows, ptr, slots;
    try {
        cnt.assign((size_t)panel_rows + 1, 0);
        for (uint64_t i = 0; i < n; ++i)
            ++cnt[(size_t)rows[i] + 1];
        std::vector<uint32_t> start((size_t)panel_rows, 0);
        ptr.push_back(0);
        uint32_t at = 0;
        for (uint32_t r = 0; r < panel_rows; ++r) {
            start[r] = at;
            if (cnt[(size_t)r + 1]) {
                urows.push_back(r);
                at += cnt[(size_t)r + 1];
                ptr.push_back(at);
            }
        }
        slots.resize(n);
        for (uint64_t i = 0; i < n; ++i)
            slots[start[rows[i]]++] = (uint32_t)i;
    } catch (const std::bad_alloc &) {
        return fail(SPC3D_ERR_ALLOC, "host allocation failed");
    }
    int rc = use_device(ctx);
    if (rc)
        return rc;
    spc3d_rowmap *m = new (std::nothrow) spc3d_rowmap();
    if (!m)
        return fail(SPC3D_ERR_ALLOC, "host allocation failed");
    m->ctx = ctx;
    m->panel_rows = panel_rows;
    m->nslots = (uint32_t)n;
    m->nuniq = (uint32_t)urows.size();
    rc = dev_alloc(&m->rows, (size_t)n);
    if (!rc) rc = dev_alloc(&m->urows, urows.size());
    if (!rc) rc = dev_alloc(&m->ptr, n ? ptr.size() : 0);
    if (!rc) rc = dev_alloc(&m->slots, (size_t)n);
    if (!rc) rc = copy_h2d(ctx, m->rows, rows, (size_t)n * 4);
    if (!rc) rc = copy_h2d(ctx, m->urows, urows.data(), urows.size() * 4);
    if (!rc && n) rc = copy_h2d(ctx, m->ptr, ptr.data(), ptr.size() * 4);
    if (!rc) rc = copy_h2d(ctx, m->slots, slots.data(), (size_t)n * 4);
    if (rc) {
        if (m->rows) (void)hipFree(m->rows);
        if (m->urows) (void)hipFree(m->urows);
        if (m->ptr) (void)hipFree(m->ptr);
        if (m->slots) (void)hipFree(m->slots);
        delete m;
        return rc;
    }
    m->magic = kMagicRowMap;
    *out = m;
    return SPC3D_OK;
}

int spc3d_rowmap_destroy(spc3d_rowmap *m)
{
    if (!live(m))
        return fail(SPC3D_ERR_INVALID_ARG, "row map is NULL or destroyed");
    if (int rc = refuse_while_capturing(m->ctx))
        return rc;
    (void)hipSetDevice(m->ctx->device);
    (void)hipStreamSynchronize(m->ctx->stream);
    if (m->rows) (void)hipFree(m->rows);
    if (m->urows) (void)hipFree(m->urows);
    if (m->ptr) (void)hipFree(m->ptr);
    if (m->slots) (void)hipFree(m->slots);
    m->magic = 0;
    delete m;
    return SPC3D_OK;
}

static int rows_op(int op, spc3d_ctx *ctx, const spc3d_panel *P, const spc3d_rowmap *map,
                   const spc3d_vals *buf)
{
    if (!live(ctx) || !live(P) || !live(map) || !live(buf))
        return fail(SPC3D_ERR_INVALID_ARG, "a handle is NULL or destroyed");
    if (P->ctx != ctx || map->ctx != ctx || buf->ctx != ctx)
        return fail(SPC3D_ERR_INVALID_ARG, "operands belong to different contexts");
    if (buf->dtype != P->dtype)
        return fail(SPC3D_ERR_SIZE_MISMATCH, "buffer dtype differs from the panel's");
    if (P->m < map->panel_rows)
        return fail(SPC3D_ERR_SIZE_MISMATCH, "panel has fewer rows than the row map was made for");
    if (buf->n < (uint64_t)map->nslots * P->n)
        return fail(SPC3D_ERR_SIZE_MISMATCH, "buffer holds fewer than n * K reals");
    int rc = use_device(ctx, true);
    if (rc)
        return rc;
    RowMapView v;
    v.rows = map->rows;
    v.urows = map->urows;
    v.ptr = map->ptr;
    v.slots = map->slots;
    v.nslots = map->nslots;
    v.nuniq = map->nuniq;
    HIP_TRY(launch_rows(op, P->dtype, P->dev, v, P->n, buf->dev, ctx->stream));
    return SPC3D_OK;
}

int spc3d_rows_pack(spc3d_ctx *ctx, const spc3d_panel *P, const spc3d_rowmap *map, spc3d_vals *buf)
{
    return rows_op(0, ctx, P, map, buf);
}

int spc3d_rows_unpack(spc3d_ctx *ctx, spc3d_panel *P, const spc3d_rowmap *map,
                      const spc3d_vals *buf)
{
    return rows_op(1, ctx, P, map, buf);
}

int spc3d_rows_unpack_sum(spc3d_ctx *ctx, spc3d_panel *P, const spc3d_rowmap *map,
                          const spc3d_vals *buf)
{
    return rows_op(2, ctx, P, map, buf);
}

} // extern "C"
