// C ABI of the local SDDMM / SpMM library (see include/spcomm3d_hip.h).
// Owns device memory for panels, value vectors and plans; launches the
// kernels of kernels.hip on the context's stream.  No CPU compute fallback:
// without a device every device call fails.
#include "../../include/spcomm3d_hip.h"

#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <atomic>
#include <condition_variable>
#include <cstring>
#include <functional>
#include <memory>
#include <mutex>
#include <thread>
#include <new>
#include <string>
#include <system_error>
#include <vector>

#include "host_cache.h"
#include "kernels.h"
#include "plan_device.h"
#include "plan_host.h"

using namespace spc3d;

namespace {

thread_local std::string g_err;

int fail(int status, const std::string &msg)
{
    g_err = msg;
    return status;
}

int fail_hip(hipError_t e, const char *what)
{
    g_err = std::string(what) + ": " + hipGetErrorString(e);
    if (e == hipErrorOutOfMemory)
        return SPC3D_ERR_ALLOC;
    if (e == hipErrorNoDevice || e == hipErrorInvalidDevice || e == hipErrorInsufficientDriver)
        return SPC3D_ERR_NO_DEVICE;
    return SPC3D_ERR_HIP;
}

#define HIP_TRY(expr)                                                                             \
    do {                                                                                          \
        hipError_t e_ = (expr);                                                                   \
        if (e_ != hipSuccess)                                                                     \
            return fail_hip(e_, #expr);                                                           \
    } while (0)

constexpr uint32_t kMagicCtx = 0x53433343;   // live handles carry a tag so that a
constexpr uint32_t kMagicPanel = 0x53433350; // stale or foreign pointer is refused
constexpr uint32_t kMagicVals = 0x53433356;  // instead of dereferenced further
constexpr uint32_t kMagicPlan = 0x5343334c;
constexpr uint32_t kMagicRowMap = 0x5343334d;
constexpr uint32_t kMagicGraph = 0x53433347;
constexpr int kTimerSlots = 4096;
constexpr uint32_t kMaxColBlocks = 4096;

inline size_t elem_size(int dtype) { return dtype == SPC3D_F64 ? 8 : 4; }
inline bool dtype_ok(int dtype) { return dtype == SPC3D_F32 || dtype == SPC3D_F64; }

} // namespace

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

// What the one-shot entry points over host memory keep between calls: plans by the
// content of the pattern, device panels with the keys of the host memory they mirror,
// and the result vector.  Defined after the handle types.
struct HostCallCache;

struct spc3d_ctx {
    uint32_t magic;
    int device;
    hipStream_t stream;
    hipStream_t aux_stream; // short-segment launches run here, beside the long-segment ones
    hipEvent_t fork_event, join_event;
    uint32_t aux_rot; // (XCD of workgroup 0 on aux - XCD of workgroup 0 on main) mod 8
    void *scratch;    // this device's copy of the static scratch array (spc3d_spmm_noalloc)
    bool capturing;   // between spc3d_capture_begin and spc3d_capture_end
    hipEvent_t timers[kTimerSlots];
    bool timer_set[kTimerSlots];
    HostCallCache *host_cache; // made by the first spc3d_*_host call
    bool use_host_cache;       // false: the one-shot calls keep nothing between calls
    unsigned host_threads;     // host threads a one-shot call may use, the caller's included
    std::mutex host_mutex;     // the one-shot calls of a context run one at a time
};

struct spc3d_panel {
    uint32_t magic;
    spc3d_ctx *ctx;
    int dtype;
    uint32_t m, n;
    void *dev;
    bool owned = true; // false: the caller's device memory (spc3d_panel_wrap)
};

struct spc3d_vals {
    uint32_t magic;
    spc3d_ctx *ctx;
    int dtype;
    uint64_t n;
    void *dev;
    bool owned = true; // false: the caller's device memory (spc3d_vals_wrap)
};

struct spc3d_rowmap {
    uint32_t magic;
    spc3d_ctx *ctx;
    uint32_t panel_rows;
    uint32_t nslots, nuniq;
    uint32_t *rows, *urows, *ptr, *slots; // device
};

struct spc3d_graph {
    uint32_t magic;
    spc3d_ctx *ctx;
    hipGraph_t graph;
    hipGraphExec_t exec;
};

struct spc3d_plan {
    uint32_t magic;
    spc3d_ctx *ctx;
    int dtype;
    spc3d_plan_info info;
    bool has_values;
    // device arrays
    Seg *segs;
    uint32_t *col;
    uint32_t *perm; // null when the caller's order is already the kernel order
    void *sval;     // values in kernel order
    SplitRow *splits;
    uint32_t *first_cols; // [(nsegments_padded - nsegments_long) * kFirstCols], see kernels.h
    void *partial; // [npartial_slots * partial_k] reals
    uint32_t partial_k;
    // Partial-sum blocks that a call at a larger K has replaced.  They stay allocated
    // until the plan is destroyed: a sequence recorded earlier (spc3d_capture_*) keeps
    // the block's address in its kernel arguments and goes on using it.
    std::vector<void *> retired_partial;
    uint64_t retired_bytes = 0;
    // A pattern kept in column blocks: one complete plan per block of columns, each over
    // the entries of its block with `perm` giving the caller's positions; this plan then
    // holds no arrays of its own, only `info` for the whole pattern.  The calls run the
    // blocks one after the other, so that one block of dense rows is what the L2s see at
    // a time.
    std::vector<spc3d_plan *> blocks;
    // SDDMM over blocks.  Stored straight at the caller's positions, the results of one
    // block are short runs between those of the other blocks, written at different times
    // (36 against 24 ms for the kernels on the 572 M-entry pattern the blocks are meant
    // for).  So the blocks write into a staging vector, and one pass brings the results
    // to the caller's positions, C[e] = c_stage[stage_pos[e]].  The staging order is by
    // tile of rows (about 2 MiB of results), inside a tile by block, inside a block the
    // block's kernel order: a block's stores are long runs, and the final pass reads one
    // tile's worth of staged results (L2-sized) while it writes that tile's C in order.
    // stage_of[g] = staging position of entry g of the blocks' concatenated kernel
    // orders; block b's part starts at stage_off.
    // A single plan whose kernel order regroups entries inside rows (hub rows cut by column
    // slice) stages the SDDMM results of those segments (build_store_staging): `store`
    // holds the positions, c_stage the store.n results.
    StoreStaging store;
    // SDDMM is symmetric in its two dense operands.  For a pattern handed over sorted by
    // column (the order of a MatrixMarket file), whose results in this plan's row-major
    // kernel order would each be stored to a place of its own, `by_col` is the plan of the
    // same entries with rows and columns exchanged: its kernel order is the caller's, and
    // spc3d_sddmm runs it with A and B exchanged (the same products summed in the same
    // order: the same bits).  SpMM and the one-pass call run this plan.
    spc3d_plan *by_col = nullptr;
    // An arbitrary entry order (no runs to store in this plan's kernel order): the kernels
    // write their results in kernel order into c_stage, and two tile-local passes through
    // c_mid bring them to the caller's positions (TwoPass in plan_device.h).  With `by_col`
    // this serves the one-pass call only.
    TwoPass two;
    void *c_mid = nullptr; // [nnz] reals
    void *c_stage = nullptr;       // [nnz] reals (column blocks, two passes), [store.n] (staged segments)
    uint32_t *stage_pos = nullptr; // [nnz] caller's position -> staging position
    uint32_t *stage_of = nullptr;  // [nnz]
    uint64_t stage_off = 0;
    uint32_t col_base = 0; // a block of a plan kept in column blocks: its first column
};

// A cached plan answers for a pattern when the keys of every block of ii and jj, the
// sizes, the type and the row width agree, and a sample of the indices read back equal.
struct CachedHostPlan {
    spc3d_plan *plan = nullptr;
    int dtype = 0;
    uint32_t nrows = 0, ncols = 0, k = 0;
    uint64_t nnz = 0;
    std::vector<BlockKey> key_ii, key_jj;
    std::vector<uint32_t> sample; // ii, jj at kSamples evenly spaced entries
    uint64_t last_use = 0;
};

// A device panel and the keys of the host memory it equals, block by block (the memory it
// was filled from, or the memory its content was fetched into).  No keys: the panel's
// content is not known to equal any host memory.
struct CachedHostPanel {
    spc3d_panel *panel = nullptr;
    std::vector<BlockKey> keys;
    const void *host = nullptr; // where it came from last: a preference among equals, never a proof
    uint64_t last_use = 0;
    // An operand the kernel changes (SpMM's Y): its result is fetched into the caller's
    // memory, so the two are equal again when the call returns, and the keys of what was
    // fetched let the next call leave in place what the caller did not touch.  When the
    // caller rewrites most of it between calls anyway, reading it for keys first is wasted:
    // the next `skip` calls send it unread, and each time that turns out right the stretch
    // doubles (to at most 16 calls).
    bool output = false;
    uint32_t skip = 0, backoff = 0;
};

struct HostCallCache {
    static constexpr size_t kMaxPlans = 4, kMaxPanels = 6, kSamples = 64;
    std::vector<CachedHostPlan> plans;
    std::vector<std::unique_ptr<CachedHostPanel>> panels; // the objects stay where they are
    spc3d_vals *c = nullptr;
    uint64_t clock = 0;
    // what the last call did, for spc3d_host_call_stats
    uint64_t bytes_sent = 0, bytes_kept = 0;
    int plan_reused = 0;
};

namespace {

bool live(const spc3d_ctx *c) { return c && c->magic == kMagicCtx; }
bool live(const spc3d_panel *p) { return p && p->magic == kMagicPanel && live(p->ctx); }
bool live(const spc3d_vals *v) { return v && v->magic == kMagicVals && live(v->ctx); }
bool live(const spc3d_plan *p) { return p && p->magic == kMagicPlan && live(p->ctx); }
bool live(const spc3d_rowmap *p) { return p && p->magic == kMagicRowMap && live(p->ctx); }

bool live(const spc3d_graph *g) { return g && g->magic == kMagicGraph && live(g->ctx); }

// Makes the context's device current.  While the context records a graph only the
// calls that merely queue kernels may run (capturable); everything that allocates,
// copies to or from the host or waits is refused.
int use_device(const spc3d_ctx *ctx, bool capturable = false)
{
    if (ctx->capturing && !capturable)
        return fail(SPC3D_ERR_INVALID_ARG,
                    "this call allocates, copies or waits: not allowed between "
                    "spc3d_capture_begin and spc3d_capture_end");
    HIP_TRY(hipSetDevice(ctx->device));
    return SPC3D_OK;
}

template <typename T> int dev_alloc(T **out, size_t count)
{
    *out = nullptr;
    if (count == 0)
        return SPC3D_OK;
    if (count > SIZE_MAX / sizeof(T))
        return fail(SPC3D_ERR_TOO_LARGE, "allocation size overflows");
    HIP_TRY(hipMalloc((void **)out, count * sizeof(T)));
    return SPC3D_OK;
}

int dev_alloc_bytes(void **out, size_t bytes)
{
    *out = nullptr;
    if (bytes == 0)
        return SPC3D_OK;
    HIP_TRY(hipMalloc(out, bytes));
    return SPC3D_OK;
}

// Pageable-host <-> device copy ordered after everything queued on the
// stream; returns when the host side may be reused / read.
int copy_h2d(spc3d_ctx *ctx, void *dst, const void *src, size_t bytes)
{
    if (bytes == 0)
        return SPC3D_OK;
    HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, ctx->stream));
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    return SPC3D_OK;
}

int copy_d2h(spc3d_ctx *ctx, void *dst, const void *src, size_t bytes)
{
    if (bytes == 0)
        return SPC3D_OK;
    HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, ctx->stream));
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    return SPC3D_OK;
}

void plan_free_device(spc3d_plan *p)
{
    if (p->segs) (void)hipFree(p->segs);
    if (p->col) (void)hipFree(p->col);
    if (p->perm) (void)hipFree(p->perm);
    if (p->sval) (void)hipFree(p->sval);
    if (p->splits) (void)hipFree(p->splits);
    if (p->first_cols) (void)hipFree(p->first_cols);
    if (p->store.perm2) (void)hipFree(p->store.perm2);
    if (p->store.dst) (void)hipFree(p->store.dst);
    if (p->store.src) (void)hipFree(p->store.src);
    if ((p->store.n || p->two.n) && p->c_stage) {
        (void)hipFree(p->c_stage);
        p->c_stage = nullptr;
    }
    p->store = StoreStaging();
    if (p->two.l1) (void)hipFree(p->two.l1);
    if (p->two.dst1) (void)hipFree(p->two.dst1);
    if (p->two.l2) (void)hipFree(p->two.l2);
    if (p->c_mid) (void)hipFree(p->c_mid);
    p->two = TwoPass();
    p->c_mid = nullptr;
    if (p->partial) (void)hipFree(p->partial);
    for (void *old : p->retired_partial)
        (void)hipFree(old);
    p->retired_partial.clear();
    p->retired_bytes = 0;
    p->segs = nullptr;
    p->col = p->perm = nullptr;
    p->sval = p->partial = nullptr;
    p->splits = nullptr;
    p->first_cols = nullptr;
}

Streams streams_of(const spc3d_ctx *c)
{
    Streams s;
    s.main = c->stream;
    s.aux = c->aux_stream;
    s.fork = c->fork_event;
    s.join = c->join_event;
    s.aux_rot = c->aux_rot;
    return s;
}

DevPlanView view_of(const spc3d_plan *p)
{
    DevPlanView v;
    v.segs = p->segs;
    v.nseg = p->info.nsegments_padded;
    v.nseg_long = p->info.nsegments_long;
    v.nqueues = p->info.nqueues;
    v.col = p->col;
    v.perm = p->perm;
    v.sval = p->sval;
    v.splits = p->splits;
    v.nsplit = p->info.nsplit_rows;
    v.partial = p->partial;
    v.first_cols = p->first_cols;
    v.nnz = p->info.nnz;
    v.seg_base = p->store.consecutive;
    if (p->two.n)
        v.perm = nullptr; // results in kernel order (into c_stage, see sddmm_out)
    if (p->store.n) {
        v.perm = p->store.perm2;
        v.stage = p->c_stage;
        v.stage_from = (uint32_t)p->info.nnz;
    }
    return v;
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
static bool env_number(const char *name, unsigned long long *out);

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

static int refuse_while_capturing(const spc3d_ctx *ctx)
{
    if (ctx->capturing)
        return fail(SPC3D_ERR_INVALID_ARG,
                    "not allowed between spc3d_capture_begin and spc3d_capture_end");
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

static bool ranges_overlap(const void *a, size_t abytes, const void *b, size_t bbytes);

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

/* ---- plan ---------------------------------------------------------------- */
int spc3d_coo_validate(uint32_t nrows, uint32_t ncols, uint64_t nnz, const uint32_t *ii,
                       const uint32_t *jj)
{
    std::string err;
    int rc = validate_coo(nrows, ncols, nnz, ii, jj, err);
    return rc == SPC3D_OK ? rc : fail(rc, err);
}

static void fill_info(spc3d_plan_info &info, const HostPlan &H)
{
    info.nrows = H.nrows;
    info.ncols = H.ncols;
    info.nnz = H.nnz;
    info.rows_touched = H.rows_touched;
    info.cols_touched = H.cols_touched;
    info.nsegments = H.nseg_real;
    info.nsegments_padded = (uint32_t)H.segs.size();
    info.nsplit_rows = (uint32_t)H.splits.size();
    info.npartial_slots = H.nslots;
    info.max_row_nnz = H.max_row_nnz;
    info.seg_max = H.seg_max;
    info.order_is_identity = H.identity ? 1 : 0;
    info.nqueues = H.nqueues;
    info.hot_cols = H.hot_cols;
    info.hub_rows = H.hub_rows;
    info.hot_entries = H.hot_entries;
    info.nsegments_long = H.nseg_long;
    info.ncol_blocks = 1;
    info.staged_entries = 0;
    info.positions_by_segment = 0;
    info.sddmm_by_column = 0;
    info.two_pass_results = 0;
    info.entries_by_column = H.by_column_in_rows ? 1 : 0;
    info.device_bytes = 0;
}

// Library defaults, overridable field by field.  With XCD slicing, 2 MiB of
// each 4 MiB L2 is planned for dense rows, the rest is left to everything else.
static int resolve_opts(int dtype, const spc3d_plan_opts *o, PlanOpts &out)
{
    spc3d_plan_opts z;
    std::memset(&z, 0, sizeof z);
    if (o)
        z = *o;
    if (z.reserved[0] || z.reserved[1] || z.reserved[2])
        return fail(SPC3D_ERR_INVALID_ARG, "spc3d_plan_opts.reserved must be 0");
    if (z.flags & ~(uint32_t)SPC3D_PLAN_ALL_FLAGS)
        return fail(SPC3D_ERR_INVALID_ARG, "spc3d_plan_opts.flags has unknown bits set");
    if (z.col_blocks > kMaxColBlocks)
        return fail(SPC3D_ERR_INVALID_ARG, "spc3d_plan_opts.col_blocks must be at most 4096");
    if (z.col_blocks > 1 && z.builder == 1)
        return fail(SPC3D_ERR_INVALID_ARG,
                    "column blocks are built on the GPU: builder must be 0 or 2 with col_blocks > 1");
    if (z.builder > 2)
        return fail(SPC3D_ERR_INVALID_ARG, "spc3d_plan_opts.builder must be 0, 1 or 2");
    if (z.xcd_slices != 0 && z.xcd_slices != 1 && z.xcd_slices != 8)
        return fail(SPC3D_ERR_INVALID_ARG, "xcd_slices must be 0, 1 or 8");
    out.seg_max = z.seg_max;
    out.keep_entry_order = (z.flags & SPC3D_PLAN_KEEP_ENTRY_ORDER) != 0;
    out.hub_min = z.hub_min;
    out.xcd_slices = z.xcd_slices;
    const uint64_t k = z.k_hint ? z.k_hint : 64;
    const uint64_t bytes = z.l2_hot_bytes ? z.l2_hot_bytes : 2u << 20;
    out.hot_cols = (uint32_t)(bytes / (k * elem_size(dtype)));
    out.row_bytes = (uint32_t)std::min<uint64_t>((uint64_t)z.k_hint * elem_size(dtype), 1u << 30);
    return SPC3D_OK;
}

int spc3d_plan_build_host(int dtype, uint32_t nrows, uint32_t ncols, uint64_t nnz,
                          const uint32_t *ii, const uint32_t *jj, const spc3d_plan_opts *opts,
                          spc3d_plan_info *info, uint32_t *col, uint32_t *perm, uint32_t *segs,
                          uint32_t seg_cap, uint32_t *splits, uint32_t split_cap)
{
    if (!info)
        return fail(SPC3D_ERR_INVALID_ARG, "info is NULL");
    if (!dtype_ok(dtype))
        return fail(SPC3D_ERR_INVALID_ARG, "unknown dtype");
    PlanOpts po;
    int rc = resolve_opts(dtype, opts, po);
    if (rc)
        return rc;
    HostPlan H;
    std::string err;
    rc = build_host_plan(nrows, ncols, nnz, ii, jj, po, H, err);
    if (rc != SPC3D_OK)
        return fail(rc, err);
    fill_info(*info, H);
    if ((segs && seg_cap < H.segs.size()) || (splits && split_cap < H.splits.size()))
        return fail(SPC3D_ERR_SIZE_MISMATCH, "output capacity is smaller than the plan");
    if (col && nnz)
        std::memcpy(col, H.col.data(), (size_t)nnz * sizeof(uint32_t));
    if (perm && nnz)
        std::memcpy(perm, H.perm.data(), (size_t)nnz * sizeof(uint32_t));
    if (segs && !H.segs.empty())
        std::memcpy(segs, H.segs.data(), H.segs.size() * sizeof(Seg));
    if (splits)
        for (size_t i = 0; i < H.splits.size(); ++i) {
            splits[3 * i + 0] = H.splits[i].row;
            splits[3 * i + 1] = H.splits[i].first_slot;
            splits[3 * i + 2] = H.splits[i].nslots;
        }
    return SPC3D_OK;
}

static int ensure_partial(spc3d_plan *p, uint32_t K);

// What a plan holds beside the builders' arrays: the table of first column indices of
// its short segments (read by the short-segment launch next to the descriptors) and
// the partial-sum rows of its cut rows for k0 columns.
static int finish_plan(spc3d_plan *p, uint32_t k0)
{
    const uint32_t nshort = p->info.nsegments_padded - p->info.nsegments_long;
    int rc = dev_alloc(&p->first_cols, (size_t)nshort * kFirstCols);
    if (rc)
        return rc;
    HIP_TRY(launch_first_cols(p->segs + p->info.nsegments_long, nshort, p->col, p->first_cols,
                              p->ctx->stream));
    return ensure_partial(p, k0);
}

// How a plan may bring SDDMM results to the caller's positions (spc3d_plan_opts.flags,
// two_pass_min): each of the three forms can be switched off, which keeps the plain stores.
struct StoreOpts {
    bool stage = true, by_column = true, two_pass = true;
    // measured on R-MAT patterns: two passes are slower at 0.95 M entries, faster at 1.9 M
    uint64_t two_pass_min = 3ull << 19;
};
static StoreOpts store_opts_of(const spc3d_plan_opts *o)
{
    StoreOpts so;
    if (o) {
        so.stage = !(o->flags & SPC3D_PLAN_NO_STAGED_STORES);
        so.by_column = !(o->flags & SPC3D_PLAN_NO_SDDMM_BY_COLUMN);
        so.two_pass = !(o->flags & SPC3D_PLAN_NO_TWO_PASS);
        if (o->two_pass_min)
            so.two_pass_min = o->two_pass_min;
    }
    return so;
}

// The result paths below are optional: when one of them cannot get its memory the plan
// goes on without it (plain stores), what it had allocated is freed by its builder, and the
// HIP error state is cleared.  Any other failure fails the plan.
static int optional_path(int rc)
{
    if (rc != SPC3D_ERR_ALLOC)
        return rc;
    (void)hipGetLastError();
    return SPC3D_OK;
}

// A finished single plan (not a block of a plan kept in column blocks) whose kernel order
// regroups entries inside rows gets the staging of its SDDMM results (see StoreStaging).
// SPC3D_PLAN_NO_STAGED_STORES keeps every result on its way straight to C.
static int add_store_staging(spc3d_plan *p, const StoreOpts &so)
{
    if (!so.stage || !p->perm || !p->blocks.empty())
        return SPC3D_OK;
    std::string err;
    StoreStaging st;
    int rc = build_store_staging(p->ctx->stream, p->segs, p->info.nsegments_padded, p->perm,
                                 p->info.nnz, st, err);
    if (rc)
        return optional_path(fail(rc, err));
    p->store.consecutive = st.consecutive;
    p->info.positions_by_segment = st.consecutive ? 1 : 0;
    if (!st.n)
        return SPC3D_OK;
    rc = dev_alloc_bytes(&p->c_stage, (size_t)st.n * elem_size(p->dtype));
    if (rc) {
        (void)hipFree(st.perm2);
        (void)hipFree(st.dst);
        (void)hipFree(st.src);
        p->store = StoreStaging();
        p->info.positions_by_segment = 0;
        return optional_path(rc);
    }
    p->store = st;
    p->info.staged_entries = st.n;
    return SPC3D_OK;
}

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

// The two-pass tables of a finished single plan whose results would each be a store of its
// own (an arbitrary entry order), from StoreOpts::two_pass_min entries on: below that the
// scattered stores mostly meet in the L2s.  SPC3D_PLAN_NO_TWO_PASS switches it off.
static int add_two_pass(spc3d_plan *p, const StoreOpts &so)
{
    if (!so.two_pass || !p->perm || p->store.consecutive || !p->blocks.empty() ||
        p->info.nnz < so.two_pass_min)
        return SPC3D_OK;
    int lds = 0;
    if (hipDeviceGetAttribute(&lds, hipDeviceAttributeMaxSharedMemoryPerBlock, p->ctx->device) !=
            hipSuccess ||
        lds < (int)two_pass_lds_bytes())
        return SPC3D_OK;
    std::string err;
    TwoPass tp;
    int rc = build_two_pass(p->ctx->stream, p->perm, p->info.nnz, two_pass_tile_elems(p->dtype), tp,
                            err);
    if (rc)
        return optional_path(fail(rc, err));
    if (!tp.n)
        return SPC3D_OK;
    const size_t bytes = (size_t)p->info.nnz * elem_size(p->dtype);
    rc = dev_alloc_bytes(&p->c_stage, bytes);
    if (!rc) rc = dev_alloc_bytes(&p->c_mid, bytes);
    if (rc) {
        (void)hipFree(tp.l1);
        (void)hipFree(tp.dst1);
        (void)hipFree(tp.l2);
        if (p->c_stage) (void)hipFree(p->c_stage);
        p->c_stage = nullptr;
        return optional_path(rc);
    }
    p->two = tp;
    p->info.two_pass_results = 1;
    return SPC3D_OK;
}

// Row width a plan is created for: sizes the partial-sum rows of its cut rows.
static uint32_t planned_k(const spc3d_plan_opts *o) { return o && o->k_hint ? o->k_hint : 64u; }

// Plan over arrays that build_device_plan left on the device.
static int adopt_device_plan(spc3d_ctx *ctx, int dtype, const HostPlan &meta, DevPlanArrays &arr,
                             uint32_t k0, spc3d_plan **out)
{
    spc3d_plan *p = new (std::nothrow) spc3d_plan();
    int rc = SPC3D_OK;
    if (!p)
        rc = fail(SPC3D_ERR_ALLOC, "host allocation failed");
    if (!rc) {
        p->ctx = ctx;
        p->dtype = dtype;
        fill_info(p->info, meta);
        p->info.nsegments_padded = arr.nseg_padded;
        p->info.nsplit_rows = arr.nsplit;
        rc = dev_alloc_bytes(&p->sval, (size_t)meta.nnz * elem_size(dtype));
    }
    if (rc) {
        if (arr.segs) (void)hipFree(arr.segs);
        if (arr.col) (void)hipFree(arr.col);
        if (arr.perm) (void)hipFree(arr.perm);
        if (arr.splits) (void)hipFree(arr.splits);
        delete p;
        return rc;
    }
    p->segs = arr.segs;
    p->col = arr.col;
    p->perm = arr.perm;
    p->splits = arr.splits;
    arr = DevPlanArrays{};
    rc = finish_plan(p, k0);
    if (rc) {
        plan_free_device(p);
        delete p;
        return rc;
    }
    p->magic = kMagicPlan;
    *out = p;
    return SPC3D_OK;
}

static void destroy_blocks(spc3d_plan *p)
{
    for (spc3d_plan *b : p->blocks) {
        plan_free_device(b);
        b->magic = 0;
        delete b;
    }
    p->blocks.clear();
    if (p->c_stage) (void)hipFree(p->c_stage);
    if (p->stage_pos) (void)hipFree(p->stage_pos);
    if (p->stage_of) (void)hipFree(p->stage_of);
    p->c_stage = nullptr;
    p->stage_pos = p->stage_of = nullptr;
}

// How many column blocks a finished single plan should be rebuilt in (1: keep it).
// Blocks pay when the dense rows the pattern gathers do not fit the L2s, the columns
// are not skewed (then a few hot rows carry the reuse, and the plan deals them to the
// XCDs instead), and the rows are long enough that a row's piece in one block still
// amortises reading its A row / updating its Y row: the entry-weighted mean segment
// length divided by the block count must stay at 16 or more.  Measured on a 2 M x 500 k
// pattern with 286 entries per row on average (capped Zipf, weighted mean 890) at 512-byte
// dense rows: 43 -> 24 ms SDDMM, 42 -> 27 ms SpMM in 48 blocks of 5 MiB; a uniform
// pattern of 256 entries per row gains 10 % in SDDMM and loses in SpMM, and stays whole.
static int choose_col_blocks(spc3d_plan *p, const spc3d_plan_opts *opts, uint32_t *nblocks)
{
    *nblocks = 1;
    const uint32_t want = opts ? opts->col_blocks : 0;
    const spc3d_plan_info &I = p->info;
    if (want == 1 || I.nnz == 0 || I.ncols < 2)
        return SPC3D_OK;
    if (want > 1) {
        *nblocks = std::min<uint32_t>(want, I.ncols);
        return SPC3D_OK;
    }
    if (I.nqueues != 1)
        return SPC3D_OK;
    const uint64_t row_bytes = (uint64_t)planned_k(opts) * elem_size(p->dtype);
    const uint64_t panel = (uint64_t)I.cols_touched * row_bytes;
    constexpr uint64_t kBlockBytes = (uint64_t)21 << 18; // 5.25 MiB of dense rows per block
    if (panel < ((uint64_t)64 << 20))
        return SPC3D_OK;
    const uint64_t nb = std::min<uint64_t>((panel + kBlockBytes - 1) / kBlockBytes, 256);
    uint64_t sumsq = 0;
    std::string err;
    int rc = sum_sq_seg_len_device(p->ctx->stream, p->segs, I.nsegments_padded, &sumsq, err);
    if (rc != SPC3D_OK)
        return fail(rc, err);
    const double wmean = (double)sumsq / (double)I.nnz;
    if (wmean / (double)nb >= 16.0)
        *nblocks = (uint32_t)nb;
    return SPC3D_OK;
}

// The companion plan for SDDMM (spc3d_plan::by_col) of a finished single plan whose results
// would be stored one by one, when the pattern is sorted by column and the exchanged plan
// does store in runs.  SPC3D_PLAN_NO_SDDMM_BY_COLUMN switches it off.
static int add_sddmm_companion(spc3d_plan *p, uint32_t nrows, uint32_t ncols, uint64_t nnz,
                               const uint32_t *d_ii, const uint32_t *d_jj, const PlanOpts &po,
                               const StoreOpts &so)
{
    if (!so.by_column || nnz < 2 || !p->perm || p->store.consecutive || !p->blocks.empty())
        return SPC3D_OK;
    std::string err;
    bool sorted = false;
    int rc = is_nondecreasing_device(p->ctx->stream, d_jj, nnz, &sorted, err);
    if (rc)
        return fail(rc, err);
    if (!sorted)
        return SPC3D_OK;
    HostPlan meta;
    DevPlanArrays arr;
    rc = build_device_plan(p->ctx->stream, ncols, nrows, nnz, d_jj, d_ii, po, meta, arr, err);
    if (rc)
        return optional_path(fail(rc, err));
    spc3d_plan *q = nullptr;
    rc = adopt_device_plan(p->ctx, p->dtype, meta, arr, 0 /* never runs SpMM */, &q);
    if (!rc)
        rc = add_store_staging(q, so);
    if (rc || (q->perm && !q->store.consecutive)) { // no better than what there is
        if (q) {
            const std::string keep = g_err;
            plan_free_device(q);
            q->magic = 0;
            delete q;
            if (rc)
                return optional_path(fail(rc, keep));
        }
        return optional_path(rc);
    }
    p->by_col = q;
    p->info.sddmm_by_column = 1;
    return SPC3D_OK;
}

// Plan of a pattern that lies on the device: the single plan first (validation, the
// whole pattern's figures), then, where choose_col_blocks says so, one plan per block
// of columns in its place.
static int build_from_device(spc3d_ctx *ctx, int dtype, uint32_t nrows, uint32_t ncols,
                             uint64_t nnz, const uint32_t *d_ii, const uint32_t *d_jj,
                             const PlanOpts &po, const spc3d_plan_opts *opts, spc3d_plan **out)
{
    HostPlan meta;
    DevPlanArrays arr;
    std::string err;
    int rc = build_device_plan(ctx->stream, nrows, ncols, nnz, d_ii, d_jj, po, meta, arr, err);
    if (rc != SPC3D_OK)
        return fail(rc, err);
    spc3d_plan *p = nullptr;
    rc = adopt_device_plan(ctx, dtype, meta, arr, planned_k(opts), &p);
    if (rc)
        return rc;
    uint32_t nb = 1;
    const StoreOpts so = store_opts_of(opts);
    rc = choose_col_blocks(p, opts, &nb);
    if (!rc && nb <= 1)
        rc = add_store_staging(p, so);
    if (!rc && nb <= 1)
        rc = add_sddmm_companion(p, nrows, ncols, nnz, d_ii, d_jj, po, so);
    if (!rc && nb <= 1)
        rc = add_two_pass(p, so);
    if (rc || nb <= 1) {
        if (rc) {
            const std::string keep = g_err;
            spc3d_plan_destroy(p);
            return fail(rc, keep);
        }
        *out = p;
        return rc;
    }
    // ---- in column blocks ----
    uint32_t *b_ii = nullptr, *b_jj = nullptr, *order = nullptr;
    std::vector<uint32_t> first;
    try {
        first.resize((size_t)nb + 1);
        p->blocks.reserve(nb);
    } catch (const std::bad_alloc &) {
        spc3d_plan_destroy(p);
        return fail(SPC3D_ERR_ALLOC, "host allocation failed");
    }
    rc = dev_alloc(&b_ii, (size_t)nnz);
    if (!rc) rc = dev_alloc(&b_jj, (size_t)nnz);
    if (!rc) rc = dev_alloc(&order, (size_t)nnz);
    if (!rc) {
        rc = partition_by_col_block(ctx->stream, nnz, d_ii, d_jj, ncols, nb, b_ii, b_jj, order,
                                    first.data(), err);
        if (rc)
            fail(rc, err);
    }
    // rows per tile of the staging order: about 2 MiB of results
    const uint64_t per_row = std::max<uint64_t>(1, nnz / std::max<uint32_t>(1, p->info.rows_touched));
    const uint32_t rows_per_tile = (uint32_t)std::max<uint64_t>(
        1, ((uint64_t)2 << 20) / (per_row * elem_size(dtype)));
    uint32_t *tile_key = nullptr;
    if (!rc) rc = dev_alloc(&tile_key, (size_t)nnz);
    spc3d_plan_info total = p->info;
    total.nsegments = total.nsegments_padded = total.nsplit_rows = total.npartial_slots = 0;
    total.nsegments_long = 0;
    total.order_is_identity = 0;
    for (uint32_t b = 0; !rc && b < nb; ++b) {
        const uint64_t cnt = (uint64_t)first[b + 1] - first[b];
        if (cnt == 0)
            continue;
        HostPlan bmeta;
        DevPlanArrays barr;
        rc = build_device_plan(ctx->stream, nrows, ncols, cnt, b_ii + first[b], b_jj + first[b], po,
                               bmeta, barr, err);
        if (rc) {
            fail(rc, err);
            break;
        }
        spc3d_plan *child = nullptr;
        rc = adopt_device_plan(ctx, dtype, bmeta, barr, planned_k(opts), &child);
        if (rc)
            break;
        p->blocks.push_back(child);
        rc = tile_keys_device(ctx->stream, b_ii + first[b], child->perm, cnt, rows_per_tile,
                              tile_key + first[b], err);
        if (rc) {
            fail(rc, err);
            break;
        }
        uint32_t *gperm = nullptr;
        rc = dev_alloc(&gperm, (size_t)cnt);
        if (!rc) {
            rc = compose_perm_device(ctx->stream, order + first[b], child->perm, cnt, gperm, err);
            if (rc)
                fail(rc, err);
        }
        if (rc) {
            if (gperm) (void)hipFree(gperm);
            break;
        }
        hipError_t e = hipStreamSynchronize(ctx->stream); // child->perm is read until here
        if (e != hipSuccess) {
            (void)hipFree(gperm);
            rc = fail_hip(e, "hipStreamSynchronize");
            break;
        }
        if (child->perm) (void)hipFree(child->perm);
        child->perm = gperm;
        child->stage_off = first[b];
        child->col_base = b * ((ncols + nb - 1) / nb);
        child->info.order_is_identity = 0;
        total.nsegments += child->info.nsegments;
        total.nsegments_padded += child->info.nsegments_padded;
        total.nsegments_long += child->info.nsegments_long;
        total.nsplit_rows += child->info.nsplit_rows;
        total.npartial_slots = std::max(total.npartial_slots, child->info.npartial_slots);
        total.nqueues = std::max(total.nqueues, child->info.nqueues);
    }
    if (!rc) rc = dev_alloc_bytes(&p->c_stage, (size_t)nnz * elem_size(dtype));
    if (!rc) rc = dev_alloc(&p->stage_pos, (size_t)nnz);
    if (!rc) rc = dev_alloc(&p->stage_of, (size_t)nnz);
    if (!rc) {
        rc = stable_ranks_device(ctx->stream, tile_key, nnz, (nrows - 1) / rows_per_tile,
                                 p->stage_of, err);
        if (rc)
            fail(rc, err);
    }
    for (spc3d_plan *child : p->blocks) {
        if (rc)
            break;
        // stage_pos[caller's position of entry q] = its staging position
        rc = scatter_device(ctx->stream, child->perm, p->stage_of + child->stage_off,
                            child->info.nnz, p->stage_pos, err);
        if (rc)
            fail(rc, err);
    }
    if (tile_key) (void)hipFree(tile_key);
    if (b_ii) (void)hipFree(b_ii);
    if (b_jj) (void)hipFree(b_jj);
    if (order) (void)hipFree(order);
    if (rc) {
        std::string keep = g_err;
        spc3d_plan_destroy(p);
        return fail(rc, keep);
    }
    // the whole pattern's arrays give way to the blocks'
    (void)hipStreamSynchronize(ctx->stream);
    plan_free_device(p);
    p->partial_k = 0;
    p->info = total;
    p->info.ncol_blocks = (uint32_t)p->blocks.size();
    *out = p;
    return SPC3D_OK;
}

int spc3d_plan_create_from_device(spc3d_ctx *ctx, int dtype, uint32_t nrows, uint32_t ncols,
                                  uint64_t nnz, const void *dev_ii, const void *dev_jj,
                                  const spc3d_plan_opts *opts, spc3d_plan **out)
{
    if (!out)
        return fail(SPC3D_ERR_INVALID_ARG, "out is NULL");
    *out = nullptr;
    if (!dtype_ok(dtype))
        return fail(SPC3D_ERR_INVALID_ARG, "unknown dtype");
    PlanOpts po;
    int rc = resolve_opts(dtype, opts, po);
    if (rc)
        return rc;
    if (!live(ctx))
        return fail(SPC3D_ERR_INVALID_ARG, "context is NULL or destroyed");
    rc = use_device(ctx);
    if (rc)
        return rc;
    return build_from_device(ctx, dtype, nrows, ncols, nnz, (const uint32_t *)dev_ii,
                             (const uint32_t *)dev_jj, po, opts, out);
}

int spc3d_plan_create_ex(spc3d_ctx *ctx, int dtype, uint32_t nrows, uint32_t ncols, uint64_t nnz,
                         const uint32_t *ii, const uint32_t *jj, const void *vv,
                         const spc3d_plan_opts *opts, spc3d_plan **out)
{
    if (!out)
        return fail(SPC3D_ERR_INVALID_ARG, "out is NULL");
    *out = nullptr;
    if (!dtype_ok(dtype))
        return fail(SPC3D_ERR_INVALID_ARG, "unknown dtype");
    PlanOpts po;
    int rc = resolve_opts(dtype, opts, po);
    if (rc)
        return rc;
    const bool on_host = opts && opts->builder == 1;
    spc3d_plan *p = nullptr;
    if (!on_host && live(ctx)) {
        if (nnz > 0 && (ii == nullptr || jj == nullptr))
            return fail(SPC3D_ERR_INVALID_ARG, "ii/jj is NULL with nnz > 0");
        if (nnz >= (1ull << 32))
            return fail(SPC3D_ERR_TOO_LARGE, "nnz >= 2^32 is not supported");
        rc = use_device(ctx);
        if (rc)
            return rc;
        // The pattern goes up as it is; validation and everything else happens there.
        uint32_t *d_ii = nullptr, *d_jj = nullptr;
        rc = dev_alloc(&d_ii, (size_t)nnz);
        if (!rc) rc = dev_alloc(&d_jj, (size_t)nnz);
        if (!rc) rc = copy_h2d(ctx, d_ii, ii, (size_t)nnz * sizeof(uint32_t));
        if (!rc) rc = copy_h2d(ctx, d_jj, jj, (size_t)nnz * sizeof(uint32_t));
        if (!rc)
            rc = build_from_device(ctx, dtype, nrows, ncols, nnz, d_ii, d_jj, po, opts, &p);
        if (d_ii) (void)hipFree(d_ii);
        if (d_jj) (void)hipFree(d_jj);
        if (rc)
            return rc;
    } else {
        // The pattern is checked before the device is touched, so that a bad
        // index is reported as such on a machine without a GPU as well.
        HostPlan H;
        std::string err;
        rc = build_host_plan(nrows, ncols, nnz, ii, jj, po, H, err);
        if (rc != SPC3D_OK)
            return fail(rc, err);
        if (!live(ctx))
            return fail(SPC3D_ERR_INVALID_ARG, "context is NULL or destroyed");
        rc = use_device(ctx);
        if (rc)
            return rc;

        p = new (std::nothrow) spc3d_plan();
        if (!p)
            return fail(SPC3D_ERR_ALLOC, "host allocation failed");
        p->ctx = ctx;
        p->dtype = dtype;
        fill_info(p->info, H);

        rc = dev_alloc(&p->segs, H.segs.size());
        if (!rc) rc = dev_alloc(&p->col, (size_t)nnz);
        if (!rc && !H.identity) rc = dev_alloc(&p->perm, (size_t)nnz);
        if (!rc) rc = dev_alloc_bytes(&p->sval, (size_t)nnz * elem_size(dtype));
        if (!rc) rc = dev_alloc(&p->splits, H.splits.size());
        if (!rc) rc = copy_h2d(ctx, p->segs, H.segs.data(), H.segs.size() * sizeof(Seg));
        if (!rc) rc = copy_h2d(ctx, p->col, H.col.data(), (size_t)nnz * sizeof(uint32_t));
        if (!rc && !H.identity)
            rc = copy_h2d(ctx, p->perm, H.perm.data(), (size_t)nnz * sizeof(uint32_t));
        if (!rc)
            rc = copy_h2d(ctx, p->splits, H.splits.data(), H.splits.size() * sizeof(SplitRow));
        if (!rc)
            rc = finish_plan(p, planned_k(opts));
        if (!rc)
            rc = add_store_staging(p, store_opts_of(opts));
        if (!rc)
            rc = add_two_pass(p, store_opts_of(opts));
        if (rc) {
            plan_free_device(p);
            delete p;
            return rc;
        }
        p->magic = kMagicPlan;
    }
    if (vv) {
        rc = spc3d_plan_set_values(p, vv);
        if (rc) {
            std::string keep = g_err;
            spc3d_plan_destroy(p);
            return fail(rc, keep);
        }
    }
    *out = p;
    return SPC3D_OK;
}

int spc3d_localize_device(spc3d_ctx *ctx, uint64_t n, void *dev_idx, void *dev_ltg,
                          uint32_t *nlocal)
{
    if (!live(ctx) || !nlocal)
        return fail(SPC3D_ERR_INVALID_ARG, "context or nlocal is NULL");
    *nlocal = 0;
    if (n && (!dev_idx || !dev_ltg))
        return fail(SPC3D_ERR_INVALID_ARG, "index or map pointer is NULL");
    int rc = use_device(ctx);
    if (rc)
        return rc;
    std::string err;
    rc = localize_device(ctx->stream, n, (uint32_t *)dev_idx, (uint32_t *)dev_ltg, nlocal, err);
    return rc == SPC3D_OK ? rc : fail(rc, err);
}

int spc3d_remap_device(spc3d_ctx *ctx, uint64_t n, void *dev_idx, const void *dev_map,
                       uint32_t map_len)
{
    if (!live(ctx))
        return fail(SPC3D_ERR_INVALID_ARG, "context is NULL or destroyed");
    if (n && (!dev_idx || (!dev_map && map_len)))
        return fail(SPC3D_ERR_INVALID_ARG, "index or map pointer is NULL");
    int rc = use_device(ctx);
    if (rc)
        return rc;
    std::string err;
    rc = remap_device(ctx->stream, n, (uint32_t *)dev_idx, (const uint32_t *)dev_map, map_len,
                      err);
    return rc == SPC3D_OK ? rc : fail(rc, err);
}

int spc3d_plan_download(spc3d_plan *plan, uint32_t *col, uint32_t *perm, uint32_t *segs,
                        uint32_t seg_cap, uint32_t *splits, uint32_t split_cap)
{
    if (!live(plan))
        return fail(SPC3D_ERR_INVALID_ARG, "plan is NULL or destroyed");
    const spc3d_plan_info &I = plan->info;
    if (!plan->blocks.empty())
        return fail(SPC3D_ERR_INVALID_ARG,
                    "the plan is kept in column blocks (spc3d_plan_info.ncol_blocks > 1): there "
                    "is one set of arrays per block, not one for the pattern");
    if ((segs && seg_cap < I.nsegments_padded) || (splits && split_cap < I.nsplit_rows))
        return fail(SPC3D_ERR_SIZE_MISMATCH, "output capacity is smaller than the plan");
    int rc = use_device(plan->ctx);
    if (rc)
        return rc;
    const size_t nnz = (size_t)I.nnz;
    if (col && nnz)
        rc = copy_d2h(plan->ctx, col, plan->col, nnz * sizeof(uint32_t));
    if (!rc && perm && nnz) {
        if (plan->perm)
            rc = copy_d2h(plan->ctx, perm, plan->perm, nnz * sizeof(uint32_t));
        else
            for (size_t e = 0; e < nnz; ++e)
                perm[e] = (uint32_t)e;
    }
    if (!rc && segs && I.nsegments_padded)
        rc = copy_d2h(plan->ctx, segs, plan->segs, (size_t)I.nsegments_padded * sizeof(Seg));
    if (!rc && splits && I.nsplit_rows) {
        std::vector<SplitRow> tmp;
        try {
            tmp.resize(I.nsplit_rows);
        } catch (const std::bad_alloc &) {
            return fail(SPC3D_ERR_ALLOC, "host allocation failed");
        }
        rc = copy_d2h(plan->ctx, tmp.data(), plan->splits, tmp.size() * sizeof(SplitRow));
        for (size_t i = 0; !rc && i < tmp.size(); ++i) {
            splits[3 * i + 0] = tmp[i].row;
            splits[3 * i + 1] = tmp[i].first_slot;
            splits[3 * i + 2] = tmp[i].nslots;
        }
    }
    return rc;
}

// A whole non-negative decimal number in the environment; anything else is ignored.
static bool env_number(const char *name, unsigned long long *out)
{
    const char *s = std::getenv(name);
    if (!s || !*s)
        return false;
    unsigned long long v = 0;
    for (const char *c = s; *c; ++c) {
        if (*c < '0' || *c > '9' || v > (~0ull - 9) / 10)
            return false;
        v = v * 10 + (unsigned)(*c - '0');
    }
    *out = v;
    return true;
}

// The defaults of spc3d_plan_create and of the one-shot host calls: the library's, each
// overridable from the environment for tuning runs and A/B comparisons (read here, once
// per plan, and nowhere else; spc3d_plan_create_ex takes what its caller passes).
static spc3d_plan_opts opts_from_env()
{
    spc3d_plan_opts o;
    std::memset(&o, 0, sizeof o);
    struct {
        const char *name;
        uint32_t *field;
    } env[] = {{"SPC3D_SEG_MAX", &o.seg_max},
               {"SPC3D_K_HINT", &o.k_hint},
               {"SPC3D_L2_HOT_BYTES", &o.l2_hot_bytes},
               {"SPC3D_HUB_MIN", &o.hub_min},
               {"SPC3D_XCD_SLICES", &o.xcd_slices},
               {"SPC3D_COL_BLOCKS", &o.col_blocks},
               {"SPC3D_TWO_PASS_MIN", &o.two_pass_min}};
    unsigned long long v = 0;
    for (auto &e : env)
        if (env_number(e.name, &v) && v > 0 && v <= 0xFFFFFFFFull)
            *e.field = (uint32_t)v;
    struct {
        const char *name;
        uint32_t off_flag;
    } sw[] = {{"SPC3D_STAGE_STORES", SPC3D_PLAN_NO_STAGED_STORES},
              {"SPC3D_SDDMM_BY_COLUMN", SPC3D_PLAN_NO_SDDMM_BY_COLUMN},
              {"SPC3D_TWO_PASS", SPC3D_PLAN_NO_TWO_PASS}};
    for (auto &e : sw)
        if (env_number(e.name, &v) && v == 0)
            o.flags |= e.off_flag;
    if (env_number("SPC3D_KEEP_ENTRY_ORDER", &v) && v != 0)
        o.flags |= SPC3D_PLAN_KEEP_ENTRY_ORDER;
    if (const char *b = std::getenv("SPC3D_PLAN_BUILDER"))
        o.builder = std::strcmp(b, "host") == 0 ? 1u : 2u;
    return o;
}

int spc3d_plan_create(spc3d_ctx *ctx, int dtype, uint32_t nrows, uint32_t ncols, uint64_t nnz,
                      const uint32_t *ii, const uint32_t *jj, const void *vv, spc3d_plan **out)
{
    const spc3d_plan_opts o = opts_from_env();
    return spc3d_plan_create_ex(ctx, dtype, nrows, ncols, nnz, ii, jj, vv, &o, out);
}

int spc3d_plan_destroy(spc3d_plan *plan)
{
    if (!live(plan))
        return fail(SPC3D_ERR_INVALID_ARG, "plan is NULL or destroyed");
    if (int rc = refuse_while_capturing(plan->ctx))
        return rc;
    (void)hipSetDevice(plan->ctx->device);
    (void)hipStreamSynchronize(plan->ctx->stream);
    destroy_blocks(plan);
    if (plan->by_col) {
        plan_free_device(plan->by_col);
        plan->by_col->magic = 0;
        delete plan->by_col;
        plan->by_col = nullptr;
    }
    plan_free_device(plan);
    plan->magic = 0;
    delete plan;
    return SPC3D_OK;
}

// The parts a call works on: the plan itself, or its column blocks.
static std::vector<spc3d_plan *> &parts_of(spc3d_plan *plan, std::vector<spc3d_plan *> &self)
{
    if (!plan->blocks.empty())
        return plan->blocks;
    self.assign(1, plan);
    return self;
}

// A block's view for SDDMM: results at their places in the parent's staging vector.
static DevPlanView staged_view(const spc3d_plan *parent, const spc3d_plan *block)
{
    DevPlanView v = view_of(block);
    v.perm = parent->stage_of + block->stage_off;
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
    return parent->c_stage;
}

int spc3d_plan_set_values(spc3d_plan *plan, const void *vv_host)
{
    if (!live(plan))
        return fail(SPC3D_ERR_INVALID_ARG, "plan is NULL or destroyed");
    const uint64_t nnz = plan->info.nnz;
    if (nnz && !vv_host)
        return fail(SPC3D_ERR_INVALID_ARG, "vv is NULL");
    int rc = use_device(plan->ctx);
    if (rc)
        return rc;
    const size_t bytes = (size_t)nnz * elem_size(plan->dtype);
    if (plan->blocks.empty() && !plan->perm && !plan->by_col) {
        rc = copy_h2d(plan->ctx, plan->sval, vv_host, bytes);
    } else {
        void *tmp = nullptr;
        rc = dev_alloc_bytes(&tmp, bytes);
        if (rc)
            return rc;
        rc = copy_h2d(plan->ctx, tmp, vv_host, bytes);
        std::vector<spc3d_plan *> self;
        for (spc3d_plan *part : parts_of(plan, self)) {
            if (rc)
                break;
            hipError_t e = launch_gather_vals(plan->dtype, tmp, part->perm, part->sval,
                                              part->info.nnz, plan->ctx->stream);
            if (e != hipSuccess)
                rc = fail_hip(e, "gather of sparse values");
        }
        if (!rc && plan->by_col) {
            hipError_t e = launch_gather_vals(plan->dtype, tmp, plan->by_col->perm,
                                              plan->by_col->sval, nnz, plan->ctx->stream);
            if (e != hipSuccess)
                rc = fail_hip(e, "gather of sparse values");
            plan->by_col->has_values = true;
        }
        if (!rc) {
            hipError_t e = hipStreamSynchronize(plan->ctx->stream);
            if (e != hipSuccess)
                rc = fail_hip(e, "gather of sparse values");
        }
        (void)hipFree(tmp);
    }
    if (!rc)
        plan->has_values = true;
    return rc;
}

int spc3d_plan_set_values_device(spc3d_plan *plan, const spc3d_vals *vv)
{
    if (!live(plan) || !live(vv))
        return fail(SPC3D_ERR_INVALID_ARG, "plan or value vector is NULL or destroyed");
    if (vv->dtype != plan->dtype || vv->n < plan->info.nnz || vv->ctx != plan->ctx)
        return fail(SPC3D_ERR_SIZE_MISMATCH,
                    "value vector dtype / length / context does not fit the plan");
    int rc = use_device(plan->ctx, true);
    if (rc)
        return rc;
    std::vector<spc3d_plan *> self;
    for (spc3d_plan *part : parts_of(plan, self))
        HIP_TRY(launch_gather_vals(plan->dtype, vv->dev, part->perm, part->sval, part->info.nnz,
                                   plan->ctx->stream));
    if (plan->by_col) {
        HIP_TRY(launch_gather_vals(plan->dtype, vv->dev, plan->by_col->perm, plan->by_col->sval,
                                   plan->info.nnz, plan->ctx->stream));
        plan->by_col->has_values = true;
    }
    plan->has_values = true;
    return SPC3D_OK;
}

// One plan's columns rewritten in place, and its table of first columns with them.
static int probe_columns_of(spc3d_plan *p, int mode, uint32_t modulus)
{
    HIP_TRY(launch_probe_cols(p->col, p->info.nnz, (uint32_t)mode, p->col_base, modulus,
                              p->info.ncols, p->ctx->stream));
    const uint32_t nshort = p->info.nsegments_padded - p->info.nsegments_long;
    HIP_TRY(launch_first_cols(p->segs + p->info.nsegments_long, nshort, p->col, p->first_cols,
                              p->ctx->stream));
    return SPC3D_OK;
}

int spc3d_plan_probe_columns(spc3d_plan *plan, int mode, uint32_t modulus)
{
    if (!live(plan))
        return fail(SPC3D_ERR_INVALID_ARG, "plan is NULL or destroyed");
    if (mode != SPC3D_PROBE_ALL_HIT && mode != SPC3D_PROBE_ALL_MISS)
        return fail(SPC3D_ERR_INVALID_ARG, "unknown probe mode");
    if (mode == SPC3D_PROBE_ALL_HIT && modulus == 0)
        return fail(SPC3D_ERR_INVALID_ARG, "modulus is 0");
    if (plan->info.nnz == 0)
        return SPC3D_OK;
    int rc = use_device(plan->ctx);
    if (rc)
        return rc;
    std::vector<spc3d_plan *> self;
    for (spc3d_plan *part : parts_of(plan, self)) {
        rc = probe_columns_of(part, mode, modulus);
        if (rc)
            return rc;
    }
    if (plan->by_col) { // its columns are the pattern's rows
        rc = probe_columns_of(plan->by_col, mode, modulus);
        if (rc)
            return rc;
    }
    HIP_TRY(hipStreamSynchronize(plan->ctx->stream));
    return SPC3D_OK;
}

// Device memory one plan object holds (its blocks and companion are added by the caller).
static uint64_t own_device_bytes(const spc3d_plan *p)
{
    const uint64_t w = elem_size(p->dtype), nnz = p->info.nnz;
    uint64_t b = 0;
    if (p->segs) b += (uint64_t)p->info.nsegments_padded * sizeof(Seg);
    if (p->col) b += nnz * 4;
    if (p->perm) b += nnz * 4;
    if (p->sval) b += nnz * w;
    if (p->splits) b += (uint64_t)p->info.nsplit_rows * sizeof(SplitRow);
    if (p->first_cols)
        b += (uint64_t)(p->info.nsegments_padded - p->info.nsegments_long) * kFirstCols * 4;
    if (p->partial) b += (uint64_t)p->info.npartial_slots * p->partial_k * w;
    b += p->retired_bytes;
    if (p->store.perm2) b += nnz * 4;
    if (p->store.n) b += (uint64_t)p->store.n * (8 + w); // dst, src, staged results
    if (p->two.n) b += nnz * (2 + 4 + 2) + 2 * nnz * w;  // l1, dst1, l2; c_stage, c_mid
    if (!p->blocks.empty()) b += nnz * (w + 8);          // c_stage, stage_pos, stage_of
    return b;
}

int spc3d_plan_get_info(const spc3d_plan *plan, spc3d_plan_info *info)
{
    if (!live(plan) || !info)
        return fail(SPC3D_ERR_INVALID_ARG, "plan or info is NULL");
    *info = plan->info;
    uint64_t b = own_device_bytes(plan);
    for (const spc3d_plan *blk : plan->blocks)
        b += own_device_bytes(blk);
    if (plan->by_col)
        b += own_device_bytes(plan->by_col);
    info->device_bytes = b;
    return SPC3D_OK;
}

// Partial-sum rows of cut rows.  They are allocated when the plan is created, for the
// row width it was planned for (k_hint, 64 by default); a call with wider rows gets a
// larger block, and the one it replaces is kept until the plan is destroyed.
static int ensure_partial(spc3d_plan *p, uint32_t K)
{
    if (!p->info.npartial_slots || p->partial_k >= K)
        return SPC3D_OK;
    if (p->ctx->capturing)
        return fail(SPC3D_ERR_INVALID_ARG,
                    "the plan's partial-sum rows are narrower than this K: create the plan with "
                    "k_hint >= K, or run the call once before recording it");
    void *grown = nullptr;
    int rc = dev_alloc_bytes(&grown, (size_t)p->info.npartial_slots * K * elem_size(p->dtype));
    if (rc)
        return rc;
    if (p->partial) {
        try {
            p->retired_partial.push_back(p->partial);
            p->retired_bytes += (uint64_t)p->info.npartial_slots * p->partial_k * elem_size(p->dtype);
        } catch (const std::bad_alloc &) {
            (void)hipFree(grown);
            return fail(SPC3D_ERR_ALLOC, "host allocation failed");
        }
    }
    p->partial = grown;
    p->partial_k = K;
    return SPC3D_OK;
}

// [lo, lo + bytes) of two device buffers intersect.
static bool ranges_overlap(const void *a, size_t abytes, const void *b, size_t bbytes)
{
    const uintptr_t a0 = (uintptr_t)a, b0 = (uintptr_t)b;
    return a0 < b0 + bbytes && b0 < a0 + abytes;
}
static size_t panel_bytes(const spc3d_panel *p)
{
    return (size_t)p->m * p->n * elem_size(p->dtype);
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
    if (S->by_col) { // the same entries with rows and columns, and so A and B, exchanged
        const spc3d_plan *T = S->by_col;
        HIP_TRY(launch_sddmm(S->dtype, view_of(T), B->dev, A->dev, C->dev, K, streams_of(ctx)));
        HIP_TRY(unstage_stores(T, C->dev));
        return SPC3D_OK;
    }
    if (S->blocks.empty()) {
        HIP_TRY(launch_sddmm(S->dtype, view_of(S), A->dev, B->dev, sddmm_out(S, C->dev), K,
                             streams_of(ctx)));
        HIP_TRY(finish_sddmm(S, C->dev));
        return SPC3D_OK;
    }
    for (spc3d_plan *part : S->blocks)
        HIP_TRY(launch_sddmm(S->dtype, staged_view(S, part), A->dev, B->dev, staged_out(S, part), K,
                             streams_of(ctx)));
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
    std::vector<spc3d_plan *> self;
    for (spc3d_plan *part : parts_of(Ap, self)) {
        rc = ensure_partial(part, K);
        if (rc)
            return rc;
    }
    // The blocks add into Y one after the other on the stream: a fixed order.
    for (spc3d_plan *part : parts_of(Ap, self))
        HIP_TRY(launch_spmm(Ap->dtype, view_of(part), X->dev, Y->dev, K, streams_of(ctx)));
    return SPC3D_OK;
}

int spc3d_spmm_noalloc(spc3d_ctx *ctx, spc3d_plan *Ap, const spc3d_panel *X, spc3d_panel *Y)
{
    uint32_t K = 0;
    int rc = spmm_check(ctx, Ap, X, Y, &K);
    if (rc || K == 0)
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
    const size_t nparts = Ap->blocks.empty() ? 1 : Ap->blocks.size(); // no container: no host heap either
    for (size_t i = 0; i < nparts; ++i) {
        DevPlanView view = view_of(Ap->blocks.empty() ? Ap : Ap->blocks[i]);
        view.partial = ctx->scratch;
        HIP_TRY(launch_spmm(Ap->dtype, view, X->dev, Y->dev, K, streams_of(ctx)));
    }
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
    std::vector<spc3d_plan *> self;
    for (spc3d_plan *part : parts_of(S, self)) {
        rc = ensure_partial(part, K);
        if (rc)
            return rc;
    }
    const bool staged = !S->blocks.empty();
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
