// What the translation units of the C ABI share (api.cpp: contexts, panels, value vectors,
// the hot path; api_plan.cpp: plans; api_host_calls.cpp: the one-shot calls over host
// memory): the handle types behind the opaque pointers of include/spcomm3d_hip.h, error
// reporting, and small helpers.  Internal to the library.
#pragma once
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


inline thread_local std::string g_err;

inline int fail(int status, const std::string &msg)
{
    g_err = msg;
    return status;
}

inline int fail_hip(hipError_t e, const char *what)
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
    int cu_count;     // compute units of the device
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
    // Row tiles x column blocks (SweepPlan in plan_device.h, the sweep kernels in kernels.h):
    // the long rows of a pattern over unskewed columns, laid out for dense rows of sweep_k
    // reals.  `blocks` then holds at most one ordinary plan, over the entries of the other
    // rows ("rest").  SDDMM results: the sweep's in kernel order at c_stage[0 .. sweep.n),
    // the rest's in its kernel order from c_stage[rest_off]; stage_pos brings both home.
    SweepPlan sweep;
    void *sweep_sval = nullptr; // [sweep.n] values in sweep order
    uint32_t sweep_k = 0;
    uint64_t rest_off = 0;
    // The tiles are laid out for dense rows of sweep_k reals.  A call at another K runs
    // `other_k`: an ordinary plan of the same pattern, made from this plan's own arrays by the
    // first such call (plan_for_k) and kept, with this plan's values.
    spc3d_plan *other_k = nullptr;
};

inline SweepView sweep_view_of(const spc3d_plan *p)
{
    SweepView v;
    v.ptr = p->sweep.ptr;
    v.tile_rows = p->sweep.tile_rows;
    v.col = p->sweep.col;
    v.lrow = p->sweep.lrow;
    v.sval = p->sweep_sval;
    v.ntiles = p->sweep.ntiles;
    v.nblocks = p->sweep.nblocks;
    v.rows_per_tile = p->sweep.rows_per_tile;
    v.lanes = p->sweep.lanes;
    v.per_launch = p->sweep.per_launch;
    return v;
}

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


inline bool live(const spc3d_ctx *c) { return c && c->magic == kMagicCtx; }
inline bool live(const spc3d_panel *p) { return p && p->magic == kMagicPanel && live(p->ctx); }
inline bool live(const spc3d_vals *v) { return v && v->magic == kMagicVals && live(v->ctx); }
inline bool live(const spc3d_plan *p) { return p && p->magic == kMagicPlan && live(p->ctx); }
inline bool live(const spc3d_rowmap *p) { return p && p->magic == kMagicRowMap && live(p->ctx); }

inline bool live(const spc3d_graph *g) { return g && g->magic == kMagicGraph && live(g->ctx); }

// Makes the context's device current.  While the context records a graph only the
// calls that merely queue kernels may run (capturable); everything that allocates,
// copies to or from the host or waits is refused.
inline int use_device(const spc3d_ctx *ctx, bool capturable = false)
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

inline int dev_alloc_bytes(void **out, size_t bytes)
{
    *out = nullptr;
    if (bytes == 0)
        return SPC3D_OK;
    HIP_TRY(hipMalloc(out, bytes));
    return SPC3D_OK;
}

// Pageable-host <-> device copy ordered after everything queued on the
// stream; returns when the host side may be reused / read.
inline int copy_h2d(spc3d_ctx *ctx, void *dst, const void *src, size_t bytes)
{
    if (bytes == 0)
        return SPC3D_OK;
    HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, ctx->stream));
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    return SPC3D_OK;
}

inline int copy_d2h(spc3d_ctx *ctx, void *dst, const void *src, size_t bytes)
{
    if (bytes == 0)
        return SPC3D_OK;
    HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, ctx->stream));
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    return SPC3D_OK;
}

inline void plan_free_device(spc3d_plan *p)
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

inline Streams streams_of(const spc3d_ctx *c)
{
    Streams s;
    s.main = c->stream;
    s.aux = c->aux_stream;
    s.fork = c->fork_event;
    s.join = c->join_event;
    s.aux_rot = c->aux_rot;
    return s;
}

inline DevPlanView view_of(const spc3d_plan *p)
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



inline int refuse_while_capturing(const spc3d_ctx *ctx)
{
    if (ctx->capturing)
        return fail(SPC3D_ERR_INVALID_ARG,
                    "not allowed between spc3d_capture_begin and spc3d_capture_end");
    return SPC3D_OK;
}

// A whole non-negative decimal number in the environment; anything else is ignored.
inline bool env_number(const char *name, unsigned long long *out)
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

// [lo, lo + bytes) of two device buffers intersect.
inline bool ranges_overlap(const void *a, size_t abytes, const void *b, size_t bbytes)
{
    const uintptr_t a0 = (uintptr_t)a, b0 = (uintptr_t)b;
    return a0 < b0 + bbytes && b0 < a0 + abytes;
}
inline size_t panel_bytes(const spc3d_panel *p)
{
    return (size_t)p->m * p->n * elem_size(p->dtype);
}

// The ordinary parts a call works on: the plan itself, or its column blocks (beside a
// sweep: the plan of the rest, if there is one).
inline std::vector<spc3d_plan *> &parts_of(spc3d_plan *plan, std::vector<spc3d_plan *> &self)
{
    if (!plan->blocks.empty())
        return plan->blocks;
    self.clear();
    if (!plan->sweep.n) // a plan that is all sweep has no ordinary part
        self.push_back(plan);
    return self;
}

// Defined in api_plan.cpp (inside its extern "C" block, hence the linkage; not exported: the
// library is built with hidden visibility and only SPC3D_API symbols are visible).
// Partial-sum rows of cut rows wide enough for K columns (allocates a larger block when needed).
extern "C" int ensure_partial(spc3d_plan *p, uint32_t K);
// The plan a call at K columns runs: `plan` itself, or for a plan in row tiles at another K
// than it was laid out for, its ordinary twin (built on first use unless may_build is false;
// never while the context records).
extern "C" int plan_for_k(spc3d_plan *plan, uint32_t K, bool may_build, spc3d_plan **out);
// The defaults of spc3d_plan_create and of the one-shot host calls: the library's, each
// overridable from the environment.
extern "C" spc3d_plan_opts opts_from_env();

