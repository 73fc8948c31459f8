// C ABI, plans: validation, the two builders, how SDDMM results reach the caller's positions,
// column blocks, values, inspection (see include/spcomm3d_hip.h and api_internal.h).
#include "api_internal.h"

extern "C" {

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
    info.sweep_entries = 0;
    info.sweep_tiles = 0;
    info.sweep_k = 0;
}

// Library defaults, overridable field by field.  With XCD slicing, 2 MiB of
// each 4 MiB L2 is planned for dense rows, the rest is left to everything else.
static int resolve_opts(int dtype, const spc3d_plan_opts *o, PlanOpts &out)
{
    spc3d_plan_opts z;
    std::memset(&z, 0, sizeof z);
    if (o)
        z = *o;
    if (z.reserved[0])
        return fail(SPC3D_ERR_INVALID_ARG, "spc3d_plan_opts.reserved must be 0");
    if (z.sweep > 2)
        return fail(SPC3D_ERR_INVALID_ARG, "spc3d_plan_opts.sweep must be 0, 1 or 2");
    if (z.sweep == 2 && z.builder == 1)
        return fail(SPC3D_ERR_INVALID_ARG,
                    "row tiles are built on the GPU: builder must be 0 or 2 with sweep = 2");
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
    out.slice_affinity = !(z.flags & SPC3D_PLAN_NO_SLICE_AFFINITY);
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
    if (p->sweep.perm) (void)hipFree(p->sweep.perm);
    if (p->sweep.col) (void)hipFree(p->sweep.col);
    if (p->sweep.lrow) (void)hipFree(p->sweep.lrow);
    if (p->sweep.ptr) (void)hipFree(p->sweep.ptr);
    if (p->sweep.tile_rows) (void)hipFree(p->sweep.tile_rows);
    if (p->sweep_sval) (void)hipFree(p->sweep_sval);
    p->sweep = SweepPlan();
    p->sweep_sval = nullptr;
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

// Whether the pattern of a finished single plan goes into row tiles x column blocks
// (spc3d_plan_opts.sweep), for how many lanes per dense row and in how many blocks;
// *lanes = 0: no.  `nb_blocks` is what choose_col_blocks said.
static void choose_sweep(const spc3d_plan *p, const spc3d_plan_opts *opts, uint32_t nb_blocks,
                         uint32_t *lanes, uint32_t *nblocks)
{
    *lanes = *nblocks = 0;
    if (!opts || opts->sweep == 1 || !opts->k_hint || opts->builder == 1)
        return;
    const uint32_t l = sweep_lanes(p->dtype, opts->k_hint);
    if (!l || p->info.nnz == 0)
        return;
    const bool forced = opts->sweep == 2;
    if (!forced && (nb_blocks <= 1 || opts->col_blocks > 1))
        return; // a caller's own block count means blocks
    uint64_t nb = forced && opts->col_blocks > 1 ? opts->col_blocks : 0;
    if (!nb) {
        // 3.25 MiB of dense rows per block: on a 244 MiB panel (572 M entries, 512-byte rows)
        // 64 to 78 blocks measured level (19.7 .. 20.5 ms SDDMM, 20.2 .. 20.4 ms SpMM), 48 and
        // 128 half a millisecond to a millisecond slower, 192 three slower in SpMM
        constexpr uint64_t kBlockBytes = (uint64_t)13 << 18;
        const uint64_t panel = (uint64_t)p->info.cols_touched * opts->k_hint * elem_size(p->dtype);
        nb = std::max<uint64_t>(1, (panel + kBlockBytes - 1) / kBlockBytes);
    }
    nb = std::min<uint64_t>(nb, std::min<uint32_t>(sweep_max_blocks(l), p->info.ncols));
    *lanes = l;
    *nblocks = (uint32_t)std::max<uint64_t>(1, nb);
}

// Rebuilds a finished single plan `p` as row tiles x column blocks plus an ordinary plan of
// the rows too short for the tiles.  *taken = false (and p untouched) when no row qualifies
// or the device memory does not reach; any other failure is returned.
static int rebuild_as_sweep(spc3d_plan *p, uint32_t nrows, uint32_t ncols, uint64_t nnz,
                            const uint32_t *d_ii, const uint32_t *d_jj, const PlanOpts &po,
                            const spc3d_plan_opts *opts, uint32_t lanes, uint32_t nb, bool *taken)
{
    *taken = false;
    if (nnz + 64 >= (1ull << 32)) // staging places are 32-bit, the rest's start rounded up to 64
        return SPC3D_OK;
    spc3d_ctx *ctx = p->ctx;
    const size_t w = elem_size(p->dtype);
    const uint32_t min_row = opts->sweep_min_row ? opts->sweep_min_row : 64;
    const uint32_t per_launch = (uint32_t)std::max(1, ctx->cu_count);
    std::string err;
    SweepPlan sw;
    int rc = build_sweep(ctx->stream, nrows, ncols, nnz, d_ii, d_jj, lanes,
                         sweep_rows_per_tile(lanes), nb, min_row, per_launch, sw, err);
    if (rc)
        return optional_path(fail(rc, err));
    if (sw.n == 0)
        return SPC3D_OK;
    const uint64_t nrest = nnz - sw.n;
    const uint64_t rest_off = (sw.n + 63) / 64 * 64; // the rest's results start on a line of their own
    spc3d_plan *child = nullptr;
    uint32_t *r_ii = nullptr, *r_jj = nullptr, *gperm = nullptr, *stage_pos = nullptr;
    void *c_stage = nullptr, *sval = nullptr;
    if (nrest) {
        rc = dev_alloc(&r_ii, (size_t)nrest);
        if (!rc) rc = dev_alloc(&r_jj, (size_t)nrest);
        if (!rc) rc = dev_alloc(&gperm, (size_t)nrest);
        if (!rc) {
            rc = gather_u32_device(ctx->stream, d_ii, sw.perm + sw.n, nrest, r_ii, err);
            if (!rc) rc = gather_u32_device(ctx->stream, d_jj, sw.perm + sw.n, nrest, r_jj, err);
            HostPlan meta;
            DevPlanArrays arr;
            if (!rc) rc = build_device_plan(ctx->stream, nrows, ncols, nrest, r_ii, r_jj, po, meta, arr, err);
            if (rc)
                fail(rc, err);
            else
                rc = adopt_device_plan(ctx, p->dtype, meta, arr, planned_k(opts), &child);
        }
        if (!rc) {
            // the rest's kernel order -> the caller's positions
            rc = compose_perm_device(ctx->stream, sw.perm + sw.n, child->perm, nrest, gperm, err);
            if (rc)
                fail(rc, err);
        }
        if (!rc) {
            hipError_t e = hipStreamSynchronize(ctx->stream); // child->perm is read until here
            if (e != hipSuccess)
                rc = fail_hip(e, "hipStreamSynchronize");
        }
        if (!rc) {
            if (child->perm) (void)hipFree(child->perm);
            child->perm = gperm;
            gperm = nullptr;
            child->info.order_is_identity = 0;
        }
    }
    // Where the tiles' SDDMM results go: in a tile's kernel order a row's entries of one
    // block follow each other; when the caller's order keeps them together too, the kernel
    // stores them straight to their places (pieces of lines that the same workgroup completes
    // a few blocks later), else in kernel order to a staging vector that one more pass reads.
    bool staged = (opts->flags & SPC3D_PLAN_SWEEP_STAGED) != 0;
    if (!rc && !staged) {
        uint64_t adjacent = 0;
        rc = count_adjacent_device(ctx->stream, sw.perm, sw.n, &adjacent, err);
        if (rc)
            fail(rc, err);
        staged = adjacent * 5 < sw.n * 4;
    }
    if (!rc && staged) rc = dev_alloc_bytes(&c_stage, (size_t)(rest_off + nrest) * w);
    if (!rc && staged) rc = dev_alloc(&stage_pos, (size_t)nnz);
    if (!rc) rc = dev_alloc_bytes(&sval, (size_t)sw.n * w);
    if (!rc && staged) {
        rc = inverse_offsets_device(ctx->stream, sw.perm, sw.n, 0, stage_pos, err);
        if (!rc && nrest)
            rc = inverse_offsets_device(ctx->stream, child->perm, nrest, (uint32_t)rest_off, stage_pos, err);
        if (rc)
            fail(rc, err);
    }
    if (!rc) {
        hipError_t e = hipStreamSynchronize(ctx->stream);
        if (e != hipSuccess)
            rc = fail_hip(e, "hipStreamSynchronize");
    }
    if (r_ii) (void)hipFree(r_ii);
    if (r_jj) (void)hipFree(r_jj);
    if (gperm) (void)hipFree(gperm);
    if (rc) {
        const std::string keep = g_err;
        if (child) {
            plan_free_device(child);
            child->magic = 0;
            delete child;
        }
        if (c_stage) (void)hipFree(c_stage);
        if (stage_pos) (void)hipFree(stage_pos);
        if (sval) (void)hipFree(sval);
        (void)hipFree(sw.perm), (void)hipFree(sw.col), (void)hipFree(sw.lrow), (void)hipFree(sw.ptr),
            (void)hipFree(sw.tile_rows);
        return optional_path(fail(rc, keep));
    }
    // the whole pattern's arrays give way
    plan_free_device(p);
    p->partial_k = 0;
    spc3d_plan_info &I = p->info;
    I.nsegments = I.nsegments_padded = I.nsplit_rows = I.npartial_slots = I.nsegments_long = 0;
    I.order_is_identity = 0;
    if (child) {
        try {
            p->blocks.push_back(child);
        } catch (const std::bad_alloc &) {
            plan_free_device(child);
            child->magic = 0;
            delete child;
            (void)hipFree(c_stage), (void)hipFree(stage_pos), (void)hipFree(sval);
            (void)hipFree(sw.perm), (void)hipFree(sw.col), (void)hipFree(sw.lrow),
                (void)hipFree(sw.ptr), (void)hipFree(sw.tile_rows);
            return fail(SPC3D_ERR_ALLOC, "host allocation failed");
        }
        I.nsegments = child->info.nsegments;
        I.nsegments_padded = child->info.nsegments_padded;
        I.nsegments_long = child->info.nsegments_long;
        I.nsplit_rows = child->info.nsplit_rows;
        I.npartial_slots = child->info.npartial_slots;
        I.nqueues = child->info.nqueues;
    }
    p->sweep = sw;
    p->sweep_sval = sval;
    p->sweep_k = opts->k_hint;
    p->rest_off = rest_off;
    p->c_stage = c_stage;
    p->stage_pos = stage_pos;
    I.ncol_blocks = sw.nblocks;
    I.staged_entries = staged ? sw.n : 0;
    I.sweep_entries = sw.n;
    I.sweep_tiles = sw.ntiles;
    I.sweep_k = opts->k_hint;
    *taken = true;
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
    if (!rc) {
        uint32_t sw_lanes = 0, sw_nb = 0;
        choose_sweep(p, opts, nb, &sw_lanes, &sw_nb);
        bool taken = false;
        if (sw_lanes)
            rc = rebuild_as_sweep(p, nrows, ncols, nnz, d_ii, d_jj, po, opts, sw_lanes, sw_nb, &taken);
        if (rc) {
            const std::string keep = g_err;
            spc3d_plan_destroy(p);
            return fail(rc, keep);
        }
        if (taken) {
            *out = p;
            return SPC3D_OK;
        }
        if (sw_lanes && opts->sweep == 2 && opts->col_blocks <= 1)
            nb = 1; // asked for tiles, not for blocks
    }
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
    if (plan->sweep.n)
        return fail(SPC3D_ERR_INVALID_ARG,
                    "the plan is kept as row tiles x column blocks "
                    "(spc3d_plan_info.sweep_entries > 0): there is no single set of arrays");
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


// The defaults of spc3d_plan_create and of the one-shot host calls: the library's, each
// overridable from the environment for tuning runs and A/B comparisons (read here, once
// per plan, and nowhere else; spc3d_plan_create_ex takes what its caller passes).
spc3d_plan_opts opts_from_env()
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
    if (env_number("SPC3D_SLICE_AFFINITY", &v) && v == 0)
        o.flags |= SPC3D_PLAN_NO_SLICE_AFFINITY;
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
    if (plan->other_k) {
        spc3d_plan *o = plan->other_k;
        plan->other_k = nullptr;
        (void)spc3d_plan_destroy(o);
    }
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
    if (plan->blocks.empty() && !plan->perm && !plan->by_col && !plan->sweep.n) {
        rc = copy_h2d(plan->ctx, plan->sval, vv_host, bytes);
    } else {
        void *tmp = nullptr;
        rc = dev_alloc_bytes(&tmp, bytes);
        if (rc)
            return rc;
        rc = copy_h2d(plan->ctx, tmp, vv_host, bytes);
        if (!rc && plan->sweep.n) {
            hipError_t e = launch_gather_vals(plan->dtype, tmp, plan->sweep.perm, plan->sweep_sval,
                                              plan->sweep.n, plan->ctx->stream);
            if (e != hipSuccess)
                rc = fail_hip(e, "gather of sparse values");
        }
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
    if (!rc && plan->other_k)
        rc = spc3d_plan_set_values(plan->other_k, vv_host);
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
    if (plan->sweep.n)
        HIP_TRY(launch_gather_vals(plan->dtype, vv->dev, plan->sweep.perm, plan->sweep_sval,
                                   plan->sweep.n, plan->ctx->stream));
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
    if (plan->other_k)
        return spc3d_plan_set_values_device(plan->other_k, vv);
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
    if (plan->sweep.n) // one range of columns for every block: all hit, or all miss
        HIP_TRY(launch_probe_cols(plan->sweep.col, plan->sweep.n, (uint32_t)mode, 0, modulus,
                                  plan->info.ncols, plan->ctx->stream));
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
    if (p->sweep.n) {
        const uint64_t n = p->sweep.n, rest = nnz - n;
        b += n * (4 + 2 + w) + nnz * 4; // col, lrow, values; perm
        b += ((uint64_t)p->sweep.ntiles * p->sweep.nblocks + 1) * 4;
        b += (uint64_t)p->sweep.ntiles * p->sweep.rows_per_tile * 4;
        if (p->c_stage)
            b += ((n + 63) / 64 * 64 + rest) * w + nnz * 4; // c_stage, stage_pos
    } else if (!p->blocks.empty()) {
        b += nnz * (w + 8); // c_stage, stage_pos, stage_of
    }
    return b;
}

// The ordinary twin of a plan in row tiles (spc3d_plan::other_k): the pattern is read back
// from the plan's own arrays (the tiles' entries and the plan of the rest, each with its
// caller's positions), planned again without tiles for K columns, and given the values the
// plan holds.
static int build_other_k(spc3d_plan *S, uint32_t K)
{
    spc3d_ctx *ctx = S->ctx;
    const uint64_t nnz = S->info.nnz;
    const size_t w = elem_size(S->dtype);
    spc3d_plan_opts o;
    std::memset(&o, 0, sizeof o);
    o.k_hint = K;
    o.sweep = 1;
    PlanOpts po;
    int rc = resolve_opts(S->dtype, &o, po);
    if (rc)
        return rc;
    uint32_t *d_ii = nullptr, *d_jj = nullptr;
    void *vals = nullptr;
    spc3d_plan *q = nullptr;
    std::string err;
    rc = dev_alloc(&d_ii, (size_t)nnz);
    if (!rc) rc = dev_alloc(&d_jj, (size_t)nnz);
    if (!rc) {
        rc = sweep_coords_device(ctx->stream, S->sweep, d_ii, d_jj, err);
        for (spc3d_plan *part : S->blocks)
            if (!rc)
                rc = seg_coords_device(ctx->stream, part->segs, part->info.nsegments_padded,
                                       part->col, part->perm, d_ii, d_jj, err);
        if (rc)
            fail(rc, err);
    }
    if (!rc)
        rc = build_from_device(ctx, S->dtype, S->info.nrows, S->info.ncols, nnz, d_ii, d_jj, po, &o, &q);
    if (!rc && S->has_values) {
        rc = dev_alloc_bytes(&vals, (size_t)nnz * w);
        if (!rc) {
            hipError_t e = launch_scatter_vals(S->dtype, S->sweep_sval, S->sweep.perm, vals,
                                               S->sweep.n, ctx->stream);
            for (spc3d_plan *part : S->blocks)
                if (e == hipSuccess)
                    e = launch_scatter_vals(S->dtype, part->sval, part->perm, vals, part->info.nnz,
                                            ctx->stream);
            std::vector<spc3d_plan *> self;
            for (spc3d_plan *part : parts_of(q, self))
                if (e == hipSuccess)
                    e = launch_gather_vals(S->dtype, vals, part->perm, part->sval, part->info.nnz,
                                           ctx->stream);
            if (e == hipSuccess && q->by_col) {
                e = launch_gather_vals(S->dtype, vals, q->by_col->perm, q->by_col->sval, nnz,
                                       ctx->stream);
                q->by_col->has_values = true;
            }
            if (e == hipSuccess)
                e = hipStreamSynchronize(ctx->stream);
            if (e != hipSuccess)
                rc = fail_hip(e, "values of the plan for another K");
            else
                q->has_values = true;
        }
    }
    if (!rc) {
        hipError_t e = hipStreamSynchronize(ctx->stream);
        if (e != hipSuccess)
            rc = fail_hip(e, "hipStreamSynchronize");
    }
    if (d_ii) (void)hipFree(d_ii);
    if (d_jj) (void)hipFree(d_jj);
    if (vals) (void)hipFree(vals);
    if (rc) {
        const std::string keep = g_err;
        if (q)
            (void)spc3d_plan_destroy(q);
        return fail(rc, keep);
    }
    S->other_k = q;
    return SPC3D_OK;
}

int plan_for_k(spc3d_plan *plan, uint32_t K, bool may_build, spc3d_plan **out)
{
    *out = plan;
    if (!plan->sweep.n || K == plan->sweep_k)
        return SPC3D_OK;
    if (!plan->other_k) {
        char msg[256];
        if (!may_build || plan->ctx->capturing) {
            std::snprintf(msg, sizeof msg,
                          "the plan is laid out as row tiles for K = %u (spc3d_plan_info.sweep_k); "
                          "the plan it runs at another K (here %u) is made by the first spc3d_sddmm, "
                          "spc3d_spmm or spc3d_sddmm_spmm at such a K outside a recording: run one first",
                          plan->sweep_k, K);
            return fail(SPC3D_ERR_INVALID_ARG, msg);
        }
        int rc = use_device(plan->ctx);
        if (!rc)
            rc = build_other_k(plan, K);
        if (rc)
            return rc;
    }
    *out = plan->other_k;
    return SPC3D_OK;
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
    if (plan->other_k) {
        spc3d_plan_info twin;
        if (spc3d_plan_get_info(plan->other_k, &twin) == SPC3D_OK)
            b += twin.device_bytes;
    }
    info->device_bytes = b;
    return SPC3D_OK;
}

// Partial-sum rows of cut rows.  They are allocated when the plan is created, for the
// row width it was planned for (k_hint, 64 by default); a call with wider rows gets a
// larger block, and the one it replaces is kept until the plan is destroyed.
int ensure_partial(spc3d_plan *p, uint32_t K)
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

} // extern "C"
