// Launch interface between the C ABI (api.cpp) and the gfx950 kernels (kernels.hip).
#pragma once
#include <hip/hip_runtime_api.h>

#include <cstdint>

#include "plan_host.h"

namespace spc3d {

// Device-side view of a plan; all pointers are device pointers.
struct DevPlanView {
    const Seg *segs = nullptr;
    uint32_t nseg = 0;                // including padding segments
    uint32_t nseg_long = 0;           // leading segments that are all long (whole chunk rounds)
    uint32_t nqueues = 1;             // 1, or 8: chunk v of the segments belongs to XCD v % 8
    const uint32_t *col = nullptr;    // [nnz] kernel order
    const uint32_t *perm = nullptr;   // [nnz] kernel order -> caller's position; null if identity
    const void *sval = nullptr;       // [nnz] values in kernel order
    const SplitRow *splits = nullptr;
    uint32_t nsplit = 0;
    void *partial = nullptr;          // [nslots * K] partial sums of cut rows (SpMM)
    // [(nseg - nseg_long) * kFirstCols] the first column indices of every segment past
    // the long ones (launch_first_cols); read by the short-segment launch
    const uint32_t *first_cols = nullptr;
    uint64_t nnz = 0;
    bool stream_c = false;            // SDDMM: streaming stores also at permuted positions
    // SDDMM results whose position in `perm` is stage_from or more go to place (position -
    // stage_from) of `stage` (see build_store_staging in plan_device.h); launch_unstage_pairs
    // brings them to the caller's positions afterwards
    void *stage = nullptr;
    uint32_t stage_from = 0xFFFFFFFFu;
    // every segment's positions in `perm` are perm[start], perm[start] + 1, ...: SDDMM
    // reads one position per segment
    bool seg_base = false;
};

// The context's stream, plus an auxiliary stream of the same (default) priority
// and two timing-free events with which a call can run two launches side by
// side and rejoin the main stream.  aux == null: everything goes to `main`.
struct Streams {
    hipStream_t main = nullptr;
    hipStream_t aux = nullptr;
    hipEvent_t fork = nullptr, join = nullptr;
    uint32_t aux_rot = 0; // workgroup b of an aux launch runs on the XCD of main's b + aux_rot
};

// dtype: 0 = float, 1 = double.  Asynchronous; everything launched is ordered
// before whatever is queued on streams.main afterwards.
hipError_t launch_sddmm(int dtype, const DevPlanView &P, const void *A, const void *B, void *C,
                        uint32_t K, const Streams &streams);
hipError_t launch_spmm(int dtype, const DevPlanView &P, const void *X, void *Y, uint32_t K,
                       const Streams &streams);
// SDDMM and the SpMM of the same pattern over the same B in one pass over the
// gathered rows: C as launch_sddmm, and Y += W B with W = the plan's values
// (chained == 0) or the C just computed (chained != 0).  P.partial must hold the
// plan's partial-sum rows for this K.  hipErrorNotSupported when K has no vector kernel
// (dense rows over 4096 bytes).
hipError_t launch_sddmm_spmm(int dtype, int chained, const DevPlanView &P, const void *A,
                             const void *B, void *C, void *Y, uint32_t K, const Streams &streams);
// ---- row tiles x column blocks ("sweep") -------------------------------------------
// Device-side view of a sweep plan (SweepPlan in plan_device.h): the entries of rows of at
// least a minimum length, ordered by tile of rows, column block, row.
struct SweepView {
    const uint32_t *ptr = nullptr;       // [ntiles * nblocks + 1] entry range of every (tile, block)
    const uint32_t *tile_rows = nullptr; // [ntiles * rows_per_tile] row of each local row, or 0xFFFFFFFF
    const uint32_t *col = nullptr;       // [n] sweep order
    const uint16_t *lrow = nullptr;      // [n] local row in the tile
    const void *sval = nullptr;          // [n] values in sweep order
    // [n] or null.  SDDMM: where result k goes in C (null: C[k]).  SpMM: value k is
    // sval[pos[k]] (null: sval[k]).
    const uint32_t *pos = nullptr;
    uint32_t ntiles = 0, nblocks = 0, rows_per_tile = 0;
    uint32_t lanes = 0;                  // lanes per dense row the plan was made for: 16, 32 or 64
    uint32_t per_launch = 0;             // tiles per generation (the GPU's CU count)
};
// Lanes per dense row of K reals when the sweep kernels take that width (dense rows of 256,
// 512 or 1024 bytes), else 0; lane groups per workgroup, rows of a tile, and the most column
// blocks a tile's range bounds fit LDS for, for that many lanes.
uint32_t sweep_lanes(int dtype, uint32_t K);
uint32_t sweep_groups(uint32_t lanes);
uint32_t sweep_rows_per_tile(uint32_t lanes);
uint32_t sweep_max_blocks(uint32_t lanes);
// SDDMM over the sweep's entries: C[k] = sval[k] * <A[row of k,:], B[col[k],:]> in sweep order
// (the caller brings them to the caller's positions); SpMM: Y[row,:] += sums.  K = lanes * 16
// bytes / sizeof(real) exactly.  One launch per generation of per_launch tiles.
hipError_t launch_sweep_sddmm(int dtype, const SweepView &S, const void *A, const void *B, void *C,
                              hipStream_t stream);
hipError_t launch_sweep_spmm(int dtype, const SweepView &S, const void *X, void *Y, hipStream_t stream);
// first_cols[s * kFirstCols + u] = column of entry min(u, len - 1) of segment segs[s], s < n
hipError_t launch_first_cols(const Seg *segs, uint32_t n, const uint32_t *col, uint32_t *first_cols,
                             hipStream_t stream);
// out[i] = in[pos[i]], i < n; pos and out 16-byte aligned
hipError_t launch_unstage(int dtype, const void *in, const uint32_t *pos, void *out, uint64_t n,
                          hipStream_t stream);
// out[dst[h]] = stage[src[h]], h < n (dst ascending, mostly consecutive)
hipError_t launch_unstage_pairs(int dtype, const void *stage, const uint32_t *src,
                                const uint32_t *dst, void *out, uint64_t n, hipStream_t stream);
// out[perm[p]] = stage[p] for the permutation whose two-pass tables (TwoPass in plan_device.h,
// built for tiles of two_pass_tile_elems(dtype) elements) are l1, dst1, l2; `mid` holds n reals
// in between.  Needs two_pass_lds_bytes() of LDS per workgroup (all 160 KiB of a gfx950 CU).
uint32_t two_pass_tile_elems(int dtype);
uint32_t two_pass_lds_bytes();
hipError_t launch_unpermute_two_pass(int dtype, const void *stage, void *mid, const uint16_t *l1,
                                     const uint32_t *dst1, const uint16_t *l2, void *out, uint64_t n,
                                     hipStream_t stream);
// out[p] = in[perm[p]] (perm == null: copy)
// out[perm[i]] = in[i], i < n (perm null: a copy).
hipError_t launch_scatter_vals(int dtype, const void *in, const uint32_t *perm, void *out,
                               uint64_t n, hipStream_t stream);
hipError_t launch_gather_vals(int dtype, const void *in, const uint32_t *perm, void *out,
                              uint64_t n, hipStream_t stream);
// Device-side view of a row map (buffer slot i <-> dense row rows[i]).
struct RowMapView {
    const uint32_t *rows = nullptr;  // [nslots]
    const uint32_t *urows = nullptr; // [nuniq] distinct rows
    const uint32_t *ptr = nullptr;   // [nuniq + 1] into slots
    const uint32_t *slots = nullptr; // [nslots] slots grouped by row, ascending inside a row
    uint32_t nslots = 0, nuniq = 0;
};
// op 0: buf[i,:] = panel[rows[i],:]; op 1: panel[rows[i],:] = buf[i,:] (last slot of a row
// wins); op 2: panel[rows[i],:] += buf[i,:] in slot order.  K reals per row.
hipError_t launch_rows(int op, int dtype, void *panel, const RowMapView &M, uint32_t K, void *buf,
                       hipStream_t stream);
// out[b] = id of the XCD workgroup b of an nblocks-wide grid ran on
hipError_t launch_xcc_probe(uint32_t *out, uint32_t nblocks, hipStream_t stream);
// Measurement aid: col[i] = base + (col[i] - base) % modulus (mode 1: every gather then hits
// a table of `modulus` dense rows) or a hash of i, uniform over [0, ncols) (mode 2: nearly
// every gather misses); the plan then computes another pattern with the same segments.
hipError_t launch_probe_cols(uint32_t *col, uint64_t n, uint32_t mode, uint32_t base,
                             uint32_t modulus, uint32_t ncols, hipStream_t stream);
// dst[0..bytes) = src[0..bytes); both 16-byte aligned, non-overlapping
hipError_t launch_copy(void *dst, const void *src, uint64_t bytes, hipStream_t stream);
hipError_t launch_fill(int dtype, void *p, uint64_t n, double value, hipStream_t stream);

// Name of the kernel variant launch_sddmm / launch_spmm picks for (dtype, K);
// for logs and profiles.
const char *kernel_variant(int dtype, uint32_t K);

} // namespace spc3d
