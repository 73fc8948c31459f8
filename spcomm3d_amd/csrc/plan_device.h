// Device-side construction of the kernel-order form of a COO pattern: the same
// arrays build_host_plan produces (plan_host.h), bit for bit, built with
// histograms, scans and stable radix sorts on the GPU.
#pragma once
#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <string>

#include "plan_host.h"

namespace spc3d {

// Device arrays of a plan, owned by the receiver (hipFree each non-null one).
struct DevPlanArrays {
    Seg *segs = nullptr;        // [nseg_padded]
    uint32_t nseg_padded = 0;
    uint32_t *col = nullptr;    // [nnz]
    uint32_t *perm = nullptr;   // [nnz]; null when the caller's order is the kernel order
    SplitRow *splits = nullptr; // [nsplit]
    uint32_t nsplit = 0;
};

// d_ii, d_jj: device arrays of nnz entries.  On success fills `meta` (every
// scalar field of HostPlan; its vectors stay empty) and `out`.  Returns 0 or an
// spc3d_status value with `err` filled; a bad index is reported with its
// position and coordinates, as validate_coo does.  Work is queued on `stream`
// and the call returns after it has finished.
int build_device_plan(hipStream_t stream, uint32_t nrows, uint32_t ncols, uint64_t nnz,
                      const uint32_t *d_ii, const uint32_t *d_jj, const PlanOpts &opts,
                      HostPlan &meta, DevPlanArrays &out, std::string &err);

// COOMatrix::localizeIndices (src/SparseMatrix.hpp:69-99) on one device array of n
// indices: every distinct value gets the next local id the first time it
// appears, d_idx[e] becomes its local id, d_ltg[local] (capacity n) the value.
int localize_device(hipStream_t stream, uint64_t n, uint32_t *d_idx, uint32_t *d_ltg,
                    uint32_t *nlocal, std::string &err);

// COOMatrix::ReMapIndices (src/SparseMatrix.hpp:100-106): d_idx[e] = d_map[d_idx[e]];
// an index >= map_len is SPC3D_ERR_BAD_INDEX and nothing is changed.
int remap_device(hipStream_t stream, uint64_t n, uint32_t *d_idx, const uint32_t *d_map,
                 uint32_t map_len, std::string &err);

// ---- column blocks -----------------------------------------------------------------
// Stable partition of a device COO by column block (block b = columns [b * w, (b + 1) * w),
// w = ceil(ncols / nblocks)): d_order[q] = caller's position of partitioned entry q (the
// caller's order kept inside a block), d_ii_out / d_jj_out the entries in that order,
// first[b] (host, nblocks + 1 words) where block b starts.  The indices must have been
// validated (jj < ncols).
int partition_by_col_block(hipStream_t stream, uint64_t nnz, const uint32_t *d_ii,
                           const uint32_t *d_jj, uint32_t ncols, uint32_t nblocks,
                           uint32_t *d_ii_out, uint32_t *d_jj_out, uint32_t *d_order,
                           uint32_t *first, std::string &err);
// d_out[q] = d_order[d_perm ? d_perm[q] : q], q < n (a block's kernel order -> the caller's
// positions).  Asynchronous on `stream`.
int compose_perm_device(hipStream_t stream, const uint32_t *d_order, const uint32_t *d_perm,
                        uint64_t n, uint32_t *d_out, std::string &err);
// d_out[d_perm[q]] = d_vals[q], q < n.  Asynchronous on `stream`.
int scatter_device(hipStream_t stream, const uint32_t *d_perm, const uint32_t *d_vals, uint64_t n,
                   uint32_t *d_out, std::string &err);
// d_key[q] = d_rows[d_perm ? d_perm[q] : q] / rows_per_tile, q < n.  Asynchronous.
int tile_keys_device(hipStream_t stream, const uint32_t *d_rows, const uint32_t *d_perm, uint64_t n,
                     uint32_t rows_per_tile, uint32_t *d_key, std::string &err);
// d_rank[i] = position of element i in the stable ascending order of d_key (keys <=
// max_key).  Synchronous.
int stable_ranks_device(hipStream_t stream, const uint32_t *d_key, uint64_t n, uint32_t max_key,
                        uint32_t *d_rank, std::string &err);
// ---- staged SDDMM results ---------------------------------------------------------
// Where the kernel order regroups the entries of a row (the pieces a hub row is cut into
// by column slice), SDDMM's results leave a segment for caller's positions that are not
// consecutive: one 4- or 8-byte store per entry, each into a line of its own.  Such
// segments are "staged": their results go to consecutive places of a staging vector, as
// the segment holds them, and one pass afterwards brings them to the caller's positions
// in ascending order of those (so that its stores are the consecutive ones).
//   perm2[p]  = perm[p] for an entry whose segment stores to consecutive positions,
//               else nnz + the entry's place in the staging vector
//   dst, src  = for staged entry h in ascending order of caller's position: that
//               position, and its place in the staging vector
// n == 0 (and null arrays) when no segment needs it, or when staging does not pay: the
// staged entries' positions are not mostly consecutive, or the final pass would not read
// near what its neighbours read (a shuffled pattern, where that pass would scatter just as
// the kernel does), or nnz + n does not fit 32 bits.
// consecutive: with `perm2` in place of `perm` (n != 0), or with `perm` as it is (n == 0),
// every segment's positions are perm[start], perm[start] + 1, ...: the kernel can read one
// position per segment.  The arrays belong to the receiver (hipFree).  Synchronous.
struct StoreStaging {
    uint32_t *perm2 = nullptr; // [nnz]
    uint32_t *dst = nullptr;   // [n]
    uint32_t *src = nullptr;   // [n]
    uint64_t n = 0;
    bool consecutive = false;
};
int build_store_staging(hipStream_t stream, const Seg *d_segs, uint32_t nseg, const uint32_t *d_perm,
                        uint64_t nnz, StoreStaging &out, std::string &err);

// ---- row tiles x column blocks ("sweep") -------------------------------------------------
// For long rows over columns without skew (see the sweep kernels in kernels.hip).  Rows of at
// least min_row entries are ranked longest first; every per_launch * rows_per_tile of them
// make a generation (one launch), inside which a tile takes rows_per_tile rows that are
// consecutive by row number.  Their entries are sorted by (tile, column block, local row),
// the caller's order kept inside a row's run; the entries of shorter rows follow in the
// caller's order ("rest"; another plan runs them).
//   perm[k]      caller's position of entry k of that order                [nnz]
//   col, lrow    column and local row of sweep entry k                     [n]
//   ptr          range bounds per (tile, block)                            [ntiles*nblocks + 1]
//   tile_rows    row of local row l of tile t, 0xFFFFFFFF where there is none [ntiles*rows_per_tile]
// The arrays belong to the receiver (hipFree).  Synchronous.
struct SweepPlan {
    uint32_t *perm = nullptr, *col = nullptr, *ptr = nullptr, *tile_rows = nullptr;
    uint16_t *lrow = nullptr;
    uint64_t n = 0; // entries in the sweep; the other nnz - n are the rest
    uint32_t ntiles = 0, nblocks = 0, rows_per_tile = 0, groups = 0, lanes = 0, per_launch = 0;
    uint32_t nrows_in = 0; // rows in the sweep
};
int build_sweep(hipStream_t stream, uint32_t nrows, uint32_t ncols, uint64_t nnz,
                const uint32_t *d_ii, const uint32_t *d_jj, uint32_t lanes, uint32_t rows_per_tile,
                uint32_t nblocks, uint32_t min_row, uint32_t per_launch, SweepPlan &out,
                std::string &err);
// The pattern back from a plan: d_ii / d_jj at the caller's positions of the entries of a
// sweep, and of a plan in segments (d_perm null: its kernel order is the caller's).
// Asynchronous on `stream`.
int sweep_coords_device(hipStream_t stream, const SweepPlan &sw, uint32_t *d_ii, uint32_t *d_jj,
                        std::string &err);
int seg_coords_device(hipStream_t stream, const Seg *d_segs, uint64_t nseg, const uint32_t *d_col,
                      const uint32_t *d_perm, uint32_t *d_ii, uint32_t *d_jj, std::string &err);
// *out = how many q < n - 1 have d[q + 1] == d[q] + 1.  Synchronous.
int count_adjacent_device(hipStream_t stream, const uint32_t *d, uint64_t n, uint64_t *out,
                          std::string &err);
// d_out[d_perm[q]] = base + q, q < n.  Asynchronous on `stream`.
int inverse_offsets_device(hipStream_t stream, const uint32_t *d_perm, uint64_t n, uint32_t base,
                           uint32_t *d_out, std::string &err);
// d_out[q] = d_in[d_idx[q]], q < n.  Asynchronous on `stream`.
int gather_u32_device(hipStream_t stream, const uint32_t *d_in, const uint32_t *d_idx, uint64_t n,
                      uint32_t *d_out, std::string &err);

// ---- SDDMM results of an arbitrary entry order, brought home in two passes -------------
// C[perm[p]] = r[p] for all p, with r in kernel order, is one store (or one load) per result
// into a line of its own however it is turned.  Any permutation of n elements is two passes
// of tile-local moves when tile^2 >= n: with T elements per tile (what fits LDS),
//   pass 1, tile t of r (kernel positions [tT, tT + T)): the tile is read into LDS and written
//           out grouped by bucket of destination (bucket b = caller's positions [bT, bT + T)),
//           into an intermediate vector laid out bucket by bucket, inside a bucket tile by
//           tile: runs of about T^2 / n elements;
//   pass 2, bucket b of the intermediate vector: read into LDS, written to C in order.
// Everything is fixed by `perm`, so the plan holds, per element,
//   l1[s]   = which element of its tile goes to slot s of the tile's output order  (uint16)
//   dst1[s] = where slot s goes in the intermediate vector                         (uint32)
//   l2[q]   = which element of its bucket (as the intermediate vector holds it) is the
//             result for caller's position q                                      (uint16)
// T <= 65536.  n == 0: not built (n < 2 tiles, or the tile pairs do not fit a 32-bit sort key).
// The arrays belong to the receiver (hipFree).  Synchronous.
struct TwoPass {
    uint16_t *l1 = nullptr;  // [n]
    uint32_t *dst1 = nullptr; // [n]
    uint16_t *l2 = nullptr;  // [n]
    uint32_t tile = 0;       // T
    uint64_t n = 0;
};
int build_two_pass(hipStream_t stream, const uint32_t *d_perm, uint64_t nnz, uint32_t tile,
                   TwoPass &out, std::string &err);

// *out = d[0] <= d[1] <= ... <= d[n - 1] (device array); synchronous.
int is_nondecreasing_device(hipStream_t stream, const uint32_t *d, uint64_t n, bool *out,
                            std::string &err);

// Sum of len^2 over a plan's segments (device array); synchronous.
int sum_sq_seg_len_device(hipStream_t stream, const Seg *d_segs, uint64_t nseg, uint64_t *out,
                          std::string &err);

} // namespace spc3d
