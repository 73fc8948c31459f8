/*
 * spcomm3d_hip.h - C ABI of the MI355X (gfx950) local SDDMM / SpMM library.
 *
 * The reference has no FFI layer: its local compute step is two C++ free
 * functions with external linkage,
 *     SpKernels::sddmm(denseMatrix& A, denseMatrix& B, cooMat& S, cooMat& C)
 *     SpKernels::spmm (denseMatrix& X, cooMat& A, denseMatrix& Y)
 * declared in src/core_ops.hpp:9-12 and defined in src/core_ops.cpp:5-35,
 * called from src/distributed_comp.cpp:53,177,220,268,314,379 and
 * miniapp/numCheckSeq.cpp:130.  A host shim with those two signatures
 * (spcomm3d_amd/host) forwards to the entry points below; they are what a
 * binding for this path binds.
 *
 * Conventions
 *  - Plain pointers and sizes only.  Every function returns an spc3d_status;
 *    spc3d_last_error() gives the message of the calling thread's last
 *    failure.  No C++ exception crosses this boundary.  (The reference
 *    returns void and fails by std::out_of_range from .at() -> terminate,
 *    core_ops.cpp:16,18,32; the C++ shim turns a non-zero status back into
 *    that exception.)
 *  - Indices are uint32, 0-based, local (src/basic.hpp:16); dense panels are
 *    row-major with K contiguous (src/basic.hpp:32,36); values are float or
 *    double (the reference's real_t is double, src/basic.hpp:17; float is an
 *    extension).
 *  - COO entries may come in any order and may repeat.  SDDMM writes result e
 *    at position e of the caller's order (core_ops.cpp:18); SpMM adds into Y
 *    (core_ops.cpp:32), duplicates add.
 *  - The reference computes panel offsets x*n+y in 32 bits
 *    (src/basic.hpp:36), so its behaviour is defined only for m*n < 2^32.
 *    This library uses 64-bit offsets; nnz must be < 2^32.
 *  - A context is used by one host thread at a time and owns one HIP stream
 *    (default priority), plus an internal one of the same priority on which
 *    part of an SDDMM / SpMM call runs, forked from and joined back to the
 *    first by events inside the call.  Kernel-launching calls are asynchronous
 *    on the context's stream; *_download and *_host calls return with host
 *    memory valid.
 *  - Nothing here falls back to the CPU: without a usable GPU every device
 *    call fails with SPC3D_ERR_NO_DEVICE.
 */
#ifndef SPCOMM3D_HIP_H
#define SPCOMM3D_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(__GNUC__)
#define SPC3D_API __attribute__((visibility("default")))
#else
#define SPC3D_API
#endif

typedef enum {
    SPC3D_OK = 0,
    SPC3D_ERR_INVALID_ARG = 1,   /* null pointer, unknown dtype, destroyed handle */
    SPC3D_ERR_BAD_INDEX = 2,     /* ii[e] >= nrows or jj[e] >= ncols (reference: out_of_range) */
    SPC3D_ERR_SIZE_MISMATCH = 3, /* panel / value-vector shape or dtype does not fit the plan */
    SPC3D_ERR_TOO_LARGE = 4,     /* nnz >= 2^32 or a byte size overflows */
    SPC3D_ERR_NO_DEVICE = 5,     /* no HIP device / device id out of range */
    SPC3D_ERR_HIP = 6,           /* a HIP runtime call failed; see spc3d_last_error() */
    SPC3D_ERR_ALLOC = 7          /* host or device allocation failed */
} spc3d_status;

typedef enum { SPC3D_F32 = 0, SPC3D_F64 = 1 } spc3d_dtype;

typedef struct spc3d_ctx spc3d_ctx;     /* device + stream */
typedef struct spc3d_panel spc3d_panel; /* device-resident denseMatrix::data (src/basic.hpp:30-36) */
typedef struct spc3d_vals spc3d_vals;   /* device-resident cooMat::vv (src/SparseMatrix.hpp:36) */
typedef struct spc3d_plan spc3d_plan;   /* device-resident cooMat pattern (ii, jj) in kernel order */

typedef struct {
    uint32_t nrows, ncols;
    uint64_t nnz;
    uint32_t rows_touched;     /* rows with at least one entry */
    uint32_t cols_touched;     /* columns with at least one entry */
    uint32_t nsegments;        /* row segments the kernels work on */
    uint32_t nsegments_padded; /* stored segments: the above plus padding of short XCD queues */
    uint32_t nsplit_rows;      /* rows cut into several segments (SpMM combines partial sums) */
    uint32_t npartial_slots;   /* partial-sum rows kept for those */
    uint32_t max_row_nnz;
    uint32_t seg_max;          /* longest segment allowed */
    int32_t  order_is_identity; /* 1: the caller's order is the kernel order, no permutation read */
    uint32_t nqueues;          /* 1, or 8: segments are dealt to the 8 XCDs by column slice */
    uint32_t hot_cols;         /* XCD slicing: columns planned to stay in some L2 (0: slicing off) */
    uint32_t hub_rows;         /* XCD slicing: rows cut by column slice */
    uint64_t hot_entries;      /* XCD slicing: entries in those columns */
    uint32_t nsegments_long;   /* leading stored segments (all of >= 16 entries) that run in the
                                  wide-batch launch; the rest run in the high-occupancy one */
    uint32_t ncol_blocks;      /* 1, or the number of column blocks the plan is kept in: the
                                  segment counts above are then sums over the blocks,
                                  npartial_slots the largest block's */
    uint64_t staged_entries;   /* entries of segments whose caller's positions are not
                                  consecutive (hub rows cut by column slice): spc3d_sddmm
                                  writes their results in kernel order to a staging vector
                                  and brings them to C in one ordered pass; 0: none, or a
                                  pattern whose order makes that pass no better */
    uint32_t positions_by_segment; /* 1: every segment's results go to consecutive positions
                                  (of C or of the staging vector), so spc3d_sddmm reads one
                                  position per segment; 0: one per entry, or none (identity) */
    uint32_t sddmm_by_column;  /* 1: the pattern came sorted by column, and spc3d_sddmm runs a
                                  second plan of the same entries with rows and columns (and
                                  so A and B) exchanged, whose kernel order is the caller's:
                                  the same bits, stored in runs instead of one by one; the
                                  plan then holds its arrays twice (GPU builder only) */
    uint32_t two_pass_results; /* 1: an arbitrary entry order of 1.5 M entries or more: the
                                  SDDMM kernels write their results in kernel order to a
                                  vector of the plan, and two passes of tile-local moves
                                  through LDS bring them to the caller's positions (24 more
                                  bytes per entry in fp64, 16 in fp32) */
    uint32_t entries_by_column; /* 1: the rows arrived unsorted, and the plan orders the entries
                                  of every row by column (spc3d_spmm then adds a row's entries
                                  in that order); 0: the caller's order inside every row */
    uint64_t device_bytes;     /* device memory the plan holds: its arrays, values, partial-sum
                                  rows, result staging, a companion plan, every column block */
    uint64_t sweep_entries;    /* entries kept as row tiles x column blocks (spc3d_plan_opts.sweep);
                                  0: none.  The segment counts above are then those of the plan
                                  of the other entries */
    uint32_t sweep_tiles;      /* tiles of rows of that layout */
    uint32_t sweep_k;          /* the K it is laid out for (k_hint); calls at another K run an
                                  ordinary plan of the same pattern, made on first use */
} spc3d_plan_info;

/* Plan tuning; a zero field selects the default.  Only speed depends on these. */
typedef struct {
    uint32_t seg_max;      /* longest segment in entries (default: nnz / 2048 rounded down to
                              a power of two, within 64 .. 2048; with k_hint given, at most
                              1024 for dense rows of 128 bytes and 512 for 64 bytes and less) */
    uint32_t k_hint;       /* K the plan will mostly run with: sizes the XCD slicing (default
                              64) and the default seg_max */
    uint32_t l2_hot_bytes; /* XCD slicing: share of one XCD's 4 MiB L2 planned for dense rows
                              (default 2 MiB) */
    uint32_t hub_min;      /* XCD slicing: rows with at least this many entries are cut by
                              column slice (default 128) */
    uint32_t xcd_slices;   /* 8 (default): when the column degrees are skewed, the entries of
                              long rows are dealt to the 8 XCDs by column, so that each L2
                              caches its own eighth of the hot dense rows; 1: never */
    uint32_t builder;      /* where spc3d_plan_create[_ex] builds the plan: 0 (default) or 2:
                              on the GPU; 1: on the host, then uploaded.  Both give the same
                              arrays bit for bit. */
    uint32_t col_blocks;   /* 0 (default): the pattern is kept in blocks of columns, run one
                              after the other so that one block of dense rows (about 5 MiB)
                              is what the L2s see at a time, when its columns are not skewed,
                              the dense rows it gathers exceed 64 MiB at k_hint columns and
                              its rows are long enough (entry-weighted mean length at least
                              16 times the block count); 1: never; n > 1: in n blocks (at
                              most 4096).  Built on the GPU only; results are those of the
                              whole plan up to summation order (SpMM adds block after block) */
    uint32_t flags;        /* SPC3D_PLAN_* bits, 0: defaults */
    uint32_t two_pass_min; /* entries from which the results of an arbitrary entry order go home
                              in two tile-local passes (default 1,572,864: measured slower
                              under 1 M entries, faster from 1.9 M on) */
    uint32_t sweep;        /* row tiles x column blocks.  Where column blocks would be chosen
                              (col_blocks above) and k_hint is given with dense rows of 256,
                              512 or 1024 bytes, the rows of at least sweep_min_row entries are
                              not cut at block boundaries: tiles of rows (128 KiB of A rows, or
                              of Y accumulators) stay in LDS while their workgroups walk the
                              column blocks in step, one workgroup per CU; the other rows form
                              an ordinary plan.  The tiles run at K = k_hint; the first
                              spc3d_sddmm, spc3d_spmm or spc3d_sddmm_spmm at another K makes an
                              ordinary plan of the same pattern out of this plan's own arrays
                              (it allocates and waits, so not while recording, and not in
                              spc3d_spmm_noalloc, which return SPC3D_ERR_INVALID_ARG until
                              another call has made it) and later calls at other widths run
                              that one; spc3d_plan_info.device_bytes then counts both.
                              spc3d_spmm adds a row's entries block after block, and runs
                              give the same bits.
                              spc3d_sddmm stores the tiles' results straight to the caller's
                              positions when four in five of them follow their predecessor
                              there (a row's entries together), else through a staging vector
                              (spc3d_plan_info.staged_entries).
                              0 (default): as described; 1: never; 2: whenever k_hint has such
                              a width, whatever the pattern (col_blocks, if given, is the
                              number of blocks) */
    uint32_t sweep_min_row; /* shortest row kept in the tiles (default 64) */
    uint32_t reserved[1];  /* must be 0 */
} spc3d_plan_opts;
/* spc3d_plan_opts.flags.  The first three keep spc3d_sddmm's plain stores where the plan
 * would otherwise stage the results of regrouped segments, run a column-sorted pattern
 * through a second plan with rows and columns exchanged, or bring an arbitrary order home in
 * two passes (spc3d_plan_info: staged_entries, sddmm_by_column, two_pass_results): the same
 * bits either way, for comparisons and for callers short of device memory.  The fourth keeps
 * the caller's order inside every row also when the rows arrive unsorted (by default such
 * rows are ordered by column, which is what the gathers of a sorted pattern see). */
#define SPC3D_PLAN_NO_STAGED_STORES 1u
#define SPC3D_PLAN_NO_SDDMM_BY_COLUMN 2u
#define SPC3D_PLAN_NO_TWO_PASS 4u
#define SPC3D_PLAN_KEEP_ENTRY_ORDER 8u
/* Row tiles (sweep): stage the tiles' SDDMM results in kernel order and bring them home in
 * one more pass also when the caller's order keeps a row's entries together (by default the
 * tile kernels then store straight to the caller's positions, and nothing is staged). */
#define SPC3D_PLAN_SWEEP_STAGED 16u
/* XCD slicing: deal the segments that have no slice of their own (rows under hub_min, the cold
 * parts of hub rows) by their rank alone.  By default such a segment goes to the queue of the
 * slice most of its entries in sliced columns belong to, while that queue has room: on R-MAT 20
 * a third instead of an eighth of those entries then gather on the XCD that keeps their dense
 * rows (SDDMM / SpMM 2 to 4 % faster). */
#define SPC3D_PLAN_NO_SLICE_AFFINITY 32u
#define SPC3D_PLAN_ALL_FLAGS 63u

/* ---- library / errors ------------------------------------------------- */
SPC3D_API const char *spc3d_version(void);
SPC3D_API const char *spc3d_last_error(void);
/* Which kernel variant spc3d_sddmm / spc3d_spmm run for dense rows of k reals of
 * `dtype`, as text ("seg<f32,LPR=16,VPL=1>": 16 lanes per row, one 16-byte vector
 * each; ",ragged" / ",odd" / ",thin": rows that leave lanes idle, end inside a
 * vector, or are shorter than one; "... per 4 KiB slice": rows over 4 KiB).  A
 * diagnostic with no counterpart in the reference; needs no GPU.  The string
 * belongs to the calling thread and lasts until its next call.  NULL for an unknown
 * dtype. */
SPC3D_API const char *spc3d_kernel_variant(int dtype, uint32_t k);
SPC3D_API const char *spc3d_status_name(int status);
SPC3D_API int spc3d_device_count(int *count);

/* ---- context ----------------------------------------------------------- */
/* A context is one device, one stream (plus an auxiliary one of the same priority on which
 * the short-segment launch of a call runs beside the long-segment one) and what the one-shot
 * host calls keep between calls.  One caller thread per context, as the reference runs one
 * thread per MPI rank (MPI_Init in miniapp/bench_both.cpp:124): host_threads is how many host
 * threads a one-shot call over host memory (spc3d_*_host) may use, the caller's included, for
 * reading operands and moving Y; the default, 1, starts none, so that several ranks per node
 * do not oversubscribe it (SPC3D_HOST_THREADS in the environment gives spc3d_ctx_create
 * another default; 8 is what one rank per node can use).  Everything else in the library
 * runs on the caller's thread. */
typedef struct {
    uint32_t host_threads; /* 0: default (1); at most 256 */
    uint32_t flags;        /* SPC3D_CTX_* bits */
    uint32_t reserved[6];  /* must be 0 */
} spc3d_ctx_opts;
#define SPC3D_CTX_NO_AUX_STREAM 1u /* every launch on the one stream */
#define SPC3D_CTX_NO_HOST_CACHE 2u /* one-shot host calls: plan, upload, run, download, free, every call */
/* spc3d_ctx_create takes its options from the environment (SPC3D_HOST_THREADS=n,
 * SPC3D_AUX_STREAM=0, SPC3D_HOST_CACHE=0; read here and nowhere else), spc3d_ctx_create_ex
 * from its argument (NULL: the library defaults). */
SPC3D_API int spc3d_ctx_create(int device, spc3d_ctx **out);
SPC3D_API int spc3d_ctx_create_ex(int device, const spc3d_ctx_opts *opts, spc3d_ctx **out);
SPC3D_API int spc3d_ctx_destroy(spc3d_ctx *ctx);
SPC3D_API int spc3d_ctx_sync(spc3d_ctx *ctx);                 /* wait for the context's stream */
SPC3D_API int spc3d_ctx_stream(spc3d_ctx *ctx, void **hip_stream); /* the hipStream_t, for callers that share it */
/* xcd[b] = id of the XCD that workgroup b of an nblocks-wide grid ran on.  The
 * kernels assume workgroups are dealt to the 8 XCDs round-robin (xcd = b % 8)
 * when they place work next to the L2 that caches its dense rows; this lets a
 * caller check that on its machine.  Synchronous. */
SPC3D_API int spc3d_ctx_probe_xcd(spc3d_ctx *ctx, uint32_t nblocks, uint32_t *xcd);

/* A sequence of kernel-launching calls recorded once and replayed with one launch
 * (a HIP graph): for steps so short that launch latency dominates them (the
 * reference's 16384 x 16384 case runs one kernel in under 10 us).  Between
 * spc3d_capture_begin and spc3d_capture_end the calls that only queue kernels -
 * spc3d_sddmm, spc3d_spmm, spc3d_sddmm_spmm, spc3d_rows_*, spc3d_panel_fill,
 * spc3d_panel_copy, spc3d_vals_fill, spc3d_plan_set_values_device - are recorded
 * instead of run; every other call on the context (anything that allocates,
 * copies to or from the host, waits or times) returns SPC3D_ERR_INVALID_ARG and
 * leaves the recording intact.  An SpMM over a plan with cut rows whose dense rows
 * are wider than the plan was created for (k_hint, 64 by default) needs wider
 * partial-sum rows than the plan holds: create the plan with k_hint >= K, or run
 * the call once before recording it.  spc3d_graph_launch replays the sequence on the
 * context's stream, asynchronously, over the same operands; their contents at
 * launch time are what the kernels read.  Has no counterpart in the reference. */
typedef struct spc3d_graph spc3d_graph;
SPC3D_API int spc3d_capture_begin(spc3d_ctx *ctx);
SPC3D_API int spc3d_capture_end(spc3d_ctx *ctx, spc3d_graph **out);
SPC3D_API int spc3d_graph_launch(spc3d_graph *graph);
SPC3D_API int spc3d_graph_destroy(spc3d_graph *graph);

/* Timing on the context's stream (the reference times the call with chrono in
 * integer ms, src/distributed_comp.cpp:176-179; a kernel here lasts well under
 * one).  spc3d_timer_mark records event `slot` (0..4095) on the stream;
 * spc3d_timer_elapsed_ms waits for `stop` and returns stop-start. */
SPC3D_API int spc3d_timer_mark(spc3d_ctx *ctx, int slot);
SPC3D_API int spc3d_timer_elapsed_ms(spc3d_ctx *ctx, int start, int stop, float *ms);

/* ---- dense panels: denseMatrix (src/basic.hpp:30-44) ------------------- */
SPC3D_API int spc3d_panel_create(spc3d_ctx *ctx, int dtype, uint32_t m, uint32_t n, spc3d_panel **out);
/* A panel over the caller's own device memory (m*n reals, row-major, 16-byte aligned,
 * on the context's GPU): a receive buffer of a collective, a block of rows of a
 * larger panel (dev + r0*n reals), a tensor of another library.  Nothing is copied
 * and spc3d_panel_destroy leaves the memory alone; it must outlive the panel and
 * every call queued on it.  No counterpart in the reference, whose panels are host
 * vectors. */
SPC3D_API int spc3d_panel_wrap(spc3d_ctx *ctx, int dtype, uint32_t m, uint32_t n, void *dev,
                     spc3d_panel **out);
SPC3D_API int spc3d_panel_destroy(spc3d_panel *p);
SPC3D_API int spc3d_panel_upload(spc3d_panel *p, const void *host);   /* m*n reals, row-major */
SPC3D_API int spc3d_panel_download(spc3d_panel *p, void *host);
SPC3D_API int spc3d_panel_fill(spc3d_panel *p, double value);
/* dst = src on the device (same shape and dtype); e.g. resetting Y to Y0 between runs. */
SPC3D_API int spc3d_panel_copy(spc3d_panel *dst, const spc3d_panel *src);
SPC3D_API int spc3d_panel_device_ptr(spc3d_panel *p, void **dev);
SPC3D_API int spc3d_panel_shape(spc3d_panel *p, uint32_t *m, uint32_t *n, int *dtype);

/* ---- value vectors: cooMat::vv (src/SparseMatrix.hpp:36) --------------- */
SPC3D_API int spc3d_vals_create(spc3d_ctx *ctx, int dtype, uint64_t n, spc3d_vals **out);
/* The same for a value vector of n reals (see spc3d_panel_wrap). */
SPC3D_API int spc3d_vals_wrap(spc3d_ctx *ctx, int dtype, uint64_t n, void *dev, spc3d_vals **out);
SPC3D_API int spc3d_vals_destroy(spc3d_vals *v);
SPC3D_API int spc3d_vals_upload(spc3d_vals *v, const void *host);
SPC3D_API int spc3d_vals_download(spc3d_vals *v, void *host);
SPC3D_API int spc3d_vals_fill(spc3d_vals *v, double value);
SPC3D_API int spc3d_vals_device_ptr(spc3d_vals *v, void **dev);
/* dst[dst_off .. dst_off + n) = src[src_off .. src_off + n) on the device (same dtype, ranges
 * that do not overlap): what a message a rank addresses to itself amounts to, sendBuff +
 * sendDisp to recvBuff + recvDisp (src/comm.hpp:113-130), and the Z reduction of SDDMM over
 * one rank, C.vv to C.ownedVals (src/denseComm.hpp:39).  Asynchronous on the context's
 * stream; may be recorded. */
SPC3D_API int spc3d_vals_copy(spc3d_vals *dst, uint64_t dst_off, const spc3d_vals *src,
                    uint64_t src_off, uint64_t n);

/* ---- plan: the sparse operand ------------------------------------------ */
/* Host-only check of a COO pattern; needs no GPU.  Mirrors the bounds checks
 * of core_ops.cpp:16,32 (.at()): SPC3D_ERR_BAD_INDEX names the first bad entry
 * in spc3d_last_error(). */
SPC3D_API int spc3d_coo_validate(uint32_t nrows, uint32_t ncols, uint64_t nnz,
                       const uint32_t *ii, const uint32_t *jj);

/* Validates (as above), groups the entries by row keeping the caller's order
 * within a row, and cuts long rows into segments.  By default the pattern is
 * uploaded as it is and all of this happens on the GPU (histograms, scans and
 * stable radix sorts; milliseconds for 16 M entries); spc3d_plan_opts.builder or
 * SPC3D_PLAN_BUILDER=host in the environment (spc3d_plan_create only) selects
 * the single-threaded host builder instead.  How spc3d_sddmm brings its results to
 * the caller's positions is settled here as well (spc3d_plan_info: staged_entries,
 * positions_by_segment, sddmm_by_column, two_pass_results; spc3d_plan_opts.flags keeps the
 * plain form, and for spc3d_plan_create and the one-shot host calls, which take no options,
 * so do SPC3D_STAGE_STORES=0, SPC3D_SDDMM_BY_COLUMN=0 and SPC3D_TWO_PASS=0 in the
 * environment, read once per plan).  `vv` (nnz reals of
 * `dtype`, caller's order) may be NULL and set later.  The pattern is copied:
 * the caller's arrays are not referenced afterwards.  Replaces nothing in the
 * reference (it walks the unsorted COO directly, core_ops.cpp:7-10); it is the
 * amortised set-up for the five identical calls the benches make
 * (miniapp/bench_both.cpp:202-203, bench_spmm.cpp:185-186). */
SPC3D_API int spc3d_plan_create(spc3d_ctx *ctx, int dtype, uint32_t nrows, uint32_t ncols,
                      uint64_t nnz, const uint32_t *ii, const uint32_t *jj,
                      const void *vv, spc3d_plan **out);
/* As above with explicit tuning (NULL = defaults). */
SPC3D_API int spc3d_plan_create_ex(spc3d_ctx *ctx, int dtype, uint32_t nrows, uint32_t ncols,
                         uint64_t nnz, const uint32_t *ii, const uint32_t *jj,
                         const void *vv, const spc3d_plan_opts *opts, spc3d_plan **out);
/* Host-only: builds the same kernel-order form spc3d_plan_create_ex uploads and
 * hands it back, for inspection and for testing without a GPU.  `info` is
 * always filled.  Each output may be NULL; otherwise col and perm hold nnz
 * entries (perm[p] = caller's position of kernel-order entry p), segs holds
 * 4 words per stored segment {row, start, len, slot} (slot 0xFFFFFFFF: the
 * segment is the whole row; len 0: padding) and needs
 * seg_cap >= info->nsegments_padded, splits holds 3 words per cut row
 * {row, first_slot, nslots} and needs split_cap >= info->nsplit_rows; a
 * capacity that is too small gives SPC3D_ERR_SIZE_MISMATCH. */
SPC3D_API int spc3d_plan_build_host(int dtype, uint32_t nrows, uint32_t ncols, uint64_t nnz,
                          const uint32_t *ii, const uint32_t *jj,
                          const spc3d_plan_opts *opts, spc3d_plan_info *info,
                          uint32_t *col, uint32_t *perm, uint32_t *segs, uint32_t seg_cap,
                          uint32_t *splits, uint32_t split_cap);
/* As spc3d_plan_create_ex for a pattern that already lives on the GPU: dev_ii and
 * dev_jj are device pointers to nnz uint32 each (memory of the context's
 * device, e.g. from spc3d_vals_device_ptr or the caller's own hipMalloc), read
 * on the context's stream.  The plan has no values until spc3d_plan_set_values[_device].
 * Has no counterpart in the reference, whose COO lives in host vectors
 * (src/SparseMatrix.hpp:35). */
SPC3D_API int spc3d_plan_create_from_device(spc3d_ctx *ctx, int dtype, uint32_t nrows,
                                  uint32_t ncols, uint64_t nnz, const void *dev_ii,
                                  const void *dev_jj, const spc3d_plan_opts *opts,
                                  spc3d_plan **out);
/* The index transforms the reference runs before its kernels, for index arrays
 * that live on the GPU (device pointers to n uint32 of the context's device).
 * spc3d_localize_device = COOMatrix::localizeIndices (src/SparseMatrix.hpp:69-99)
 * for one of the two arrays: every distinct value gets the next local id the
 * first time it appears in the array, dev_idx[e] is replaced by its local id,
 * dev_ltg[local] (capacity n) receives the value and *nlocal the number of ids
 * (the reference's nrows / ncols and ltgR / ltgC; call it once for ii, once for
 * jj).  spc3d_remap_device = COOMatrix::ReMapIndices (src/SparseMatrix.hpp:100-106):
 * dev_idx[e] = dev_map[dev_idx[e]]; an index >= map_len gives SPC3D_ERR_BAD_INDEX
 * (the reference's .at()) and changes nothing.  Both synchronous. */
SPC3D_API int spc3d_localize_device(spc3d_ctx *ctx, uint64_t n, void *dev_idx, void *dev_ltg,
                          uint32_t *nlocal);
SPC3D_API int spc3d_remap_device(spc3d_ctx *ctx, uint64_t n, void *dev_idx, const void *dev_map,
                       uint32_t map_len);
/* Copies a plan's arrays back from the device, in the layout of
 * spc3d_plan_build_host (each output may be NULL; perm is the identity when the
 * plan stores none).  For inspection and tests.  Synchronous. */
SPC3D_API int spc3d_plan_download(spc3d_plan *plan, uint32_t *col, uint32_t *perm, uint32_t *segs,
                        uint32_t seg_cap, uint32_t *splits, uint32_t split_cap);
SPC3D_API int spc3d_plan_destroy(spc3d_plan *plan);
SPC3D_API int spc3d_plan_set_values(spc3d_plan *plan, const void *vv_host);       /* caller's COO order */
SPC3D_API int spc3d_plan_set_values_device(spc3d_plan *plan, const spc3d_vals *vv); /* caller's COO order */
SPC3D_API int spc3d_plan_get_info(const spc3d_plan *plan, spc3d_plan_info *info);
/* Measurement aid, for the floors a benchmark quotes beside its timings; has no counterpart
 * in the reference.  Rewrites the columns of a plan's entries in place on the device, so
 * that the same launches over the same segments, queues and streams find every gathered
 * dense row in the L2 (SPC3D_PROBE_ALL_HIT: column c becomes c % modulus, inside its own
 * block of columns for a plan kept in column blocks; choose modulus * K * sizeof(real) well
 * under one 4 MiB L2) or nearly none of them (SPC3D_PROBE_ALL_MISS: a hash of the entry's
 * position, uniform over all columns; modulus is ignored).  The plan afterwards computes
 * another pattern than the caller's: time it, then destroy it.  Synchronous. */
#define SPC3D_PROBE_ALL_HIT 1
#define SPC3D_PROBE_ALL_MISS 2
SPC3D_API int spc3d_plan_probe_columns(spc3d_plan *plan, int mode, uint32_t modulus);

/* ---- the hot path -------------------------------------------------------
 * spc3d_sddmm  = SpKernels::sddmm (src/core_ops.cpp:5-22):
 *     C[e] = S.vv[e] * sum_j A[ii[e],j] * B[jj[e],j],  e in the caller's order.
 *     K = A.n (core_ops.cpp:6); requires B.n == K, A.m >= nrows, B.m >= ncols,
 *     C length >= nnz, all dtypes equal to the plan's.
 * spc3d_spmm   = SpKernels::spmm  (src/core_ops.cpp:24-35):
 *     Y[ii[e],:] += A.vv[e] * X[jj[e],:]   (accumulates; duplicates add).
 *     K = X.n (core_ops.cpp:25); requires Y.n == K, X.m >= ncols, Y.m >= nrows.
 * Both are asynchronous on the context's stream. */
SPC3D_API int spc3d_sddmm(spc3d_ctx *ctx, spc3d_plan *S, const spc3d_panel *A,
                const spc3d_panel *B, spc3d_vals *C);
SPC3D_API int spc3d_spmm(spc3d_ctx *ctx, spc3d_plan *A, const spc3d_panel *X, spc3d_panel *Y);
/* spc3d_spmm for callers that cannot allocate device memory (code under HIP graph
 * capture that was never primed, tight serving loops, harnesses that forbid
 * hipMalloc): has no counterpart in the reference.  Same operands, checks and
 * results as spc3d_spmm, bit for bit (the same kernels in the same order); the
 * partial sums of rows that the plan cut into several segments go to an array of
 * SPC3D_NOALLOC_SCRATCH_BYTES that is part of the library's device code (each GPU the
 * library is used on holds it until the process ends) instead of to memory owned by
 * the plan, and the call performs no allocation and frees nothing.  A plan whose
 * partial sums need more (npartial_slots * K * sizeof(real) bytes) is refused with
 * SPC3D_ERR_TOO_LARGE and nothing is queued.  All calls on one GPU share the array:
 * two such calls must not overlap in time (calls on one context never do; contexts
 * on the same GPU must not run it concurrently).  Asynchronous on the context's
 * stream; may be recorded between spc3d_capture_begin and spc3d_capture_end. */
#define SPC3D_NOALLOC_SCRATCH_BYTES (32u << 20)
SPC3D_API int spc3d_spmm_noalloc(spc3d_ctx *ctx, spc3d_plan *A, const spc3d_panel *X,
                       spc3d_panel *Y);
/* Both kernels over one pattern and one dense operand B in a single pass, so that
 * each gathered row of B is used twice: C as spc3d_sddmm(ctx, S, A, B, C), and
 *   chained == 0:  Y += S B, as spc3d_spmm(ctx, S, B, Y) with S's own values;
 *   chained != 0:  Y += C B, the SpMM whose sparse values are the SDDMM result
 *                  just computed (what calling spc3d_plan_set_values_device(S, C)
 *                  and spc3d_spmm(ctx, S, B, Y) afterwards would give, without
 *                  changing the plan's values).
 * Same results as the separate calls within the summation-order tolerance;
 * requires A.n == B.n == Y.n, Y.m >= nrows, Y aliasing neither A nor B.  The
 * chained form needs dense rows of at most 4096 bytes (K <= 1024 in fp32, 512 in
 * fp64; SPC3D_ERR_INVALID_ARG otherwise); the other falls back to the two calls.
 * Has no counterpart in the reference, which runs its two kernels in separate
 * passes (miniapp/bench_both.cpp:202-203; miniapp/bench_spmm.cpp:185-186).
 * Asynchronous on the context's stream. */
SPC3D_API int spc3d_sddmm_spmm(spc3d_ctx *ctx, spc3d_plan *S, const spc3d_panel *A,
                     const spc3d_panel *B, spc3d_vals *C, spc3d_panel *Y, int chained);

/* ---- the copies either side of a sparse exchange ---------------------------
 * A row map ties buffer slot i to dense row rows[i] of a panel: the device form
 * of SparseComm::sendptr / recvptr (src/comm.hpp:41,49; one pointer per row of
 * dataUnitSize = K reals).  Rows may repeat (several peers can return partial
 * sums of one row).  rows[i] < panel_rows is checked on the host
 * (SPC3D_ERR_BAD_INDEX).  The buffer is an spc3d_vals of at least n * K reals,
 * slot after slot, as sendBuff / recvBuff are.
 *   spc3d_rows_pack       = copy_to_sendbuff   (src/comm.hpp:90-103):  buf[i,:]  = P[rows[i],:]
 *   spc3d_rows_unpack     = copy_from_recvbuff (src/comm.hpp:166-177): P[rows[i],:]  = buf[i,:]
 *   spc3d_rows_unpack_sum = SUM_from_recvbuff  (src/comm.hpp:178-189): P[rows[i],:] += buf[i,:]
 * For a repeated row the results are those of the reference's sequential loop:
 * the last slot wins (unpack), slots are added in ascending order (unpack_sum,
 * no atomics).  Asynchronous on the context's stream. */
typedef struct spc3d_rowmap spc3d_rowmap;
SPC3D_API int spc3d_rowmap_create(spc3d_ctx *ctx, uint32_t panel_rows, uint64_t n,
                        const uint32_t *rows, spc3d_rowmap **out);
SPC3D_API int spc3d_rowmap_destroy(spc3d_rowmap *map);
SPC3D_API int spc3d_rows_pack(spc3d_ctx *ctx, const spc3d_panel *P, const spc3d_rowmap *map,
                    spc3d_vals *buf);
SPC3D_API int spc3d_rows_unpack(spc3d_ctx *ctx, spc3d_panel *P, const spc3d_rowmap *map,
                      const spc3d_vals *buf);
SPC3D_API int spc3d_rows_unpack_sum(spc3d_ctx *ctx, spc3d_panel *P, const spc3d_rowmap *map,
                          const spc3d_vals *buf);

/* One-shot forms over host memory with exactly the reference's operands
 * (SpKernels::sddmm / spmm, src/core_ops.hpp:9-12, on the data() of the caller's
 * vectors).  Synchronous: the results are in cvv / Y when the call returns.
 *
 * The reference's drivers call the kernel five times over one pattern and the same
 * panels (miniapp/bench_both.cpp:202-203, bench_spmm.cpp:185-186), so the context keeps
 * what a call built for the next one, decided by CONTENT, never by address (ReMapIndices
 * rewrites ii / jj in place between groups of calls, bench_both.cpp:200-205):
 *   - up to four plans, reused when every 4 MiB block of ii and of jj has the key it had
 *     when the plan was made (four CRC-32C streams, a sum and a fold over every word),
 *     nnz, sizes, type and k agree, and a sample of the indices compares equal; a new
 *     pattern is planned, and validated, as before;
 *   - up to six device panels with the keys of the host memory they equal: blocks of
 *     A, B, X whose key is unchanged are not sent again, changed blocks are.  Y, which the
 *     kernel changes, is fetched into the caller's memory in pieces that are keyed while
 *     the next piece is on its way, so the next call sends only what the caller touched
 *     since (a caller that rewrites most of Y between calls is noticed, and Y then goes
 *     up unread for a stretch of calls that doubles, up to 16, each time that proves
 *     right); Y goes up on a thread of its own while X is read for its keys.  The values
 *     svv / avv are sent on every call;
 *   - the result vector of SDDMM.
 * Reading an unchanged operand for its keys (several threads) takes about half the time
 * of sending it.  The cache holds device memory until spc3d_host_cache_clear or
 * spc3d_ctx_destroy; a context created with SPC3D_CTX_NO_HOST_CACHE does plan, upload, run,
 * download, free on every call instead.  The reading and the Y transfers use the context's
 * host_threads (spc3d_ctx_opts): with the default, 1, everything runs on the caller's thread.  One-shot calls on one context run one at a time
 * (they take a lock).  The kernels of the last one-shot call lie between the timer slots
 * SPC3D_TIMER_HOST_CALL_BEGIN and _END. */
#define SPC3D_TIMER_HOST_CALL_BEGIN 4094
#define SPC3D_TIMER_HOST_CALL_END 4095
SPC3D_API int spc3d_sddmm_host(spc3d_ctx *ctx, int dtype, uint32_t m, uint32_t n, uint32_t k,
                     const void *A, const void *B, uint64_t nnz, const uint32_t *ii,
                     const uint32_t *jj, const void *svv, void *cvv);
SPC3D_API int spc3d_spmm_host(spc3d_ctx *ctx, int dtype, uint32_t ncols, uint32_t nrows, uint32_t k,
                    const void *X, uint64_t nnz, const uint32_t *ii, const uint32_t *jj,
                    const void *avv, void *Y);
/* Frees what the one-shot calls keep (no counterpart in the reference, whose operands
 * live in host vectors). */
SPC3D_API int spc3d_host_cache_clear(spc3d_ctx *ctx);
/* What the last one-shot call on this context moved: bytes sent to the device, bytes of
 * dense operands left in place because their content had not changed, and whether the
 * plan was reused (1) or made (0).  Any pointer may be NULL. */
SPC3D_API int spc3d_host_call_stats(spc3d_ctx *ctx, uint64_t *bytes_sent, uint64_t *bytes_kept,
                          int *plan_reused);

#ifdef __cplusplus
}
#endif
#endif /* SPCOMM3D_HIP_H */
