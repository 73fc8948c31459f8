// Host-side construction of the kernel-order form of a COO pattern.
// Pure C++ (no HIP): testable and usable without a GPU.
#pragma once
#include <cstdint>
#include <string>
#include <vector>

#if defined(__HIPCC__)
#define SPC3D_HD __host__ __device__
#else
#define SPC3D_HD
#endif

namespace spc3d {

// One unit of work for a lane group: `len` consecutive entries of one row in
// kernel order.  slot == kWholeRow: the segment is the whole row (SpMM adds its
// sum straight into Y); otherwise the row was cut and the segment's sum goes to
// partial-sum row `slot`.  len == 0 is padding.
struct Seg {
    uint32_t row;
    uint32_t start;
    uint32_t len;
    uint32_t slot;
};
constexpr uint32_t kWholeRow = 0xFFFFFFFFu;
constexpr uint32_t kChunk = 64; // segments per chunk; one chunk is dealt to one XCD
constexpr uint32_t kLongSegment = 16; // segments this long fill the wide kernel's batches
constexpr uint32_t kFirstCols = 8;    // column indices kept per short segment beside its descriptor

// A row cut into several segments: its partial sums are slots
// [first_slot, first_slot + nslots).
struct SplitRow {
    uint32_t row;
    uint32_t first_slot;
    uint32_t nslots;
    uint32_t pad;
};

// Zero in any field selects the default.
struct PlanOpts {
    uint32_t seg_max = 0;    // longest segment (default: by nnz and row_bytes, 64 .. 2048)
    uint32_t row_bytes = 0;  // bytes of the dense rows the plan will mostly run with (0: unknown)
    uint32_t xcd_slices = 0; // 8 (default): hot columns are dealt to the 8 XCD L2s; 1: off
    uint32_t hot_cols = 0;   // slicing: dense rows one L2 is expected to keep
    uint32_t hub_min = 0;    // slicing: rows with at least this many entries are cut by slice (default 128)
    // A pattern whose rows arrive unsorted (ii steps down somewhere) has no order inside
    // its rows worth keeping for the gathers: its entries are then ordered by column inside
    // every row (equal columns in the caller's order), which is what a row-sorted
    // pattern's entries usually are.  true: always keep the caller's order inside a row.
    bool keep_entry_order = false;
    // slicing: false keeps the free segments dealt by rank alone (no affinity to the slice of
    // their entries, see deal_plan)
    bool slice_affinity = true;
};

struct HostPlan {
    uint32_t nrows = 0, ncols = 0;
    uint64_t nnz = 0;
    uint32_t rows_touched = 0, cols_touched = 0;
    uint32_t max_row_nnz = 0;
    uint32_t seg_max = 0;
    uint32_t nslots = 0;
    uint32_t nseg_real = 0;        // segments with entries (segs.size() includes padding)
    uint32_t nseg_long = 0;        // leading stored segments, a whole number of chunk rounds, all
                                   // of at least kLongSegment entries
    uint32_t nqueues = 1;          // 1, or 8 when chunks are dealt round-robin to XCDs
    uint32_t hot_cols = 0;         // columns dealt to slices or replicated (0: slicing off)
    uint64_t hot_entries = 0;      // entries in those columns
    uint32_t hub_rows = 0;         // rows cut by column slice
    bool identity = true;          // perm[p] == p for all p
    bool by_column_in_rows = false; // unsorted rows: entries ordered by column inside each row
    std::vector<uint32_t> col;     // [nnz] column of kernel-order entry p
    std::vector<uint32_t> perm;    // [nnz] caller's position of kernel-order entry p
    std::vector<Seg> segs;         // chunked: chunk v (64 segments) belongs to queue v % nqueues
    std::vector<SplitRow> splits;
};

constexpr uint32_t kDefaultHubMin = 128;

// ---- column classes of the XCD-sliced layout ---------------------------------
// A "replicated" column is hot enough that every L2 keeps its dense row; a
// "slice s" column (class s < 8) is meant to be kept by the L2 of XCD s, so the
// entries of hub rows in it are queued to XCD s; "cold" columns are not expected
// to stay in any L2.
constexpr uint8_t kClsRep = 8, kClsCold = 9;
constexpr uint8_t kAnyQueue = 0xFF;
constexpr uint32_t kSlices = 8;

// Columns are dealt to slices in degree order, back and forth (0..7, 7..0, ...),
// so that no slice collects the larger column of every round.
SPC3D_HD inline uint8_t slice_of_rank(uint64_t i)
{
    const uint32_t pos = (uint32_t)(i % kSlices);
    return (uint8_t)(((i / kSlices) & 1) ? kSlices - 1 - pos : pos);
}

// Replicated-hot entries of a hub row ride with one of its slices; a hash of
// the row id picks it (low row-id bits correlate with degree in R-MAT-like
// graphs, so they would not spread the rows evenly).
SPC3D_HD inline uint32_t rep_slice(uint32_t row) { return (row * 2654435761u) >> 29; }

// Group (0..7: slice, 8: cold) of an entry of hub row `row` in a column of class `cls`.
SPC3D_HD inline uint32_t hub_group(uint32_t row, uint8_t cls)
{
    return cls == kClsRep ? rep_slice(row) : (cls == kClsCold ? 8u : cls);
}

// ---- dealing of free segments to the 8 XCD queues -------------------------
// A segment weighs its length plus kSegCost (descriptor, dense row, write-back).
constexpr uint32_t kSegCost = 4;
constexpr uint32_t kDealQueues = 8;

// upto[q] = end of queue q's share of [0, 2^32), shares proportional to what
// queue q lacks to reach the mean of (load[] + free_load / 8); upto[7] = 2^32 - 1.
inline void deal_thresholds(const uint64_t (&load)[kDealQueues], uint64_t free_load,
                            uint32_t (&upto)[kDealQueues])
{
    // Water level: queues above it get nothing, the others are filled up to it.
    uint64_t lack[kDealQueues];
    uint64_t level_num = free_load; // level = level_num / active over the active queues
    bool active[kDealQueues];
    uint32_t nact = kDealQueues;
    for (uint32_t q = 0; q < kDealQueues; ++q) {
        active[q] = true;
        level_num += load[q];
    }
    for (bool again = true; again;) {
        again = false;
        for (uint32_t q = 0; q < kDealQueues; ++q)
            if (active[q] && nact > 1 && load[q] * nact > level_num) {
                active[q] = false;
                level_num -= load[q];
                --nact;
                again = true;
            }
    }
    uint64_t total = 0;
    for (uint32_t q = 0; q < kDealQueues; ++q) {
        lack[q] = active[q] ? (level_num / nact > load[q] ? level_num / nact - load[q] : 0) : 0;
        total += lack[q];
    }
    uint64_t acc = 0;
    for (uint32_t q = 0; q < kDealQueues; ++q) {
        acc += total ? lack[q] : 1;
        const uint64_t den = total ? total : kDealQueues;
        // acc / den of 2^32, without overflow: loads are < 2^40 (nnz < 2^32, cost 4)
        const uint64_t hi = (acc << 20) / den; // 20 fractional bits, then 12 more
        const uint64_t t = hi >= (1ull << 20) ? 0xFFFFFFFFull : (hi << 12);
        upto[q] = (uint32_t)(t > 0xFFFFFFFFull ? 0xFFFFFFFFull : t);
    }
    upto[kDealQueues - 1] = 0xFFFFFFFFu;
}

// Queue of the i-th free segment (longest first): the share that holds the i-th
// point of the golden-ratio sequence i * 0x9E3779B9 mod 2^32.
SPC3D_HD inline uint32_t deal_queue(uint32_t i, const uint32_t (&upto)[kDealQueues])
{
    const uint32_t x = i * 0x9E3779B9u;
    uint32_t q = 0;
    while (q + 1 < kDealQueues && x > upto[q])
        ++q;
    return q;
}

// ---- affinity of free segments to a slice ------------------------------------
// A free segment (a row under the hub threshold, or the cold part of a hub row) has no
// queue of its own, but its entries in sliced columns hit only in the L2 of their slice:
// one in eight by chance.  Such a segment PREFERS the slice most of its sliced entries
// belong to (on ties the first from a start picked by the row's hash; kNoPref without any), and is queued there while that queue
// has room below the common level; the others are dealt as before.  R-MAT 20: 32 % instead
// of 12.5 % of the sliced entries of free segments then gather in their slice's XCD.
constexpr uint8_t kNoPref = 8;

struct DealPlan {
    uint32_t keep[kDealQueues]; // a free segment of rank i that prefers q stays with q when
                                // i * 0x85EBCA6B mod 2^32 <= keep[q]
    uint32_t upto[kDealQueues]; // deal_queue() shares for the others
};

// load[q]: work bound to queue q; pref_load[q]: free work that prefers q; free_load: all
// free work (the preferring part included).  Every queue accepts of its preferrers what
// fits under the common level (total / 8), a hashed share of them when they are too many.
inline void deal_plan(const uint64_t (&load)[kDealQueues], const uint64_t (&pref_load)[kDealQueues],
                      uint64_t free_load, bool affinity, DealPlan &out)
{
    uint64_t total = free_load, with_pref[kDealQueues], left = free_load;
    for (uint32_t q = 0; q < kDealQueues; ++q)
        total += load[q];
    const uint64_t level = total / kDealQueues;
    for (uint32_t q = 0; q < kDealQueues; ++q) {
        const uint64_t room = level > load[q] ? level - load[q] : 0;
        const uint64_t want = affinity ? pref_load[q] : 0;
        const uint64_t take = want < room ? want : room;
        // take / want of 2^32 (loads are < 2^40: 24 fractional bits, then 8 more)
        uint64_t k = 0;
        if (want != 0 && take == want)
            k = 0xFFFFFFFFull;
        else if (want != 0)
            k = ((take << 24) / want) << 8;
        out.keep[q] = (uint32_t)(k > 0xFFFFFFFFull ? 0xFFFFFFFFull : k);
        with_pref[q] = load[q] + take;
        left -= take;
    }
    deal_thresholds(with_pref, left, out.upto);
}

// Queue of the free segment of rank i (longest first) with preference `pref`.
SPC3D_HD inline uint32_t deal_queue_pref(uint32_t i, uint8_t pref, const DealPlan &d)
{
    if (pref < kNoPref && i * 0x85EBCA6Bu <= d.keep[pref])
        return pref;
    return deal_queue(i, d.upto);
}

// Default longest segment: long enough that few rows are cut (each cut costs a
// partial-sum row in SpMM), short enough that the longest segments do not
// outlast the rest of the grid: nnz / 2048 rounded down to a power of two,
// within [64, 2048].
uint32_t default_seg_max(uint64_t nnz, uint32_t row_bytes);

// A requested longest segment, brought into [1, 2^20]: the builders keep one counter
// per segment length.
inline uint32_t clamp_seg_max(uint32_t want, uint64_t /*nnz*/)
{
    constexpr uint32_t cap = 1u << 20;
    return want < 1 ? 1 : (want > cap ? cap : want);
}

// Returns 0, or an spc3d_status value with `err` filled.
int validate_coo(uint32_t nrows, uint32_t ncols, uint64_t nnz, const uint32_t *ii,
                 const uint32_t *jj, std::string &err);

// Validates, then builds.  Entries are grouped by row, the caller's order kept
// inside a row (the order the reference accumulates in, core_ops.cpp:26-34) when the
// rows arrive sorted or PlanOpts::keep_entry_order is set, else ascending by column.
// With XCD slicing, the entries of a hub row are further grouped by the slice
// of their column, the caller's order kept inside each group.
int build_host_plan(uint32_t nrows, uint32_t ncols, uint64_t nnz, const uint32_t *ii,
                    const uint32_t *jj, const PlanOpts &opts, HostPlan &out, std::string &err);

} // namespace spc3d
