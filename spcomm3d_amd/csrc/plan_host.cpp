// Host-side plan construction: validation, column classification, row
// grouping, segmentation and the dealing of segments to XCD queues.
#include "plan_host.h"

#include <algorithm>
#include <cstdio>
#include <new>

#include "../../include/spcomm3d_hip.h"

namespace spc3d {

int validate_coo(uint32_t nrows, uint32_t ncols, uint64_t nnz, const uint32_t *ii,
                 const uint32_t *jj, std::string &err)
{
    if (nnz > 0 && (ii == nullptr || jj == nullptr)) {
        err = "ii/jj is NULL with nnz > 0";
        return SPC3D_ERR_INVALID_ARG;
    }
    if (nnz >= (1ull << 32)) {
        err = "nnz >= 2^32 is not supported";
        return SPC3D_ERR_TOO_LARGE;
    }
    // Branch-free scan first; locate the offender only if there is one.
    uint32_t bad = 0;
    for (uint64_t e = 0; e < nnz; ++e)
        bad |= (uint32_t)(ii[e] >= nrows) | (uint32_t)(jj[e] >= ncols);
    if (!bad)
        return SPC3D_OK;
    for (uint64_t e = 0; e < nnz; ++e) {
        if (ii[e] >= nrows || jj[e] >= ncols) {
            char buf[160];
            std::snprintf(buf, sizeof buf,
                          "entry %llu = (%u, %u) is outside the %u x %u pattern",
                          (unsigned long long)e, ii[e], jj[e], nrows, ncols);
            err = buf;
            break;
        }
    }
    return SPC3D_ERR_BAD_INDEX;
}

namespace {

constexpr uint8_t kRep = kClsRep, kCold = kClsCold;

struct Piece {
    Seg seg;
    uint8_t queue;
    uint8_t pref = kNoPref; // a free piece: the slice most of its sliced entries belong to
};

inline uint32_t seg_len(const Seg &s) { return s.len; }

// Stable counting sort of `v` by segment length, longest first.
void sort_longest_first(std::vector<Piece> &v, uint32_t seg_max)
{
    std::vector<uint32_t> bucket((size_t)seg_max + 2, 0);
    for (const Piece &p : v)
        ++bucket[seg_max - seg_len(p.seg) + 1];
    for (uint32_t i = 0; i <= seg_max; ++i)
        bucket[i + 1] += bucket[i];
    std::vector<Piece> out(v.size());
    for (const Piece &p : v)
        out[bucket[seg_max - seg_len(p.seg)]++] = p;
    v.swap(out);
}

} // namespace

// nnz / 2048 rounded down to a power of two, within 64 .. 2048; at most 1024 for dense
// rows of 128 bytes and 512 for rows of 64 bytes and less.  One lane group walks a
// segment batch after batch, two memory latencies per batch, and the narrower the rows
// the more segments share a wavefront and the fewer wavefronts a launch has: the
// longest segments then set its duration (R-MAT 20, fp32 K = 16: SDDMM 542 us at 2048,
// 421 at 512; SpMM 322 and 244; at 256-byte rows and more 1024 and 2048 are level).
uint32_t default_seg_max(uint64_t nnz, uint32_t row_bytes)
{
    const uint32_t cap = row_bytes == 0 || row_bytes > 128 ? 2048u : (row_bytes > 64 ? 1024u : 512u);
    uint32_t s = 64;
    while (s < cap && (uint64_t)s * 2 * 2048 <= nnz)
        s *= 2;
    return s;
}

int build_host_plan(uint32_t nrows, uint32_t ncols, uint64_t nnz, const uint32_t *ii,
                    const uint32_t *jj, const PlanOpts &opts, HostPlan &out, std::string &err)
{
    int rc = validate_coo(nrows, ncols, nnz, ii, jj, err);
    if (rc != SPC3D_OK)
        return rc;
    const uint32_t seg_max =
        clamp_seg_max(opts.seg_max ? opts.seg_max : default_seg_max(nnz, opts.row_bytes), nnz);
    const uint32_t hub_min = opts.hub_min ? opts.hub_min : kDefaultHubMin;
    const bool want_slices = opts.xcd_slices == 0 || opts.xcd_slices == kSlices;

    HostPlan P;
    P.nrows = nrows;
    P.ncols = ncols;
    P.nnz = nnz;
    P.seg_max = seg_max;
    try {
        // ---- histograms -------------------------------------------------
        std::vector<uint32_t> rowptr((size_t)nrows + 1, 0), coldeg((size_t)ncols, 0);
        for (uint64_t e = 0; e < nnz; ++e) {
            ++rowptr[(size_t)ii[e] + 1];
            ++coldeg[jj[e]];
        }
        uint32_t touched = 0, maxlen = 0;
        for (uint32_t r = 0; r < nrows; ++r) {
            const uint32_t len = rowptr[(size_t)r + 1];
            touched += len != 0;
            maxlen = std::max(maxlen, len);
            rowptr[(size_t)r + 1] += rowptr[r];
        }
        uint32_t ctouched = 0, maxcdeg = 0;
        for (uint32_t c = 0; c < ncols; ++c) {
            ctouched += coldeg[c] != 0;
            maxcdeg = std::max(maxcdeg, coldeg[c]);
        }
        P.rows_touched = touched;
        P.cols_touched = ctouched;
        P.max_row_nnz = maxlen;

        // ---- column classes (XCD slicing only) -----------------------------
        // One L2 is expected to keep hot_cols dense rows.  A sixth of that goes to
        // the columns replicated in every L2, the rest to this XCD's slice of
        // the next 8 * (5/6) hot_cols columns.  Slicing is used only when the
        // column degrees are skewed enough for that hot set to cover well more
        // than its share of the entries.
        std::vector<uint8_t> cls;
        bool slices = false;
        if (want_slices && opts.hot_cols > 0 && ctouched > opts.hot_cols && nnz > 0) {
            const uint32_t h1 = opts.hot_cols;
            const uint32_t hrep = std::max<uint32_t>(h1 / 6, 1);
            const uint64_t htot =
                std::min<uint64_t>((uint64_t)hrep + (uint64_t)(h1 - hrep) * kSlices, ctouched);
            // columns by degree, highest first (counting sort, stable in column id)
            std::vector<uint32_t> bucket((size_t)maxcdeg + 2, 0);
            for (uint32_t c = 0; c < ncols; ++c)
                if (coldeg[c])
                    ++bucket[maxcdeg - coldeg[c] + 1];
            for (uint32_t d = 0; d <= maxcdeg; ++d)
                bucket[d + 1] += bucket[d];
            std::vector<uint32_t> order(ctouched);
            for (uint32_t c = 0; c < ncols; ++c)
                if (coldeg[c])
                    order[bucket[maxcdeg - coldeg[c]]++] = c;
            uint64_t covered = 0;
            for (uint64_t i = 0; i < htot; ++i)
                covered += coldeg[order[i]];
            const double coverage = (double)covered / (double)nnz;
            const double share = (double)htot / (double)ctouched;
            if (coverage >= 0.2 && coverage >= 2.0 * share) {
                slices = true;
                cls.assign((size_t)ncols, kCold);
                for (uint64_t i = 0; i < htot; ++i)
                    cls[order[i]] = i < hrep ? kRep : slice_of_rank(i - hrep);
                P.hot_cols = (uint32_t)htot;
                P.hot_entries = covered;
            }
        }

        // ---- hub rows: group counts -------------------------------------------
        // A hub row's entries are grouped [slice 0 | ... | slice 7 | cold], its
        // replicated-hot entries riding with slice rep_slice(row).  Other rows
        // keep the caller's order.
        std::vector<int32_t> hubidx;
        std::vector<uint32_t> hubcnt; // 9 group counts per hub row
        auto group_of = [&](uint32_t r, uint32_t c) -> uint32_t { return hub_group(r, cls[c]); };
        if (slices) {
            hubidx.assign((size_t)nrows, -1);
            uint32_t nh = 0;
            for (uint32_t r = 0; r < nrows; ++r)
                if (rowptr[(size_t)r + 1] - rowptr[r] >= hub_min)
                    hubidx[r] = (int32_t)nh++;
            P.hub_rows = nh;
            hubcnt.assign((size_t)nh * 9, 0);
            for (uint64_t e = 0; e < nnz; ++e)
                if (hubidx[ii[e]] >= 0)
                    ++hubcnt[(size_t)hubidx[ii[e]] * 9 + group_of(ii[e], jj[e])];
        }

        // ---- stable scatter into kernel order ------------------------------
        // Rows that arrive unsorted: the entries are visited in ascending column order
        // (a stable counting sort), so that every row ends up ordered by column.
        std::vector<uint32_t> visit;
        {
            bool down = false;
            for (uint64_t e = 1; e < nnz && !down; ++e)
                down = ii[e - 1] > ii[e];
            if (down && !opts.keep_entry_order) {
                std::vector<uint32_t> at((size_t)ncols + 1, 0);
                for (uint32_t c = 0; c < ncols; ++c)
                    at[(size_t)c + 1] = at[c] + coldeg[c];
                visit.resize(nnz);
                for (uint64_t e = 0; e < nnz; ++e)
                    visit[at[jj[e]]++] = (uint32_t)e;
                P.by_column_in_rows = true;
            }
        }
        P.col.resize(nnz);
        P.perm.resize(nnz);
        {
            std::vector<uint32_t> cur(rowptr.begin(), rowptr.end() - 1);
            std::vector<uint32_t> cur_h(hubcnt.size()); // hub rows: 9 cursors
            for (uint32_t r = 0; slices && r < nrows; ++r) {
                if (hubidx[r] < 0)
                    continue;
                uint32_t at = rowptr[r];
                for (uint32_t k = 0; k < 9; ++k) {
                    cur_h[(size_t)hubidx[r] * 9 + k] = at;
                    at += hubcnt[(size_t)hubidx[r] * 9 + k];
                }
            }
            uint32_t notid = 0;
            for (uint64_t v = 0; v < nnz; ++v) {
                const uint64_t e = visit.empty() ? v : visit[v];
                const uint32_t r = ii[e];
                const uint32_t p = (slices && hubidx[r] >= 0)
                                       ? cur_h[(size_t)hubidx[r] * 9 + group_of(r, jj[e])]++
                                       : cur[r]++;
                P.perm[p] = (uint32_t)e;
                P.col[p] = jj[e];
                notid |= (uint32_t)(p != (uint32_t)e);
            }
            P.identity = notid == 0;
        }

        // ---- segments --------------------------------------------------------
        std::vector<Piece> pieces;
        pieces.reserve((size_t)touched + nnz / seg_max + (size_t)P.hub_rows * 4 + 1);
        uint32_t nslots = 0;
        std::vector<Piece> rowp;
        // Cuts [start, start+len) into balanced parts of at most seg_max entries.
        auto add_range = [&](uint32_t row, uint32_t start, uint32_t len, uint8_t queue) {
            if (len == 0)
                return;
            const uint32_t parts = (len + seg_max - 1) / seg_max;
            const uint32_t base = len / parts, rem = len % parts;
            uint32_t at = 0;
            for (uint32_t q = 0; q < parts; ++q) {
                const uint32_t l = base + (q < rem ? 1u : 0u);
                rowp.push_back(Piece{Seg{row, start + at, l, kWholeRow}, queue});
                at += l;
            }
        };
        for (uint32_t r = 0; r < nrows; ++r) {
            const uint32_t s = rowptr[r], len = rowptr[(size_t)r + 1] - s;
            if (len == 0)
                continue;
            rowp.clear();
            if (slices && hubidx[r] >= 0) {
                uint32_t at = s;
                for (uint32_t k = 0; k < 9; ++k) {
                    const uint32_t n = hubcnt[(size_t)hubidx[r] * 9 + k];
                    add_range(r, at, n, k < 8 ? (uint8_t)k : kAnyQueue);
                    at += n;
                }
            } else {
                add_range(r, s, len, kAnyQueue);
            }
            if (rowp.size() > 1) {
                P.splits.push_back(SplitRow{r, nslots, (uint32_t)rowp.size(), 0});
                for (Piece &p : rowp)
                    p.seg.slot = nslots++;
            }
            pieces.insert(pieces.end(), rowp.begin(), rowp.end());
        }
        P.nslots = nslots;
        P.nseg_real = (uint32_t)pieces.size();

        // ---- order and deal ----------------------------------------------------
        // Longest first, so that the lane groups of one wavefront run the same
        // trip count; equal lengths keep row order (neighbouring rows of banded
        // patterns share dense rows).
        if (!slices) {
            sort_longest_first(pieces, seg_max);
            P.nqueues = 1;
            P.segs.resize(pieces.size());
            for (size_t i = 0; i < pieces.size(); ++i)
                P.segs[i] = pieces[i].seg;
        } else {
            // Hub pieces go to the queue of their column slice.  Of the rest, longest
            // first, a piece with entries in sliced columns goes to the queue of the
            // slice that holds most of them while that queue has room (deal_plan);
            // the others fill every queue up to the same total: piece i of that order
            // goes to the queue whose share of the unit interval holds the i-th
            // point of a low-discrepancy sequence, shares being proportional to
            // what each queue still lacks.  Any window of consecutive (hence
            // similar) pieces is thereby split among the queues in those
            // proportions, and the rule needs nothing but i, so that a parallel
            // builder deals identically.
            P.nqueues = kSlices;
            std::vector<Piece> queue[kSlices], any;
            uint64_t load[kSlices] = {0}, pref_load[kSlices] = {0}, any_load = 0;
            for (Piece &p : pieces) {
                if (p.queue == kAnyQueue) {
                    // the slice most of its sliced entries belong to (see deal_plan)
                    uint32_t cnt[kSlices] = {0};
                    for (uint32_t q = p.seg.start; q < p.seg.start + seg_len(p.seg); ++q) {
                        const uint8_t c = cls[P.col[q]];
                        if (c < kSlices)
                            ++cnt[c];
                    }
                    // (ties go to the first slice from a start that the row's hash picks, so
                    // that no slice collects the short pieces)
                    uint32_t best = rep_slice(p.seg.row);
                    for (uint32_t k = 1; k < kSlices; ++k) {
                        const uint32_t q = (rep_slice(p.seg.row) + k) % kSlices;
                        if (cnt[q] > cnt[best])
                            best = q;
                    }
                    p.pref = cnt[best] ? (uint8_t)best : kNoPref;
                    if (p.pref < kNoPref)
                        pref_load[p.pref] += seg_len(p.seg) + kSegCost;
                    any.push_back(p);
                    any_load += seg_len(p.seg) + kSegCost;
                } else {
                    queue[p.queue].push_back(p);
                    load[p.queue] += seg_len(p.seg) + kSegCost;
                }
            }
            sort_longest_first(any, seg_max);
            DealPlan deal;
            deal_plan(load, pref_load, any_load, opts.slice_affinity, deal);
            for (size_t i = 0; i < any.size(); ++i)
                queue[deal_queue_pref((uint32_t)i, any[i].pref, deal)].push_back(any[i]);
            size_t nchunks = 0;
            for (uint32_t q = 0; q < kSlices; ++q) {
                sort_longest_first(queue[q], seg_max);
                nchunks = std::max(nchunks, (queue[q].size() + kChunk - 1) / kChunk);
            }
            // Chunk i of queue q is global chunk i * 8 + q; short queues are padded
            // with empty segments.
            P.segs.assign(nchunks * kSlices * kChunk, Seg{0, 0, 0, kWholeRow});
            for (uint32_t q = 0; q < kSlices; ++q)
                for (size_t i = 0; i < queue[q].size(); ++i)
                    P.segs[((i / kChunk) * kSlices + q) * kChunk + i % kChunk] = queue[q][i].seg;
        }
        // Leading whole rounds of chunks (one chunk per queue) made of long
        // segments only; every queue is sorted longest first.
        {
            const size_t round = (size_t)P.nqueues * kChunk;
            size_t rounds = 0;
            while ((rounds + 1) * round <= P.segs.size()) {
                bool all_long = true;
                for (uint32_t q = 0; q < P.nqueues && all_long; ++q)
                    all_long = P.segs[rounds * round + (size_t)q * kChunk + kChunk - 1].len >=
                               kLongSegment;
                if (!all_long)
                    break;
                ++rounds;
            }
            P.nseg_long = (uint32_t)(rounds * round);
        }
    } catch (const std::bad_alloc &) {
        err = "host allocation failed while building the plan";
        return SPC3D_ERR_ALLOC;
    }
    out = std::move(P);
    return SPC3D_OK;
}

} // namespace spc3d
