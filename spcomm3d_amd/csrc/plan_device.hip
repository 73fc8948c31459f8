// Device-side plan construction (see plan_device.h).  Every step restates one
// step of build_host_plan (plan_host.cpp) with a parallel primitive that gives
// the same result: histograms by atomics, prefix sums by device scans, the
// stable counting sorts by stable radix sorts.
#include "plan_device.h"

#include <hip/hip_runtime.h>
#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_scan.hpp>

#include <algorithm>
#include <cstdio>

#include "../../include/spcomm3d_hip.h"

namespace spc3d {
namespace {

constexpr int kTB = 256;

struct Counters { // one device-resident block, zeroed (first_bad: all ones) before use
    uint32_t first_bad;
    uint32_t rows_touched, max_row, cols_touched, max_cdeg;
    uint32_t not_identity;
    uint32_t qcount[kSlices], qlong[kSlices];
    uint32_t nlong;
    uint32_t rows_unsorted;
    unsigned long long covered;
    unsigned long long load[kSlices];
    unsigned long long any_load;
    unsigned long long pref_load[kSlices];
};

// Owning device buffer; freed on scope exit unless released.
template <typename T> struct DBuf {
    T *p = nullptr;
    DBuf() = default;
    DBuf(const DBuf &) = delete;
    DBuf &operator=(const DBuf &) = delete;
    ~DBuf() { reset(); }
    void reset()
    {
        if (p)
            (void)hipFree(p);
        p = nullptr;
    }
    hipError_t alloc(size_t count)
    {
        reset();
        if (count == 0)
            return hipSuccess;
        return hipMalloc((void **)&p, count * sizeof(T));
    }
    T *release()
    {
        T *r = p;
        p = nullptr;
        return r;
    }
};

// Scratch device memory of one call: a few large blocks, handed out front to back
// and freed together when the call returns.  (hipFree waits for the device: forty
// hipMalloc / hipFree pairs per build cost more than all of its kernels.)
class Arena {
  public:
    Arena() = default;
    Arena(const Arena &) = delete;
    Arena &operator=(const Arena &) = delete;
    ~Arena()
    {
        for (int i = 0; i < nblocks_; ++i)
            (void)hipFree(blocks_[i]);
    }
    // Makes sure that the next `bytes` come out of one block.
    hipError_t reserve(size_t bytes)
    {
        if (bytes <= left_)
            return hipSuccess;
        if (nblocks_ == kMaxBlocks)
            return hipErrorOutOfMemory;
        void *b = nullptr;
        const hipError_t e = hipMalloc(&b, bytes);
        if (e != hipSuccess)
            return e;
        blocks_[nblocks_++] = b;
        cur_ = static_cast<char *>(b);
        left_ = bytes;
        return hipSuccess;
    }
    hipError_t take(void **p, size_t bytes)
    {
        *p = nullptr;
        if (bytes == 0)
            return hipSuccess;
        bytes = (bytes + 255) / 256 * 256;
        const hipError_t e = reserve(bytes > left_ && bytes < kMinBlock ? kMinBlock : bytes);
        if (e != hipSuccess)
            return e;
        *p = cur_;
        cur_ += bytes;
        left_ -= bytes;
        return hipSuccess;
    }

  private:
    static constexpr int kMaxBlocks = 64;
    static constexpr size_t kMinBlock = (size_t)4 << 20;
    void *blocks_[kMaxBlocks] = {};
    int nblocks_ = 0;
    char *cur_ = nullptr;
    size_t left_ = 0;
};

// An array in the arena; nothing to free.
template <typename T> struct SBuf {
    T *p = nullptr;
    hipError_t alloc(Arena &a, size_t count)
    {
        return a.take(reinterpret_cast<void **>(&p), count * sizeof(T));
    }
};

inline uint32_t grid_for(uint64_t n)
{
    const uint64_t want = (n + kTB - 1) / kTB;
    const uint64_t cap = 256 * 32;
    return (uint32_t)(want < 1 ? 1 : (want > cap ? cap : want));
}

inline uint32_t small_grid_for(uint64_t n) // kernels that end in one atomic per workgroup
{
    const uint32_t g = grid_for(n);
    return g > 1024 ? 1024 : g;
}

inline int bits_for(uint64_t max_value) // bits needed to hold max_value (at least 1)
{
    int b = 1;
    while (b < 64 && (max_value >> b) != 0)
        ++b;
    return b;
}

#define GRID_STRIDE(i, n)                                                                         \
    for (uint64_t i = (uint64_t)blockIdx.x * kTB + threadIdx.x; i < (n);                         \
         i += (uint64_t)gridDim.x * kTB)

template <typename T> __device__ __forceinline__ T wave_sum(T v)
{
    for (int s = 32; s >= 1; s >>= 1)
        v += __shfl_xor(v, s, 64);
    return v;
}

// Sum (maximum) of v over the workgroup, valid in thread 0; every thread of the
// workgroup calls.  The kernels that count into the Counters block add one value
// per workgroup and run on a small grid: device-wide atomics on a handful of
// addresses are served one after the other, and one per wavefront of a full-size
// grid cost more than the rest of the kernel.
template <typename T> __device__ __forceinline__ T block_sum(T v)
{
    __shared__ T part[kTB / 64];
    v = wave_sum(v);
    __syncthreads(); // an earlier call's part[] has been read
    if ((threadIdx.x & 63) == 0)
        part[threadIdx.x >> 6] = v;
    __syncthreads();
    T t = 0;
    if (threadIdx.x == 0)
        for (int w = 0; w < kTB / 64; ++w)
            t += part[w];
    return t;
}
__device__ __forceinline__ uint32_t block_max(uint32_t v)
{
    __shared__ uint32_t part[kTB / 64];
    for (int s = 32; s >= 1; s >>= 1) {
        const uint32_t o = __shfl_xor(v, s, 64);
        v = v > o ? v : o;
    }
    __syncthreads();
    if ((threadIdx.x & 63) == 0)
        part[threadIdx.x >> 6] = v;
    __syncthreads();
    uint32_t t = 0;
    if (threadIdx.x == 0)
        for (int w = 0; w < kTB / 64; ++w)
            t = t > part[w] ? t : part[w];
    return t;
}

template <typename T> __global__ void fill_k(T *p, uint64_t n, T v)
{
    GRID_STRIDE(i, n) p[i] = v;
}

__global__ void iota_k(uint32_t *p, uint64_t n)
{
    GRID_STRIDE(i, n) p[i] = (uint32_t)i;
}

// Adds 1 to cnt[key] for every lane with a valid key, with one atomic per run of
// equal keys in consecutive lanes (sorted COO puts a whole wavefront on one row,
// and same-address atomics of a wavefront are served one after the other).
__device__ __forceinline__ void count_runs(uint32_t *cnt, uint32_t key, bool valid)
{
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t prev = __shfl_up(key, 1, 64);
    const bool prev_valid = __shfl_up((int)valid, 1, 64) != 0;
    const bool head = valid && (lane == 0 || !prev_valid || prev != key);
    // a run ends where the next head starts or where the keys stop being valid
    const unsigned long long stops = __ballot(head || !valid);
    if (head) {
        const unsigned long long above = lane == 63 ? 0ull : stops >> (lane + 1);
        const uint32_t len = above ? (uint32_t)__ffsll((long long)above) : 64u - lane;
        atomicAdd(cnt + key, len);
    }
}

// The first out-of-range entry, if any; whether the rows ever step down.
__global__ void check_k(const uint32_t *__restrict__ ii, const uint32_t *__restrict__ jj,
                        uint64_t nnz, uint32_t nrows, uint32_t ncols, Counters *C)
{
    uint32_t bad = 0xFFFFFFFFu;
    int down = 0;
    GRID_STRIDE(e, nnz)
    {
        const uint32_t r = ii[e];
        if ((r >= nrows || jj[e] >= ncols) && (uint32_t)e < bad)
            bad = (uint32_t)e;
        down |= e > 0 && ii[e - 1] > r;
    }
    if (bad != 0xFFFFFFFFu)
        atomicMin(&C->first_bad, bad); // rare: the build fails
    down = __syncthreads_or(down);
    if (threadIdx.x == 0 && down)
        atomicOr(&C->rows_unsorted, 1u);
}

// Row histogram of entries sorted by row: whole wavefronts walk the entries
// together and pool their counts, one atomic per run of equal rows.
__global__ void hist_sorted_k(const uint32_t *__restrict__ ii, uint64_t nnz, uint32_t *rowcnt)
{
    const uint64_t stride = (uint64_t)gridDim.x * kTB;
    for (uint64_t base = (uint64_t)blockIdx.x * kTB + (threadIdx.x & ~63u); base < nnz;
         base += stride) {
        const uint64_t e = base + (threadIdx.x & 63u);
        const bool ok = e < nnz;
        count_runs(rowcnt, ok ? ii[e] : 0u, ok);
    }
}

// Histogram from sorted ids: the columns', and the rows' of a pattern that is not
// sorted by row (a device-wide atomic per entry is served at the memory side, 1.5 ms
// for 16 M entries; the radix sort and these two passes take a third of that).
// Where a run of equal ids starts, its position goes to start[id]; where it ends,
// the position after it goes to deg[id] (zeroed before); deg[id] -= start[id] then
// leaves the run's length.  The ids were checked against nbins before.
__global__ void run_bounds_k(const uint32_t *__restrict__ sorted, uint64_t n, uint32_t nbins,
                             uint32_t *start, uint32_t *deg)
{
    GRID_STRIDE(i, n)
    {
        const uint32_t k = sorted[i];
        if (k >= nbins)
            continue;
        if (i == 0 || sorted[i - 1] != k)
            start[k] = (uint32_t)i;
        if (i + 1 == n || sorted[i + 1] != k)
            deg[k] = (uint32_t)(i + 1);
    }
}
__global__ void run_lengths_k(const uint32_t *__restrict__ start, uint64_t nbins, uint32_t *deg)
{
    GRID_STRIDE(c, nbins)
    {
        const uint32_t end = deg[c];
        if (end)
            deg[c] = end - start[c];
    }
}

// Number of non-zero counts and the largest count.
__global__ void stats_k(const uint32_t *__restrict__ cnt, uint64_t n, uint32_t *touched,
                        uint32_t *maxv)
{
    uint32_t t = 0, m = 0;
    GRID_STRIDE(i, n)
    {
        const uint32_t v = cnt[i];
        t += v != 0;
        m = m > v ? m : v;
    }
    t = block_sum(t);
    m = block_max(m);
    if (threadIdx.x == 0) {
        if (t)
            atomicAdd(touched, t);
        if (m)
            atomicMax(maxv, m);
    }
}

__global__ void sum_first_k(const uint32_t *__restrict__ v, uint64_t n, unsigned long long *out)
{
    unsigned long long s = 0;
    GRID_STRIDE(i, n) s += v[i];
    s = block_sum(s);
    if (threadIdx.x == 0 && s)
        atomicAdd(out, s);
}

// Classes of the htot hottest columns (order[] = columns by degree, highest first).
__global__ void classify_k(const uint32_t *__restrict__ order, uint64_t htot, uint32_t hrep,
                           uint8_t *cls)
{
    GRID_STRIDE(i, htot)
    cls[order[i]] = i < hrep ? kClsRep : slice_of_rank(i - hrep);
}

__global__ void hubflag_k(const uint32_t *__restrict__ rowcnt, uint32_t nrows, uint32_t hub_min,
                          uint32_t *flag)
{
    GRID_STRIDE(r, (uint64_t)nrows + 1) flag[r] = (r < nrows && rowcnt[r] >= hub_min) ? 1u : 0u;
}

// Per hub row, the number of entries in each of the 9 groups.  Whole wavefronts
// walk the entries together: per group, the lanes that share the row of the first
// such lane add their count with one atomic (sorted COO puts a wavefront on one or
// two rows), the others one each.
__global__ void hubcount_k(const uint32_t *__restrict__ ii, const uint32_t *__restrict__ jj,
                           uint64_t nnz, const uint32_t *__restrict__ hubflag,
                           const uint32_t *__restrict__ hubpos, const uint8_t *__restrict__ cls,
                           uint32_t *hubcnt)
{
    const uint32_t lane = threadIdx.x & 63u;
    const uint64_t stride = (uint64_t)gridDim.x * kTB;
    for (uint64_t base = (uint64_t)blockIdx.x * kTB + (threadIdx.x & ~63u); base < nnz;
         base += stride) {
        const uint64_t e = base + lane;
        uint32_t r = 0, grp = 0;
        bool hub = false;
        if (e < nnz) {
            r = ii[e];
            hub = hubflag[r] != 0;
            if (hub)
                grp = hub_group(r, cls[jj[e]]);
        }
        if (!__any(hub))
            continue;
        for (uint32_t g = 0; g < 9; ++g) {
            const bool mine = hub && grp == g;
            const unsigned long long m = __ballot(mine);
            if (m == 0)
                continue;
            const int lead = __ffsll((long long)m) - 1;
            const uint32_t r0 = __shfl(r, lead, 64);
            const unsigned long long same = __ballot(mine && r == r0);
            if ((int)lane == lead)
                atomicAdd(hubcnt + (size_t)hubpos[r] * 9 + g, (uint32_t)__popcll(same));
            else if (mine && r != r0)
                atomicAdd(hubcnt + (size_t)hubpos[r] * 9 + g, 1u);
        }
    }
}

// Sort key of entry e: its row, then (hub rows of the sliced layout) its group.
// `visit` (may be null): the keys are laid out in that order of the entries, key[v] = key of
// entry visit[v].
template <typename KeyT>
__global__ void keys_k(const uint32_t *__restrict__ ii, const uint32_t *__restrict__ jj,
                       uint64_t nnz, bool slices, const uint32_t *__restrict__ hubflag,
                       const uint8_t *__restrict__ cls, const uint32_t *__restrict__ visit,
                       KeyT *key)
{
    GRID_STRIDE(v, nnz)
    {
        const uint64_t e = visit ? visit[v] : v;
        const uint32_t r = ii[e];
        if (!slices) {
            key[v] = (KeyT)r;
        } else {
            const uint32_t g = hubflag[r] ? hub_group(r, cls[jj[e]]) : 0u;
            key[v] = (KeyT)(((KeyT)r << 4) | (KeyT)g);
        }
    }
}

// col[p] = jj[perm[p]]; flags an order that is not the identity.
__global__ void gather_cols_k(const uint32_t *__restrict__ jj, const uint32_t *__restrict__ perm,
                              uint64_t nnz, uint32_t *col, Counters *C)
{
    bool moved = false;
    GRID_STRIDE(p, nnz)
    {
        const uint32_t e = perm[p];
        col[p] = jj[e];
        moved |= e != (uint32_t)p;
    }
    if (__any(moved) && (threadIdx.x & 63) == 0)
        atomicOr(&C->not_identity, 1u);
}

__device__ __forceinline__ uint32_t parts_of(uint32_t len, uint32_t seg_max)
{
    return len == 0 ? 0u : (len + seg_max - 1) / seg_max;
}

// Pieces per row; rows cut into several pieces also count as a split row and
// take one partial-sum slot per piece.
__global__ void count_pieces_k(const uint32_t *__restrict__ rowcnt, uint32_t nrows,
                               uint32_t seg_max, bool slices,
                               const uint32_t *__restrict__ hubflag,
                               const uint32_t *__restrict__ hubpos,
                               const uint32_t *__restrict__ hubcnt, uint32_t *npieces,
                               uint32_t *issplit, uint32_t *nslot)
{
    GRID_STRIDE(r, (uint64_t)nrows + 1)
    {
        uint32_t np = 0;
        if (r < nrows) {
            if (slices && hubflag[r]) {
                for (uint32_t k = 0; k < 9; ++k)
                    np += parts_of(hubcnt[(size_t)hubpos[r] * 9 + k], seg_max);
            } else {
                np = parts_of(rowcnt[r], seg_max);
            }
        }
        npieces[r] = np;
        issplit[r] = np > 1;
        nslot[r] = np > 1 ? np : 0u;
    }
}

// Writes the pieces of every row, in row order: balanced parts of at most
// seg_max entries per range (a non-hub row is one range, a hub row one per group).
__global__ void emit_pieces_k(const uint32_t *__restrict__ rowptr, uint32_t nrows,
                              uint32_t seg_max, bool slices,
                              const uint32_t *__restrict__ hubflag,
                              const uint32_t *__restrict__ hubpos,
                              const uint32_t *__restrict__ hubcnt,
                              const uint32_t *__restrict__ piece_off,
                              const uint32_t *__restrict__ split_off,
                              const uint32_t *__restrict__ slot_off, Seg *pseg, uint8_t *pqueue,
                              SplitRow *splits)
{
    GRID_STRIDE(r, nrows)
    {
        const uint32_t np = piece_off[r + 1] - piece_off[r];
        if (np == 0)
            continue;
        const uint32_t s = rowptr[r], len = rowptr[r + 1] - s;
        const bool hub = slices && hubflag[r];
        uint32_t at = piece_off[r];
        uint32_t slot = np > 1 ? slot_off[r] : kWholeRow;
        if (np > 1)
            splits[split_off[r]] = SplitRow{(uint32_t)r, slot_off[r], np, 0u};
        uint32_t start = s;
        const uint32_t ngroups = hub ? 9u : 1u;
        for (uint32_t k = 0; k < ngroups; ++k) {
            const uint32_t n = hub ? hubcnt[(size_t)hubpos[r] * 9 + k] : len;
            if (n == 0)
                continue;
            const uint8_t queue = (hub && k < 8) ? (uint8_t)k : kAnyQueue;
            const uint32_t parts = (n + seg_max - 1) / seg_max;
            const uint32_t base = n / parts, rem = n % parts;
            for (uint32_t q = 0; q < parts; ++q) {
                const uint32_t l = base + (q < rem ? 1u : 0u);
                pseg[at] = Seg{(uint32_t)r, start, l, slot};
                pqueue[at] = queue;
                ++at;
                start += l;
                if (np > 1)
                    ++slot;
            }
        }
    }
}

// Unsliced layout: key for "longest first", and the number of long pieces.
__global__ void len_keys_k(const Seg *__restrict__ pseg, uint64_t n, uint32_t seg_max,
                           uint32_t *key, Counters *C)
{
    uint32_t nl = 0;
    GRID_STRIDE(i, n)
    {
        const uint32_t l = pseg[i].len;
        key[i] = seg_max - l;
        nl += l >= kLongSegment;
    }
    nl = block_sum(nl);
    if (threadIdx.x == 0 && nl)
        atomicAdd(&C->nlong, nl);
}

__global__ void gather_segs_k(const Seg *__restrict__ pseg, const uint32_t *__restrict__ idx,
                              uint64_t n, Seg *out)
{
    GRID_STRIDE(i, n) out[i] = pseg[idx[i]];
}

// Sliced layout, step 1: which pieces are free (any queue), the work already
// bound to each queue, and the work that is free.
__global__ void any_flags_k(const Seg *__restrict__ pseg, const uint8_t *__restrict__ pqueue,
                            uint64_t n, uint32_t *anyflag, Counters *C)
{
    unsigned long long w[kSlices + 1] = {0}; // [8] = free work
    GRID_STRIDE(i, (uint64_t)n + 1)
    {
        if (i == n) {
            anyflag[i] = 0;
            continue;
        }
        const uint8_t q = pqueue[i];
        const unsigned long long wi = (unsigned long long)pseg[i].len + kSegCost;
        anyflag[i] = q == kAnyQueue;
#pragma unroll
        for (uint32_t k = 0; k <= kSlices; ++k)
            w[k] += (k == kSlices ? q == kAnyQueue : q == k) ? wi : 0ull;
    }
#pragma unroll
    for (uint32_t k = 0; k <= kSlices; ++k) {
        const unsigned long long t = block_sum(w[k]);
        if (threadIdx.x == 0 && t)
            atomicAdd(k == kSlices ? &C->any_load : &C->load[k], t);
    }
}

// Step 1b: the slice a free piece prefers (the one most of its sliced entries belong to;
// kNoPref without any), and the free work that prefers each slice.
__global__ void pref_k(const Seg *__restrict__ pseg, const uint8_t *__restrict__ pqueue, uint64_t n,
                       const uint32_t *__restrict__ col, const uint8_t *__restrict__ cls,
                       uint8_t *pref, Counters *C)
{
    unsigned long long w[kSlices] = {0};
    GRID_STRIDE(i, n)
    {
        uint8_t p = kNoPref;
        if (pqueue[i] == kAnyQueue) {
            const Seg g = pseg[i];
            uint32_t cnt[kSlices] = {0};
            for (uint32_t q = g.start; q < g.start + g.len; ++q) {
                const uint8_t c = cls[col[q]];
#pragma unroll
                for (uint32_t k = 0; k < kSlices; ++k)
                    cnt[k] += c == k;
            }
            // ties go to the first slice from a start that the row's hash picks
            const uint32_t first = rep_slice(g.row);
            uint32_t best = first, most = 0;
#pragma unroll
            for (uint32_t k = 0; k < kSlices; ++k)
                most = k == first ? cnt[k] : most;
            for (uint32_t k = 1; k < kSlices; ++k) {
                const uint32_t q = (first + k) % kSlices;
                uint32_t c = 0;
#pragma unroll
                for (uint32_t j = 0; j < kSlices; ++j)
                    c = j == q ? cnt[j] : c;
                if (c > most) {
                    most = c;
                    best = q;
                }
            }
            if (most)
                p = (uint8_t)best;
#pragma unroll
            for (uint32_t k = 0; k < kSlices; ++k)
                w[k] += (most && best == k) ? (unsigned long long)g.len + kSegCost : 0ull;
        }
        pref[i] = p;
    }
#pragma unroll
    for (uint32_t k = 0; k < kSlices; ++k) {
        const unsigned long long t = block_sum(w[k]);
        if (threadIdx.x == 0 && t)
            atomicAdd(&C->pref_load[k], t);
    }
}

// Step 2: the free pieces, compacted in piece order, with their length keys.
__global__ void compact_any_k(const Seg *__restrict__ pseg, const uint32_t *__restrict__ anyflag,
                              const uint32_t *__restrict__ anypos, uint64_t n, uint32_t seg_max,
                              uint32_t *any_idx, uint32_t *any_key)
{
    GRID_STRIDE(i, n)
    if (anyflag[i]) {
        any_idx[anypos[i]] = (uint32_t)i;
        any_key[anypos[i]] = seg_max - pseg[i].len;
    }
}


// Step 3: every piece gets its queue.  The combined list is [bound pieces in piece
// order | free pieces longest first]; its key is (queue, seg_max - len).
__global__ void combine_k(const Seg *__restrict__ pseg, const uint8_t *__restrict__ pqueue,
                          const uint32_t *__restrict__ anyflag,
                          const uint32_t *__restrict__ anypos,
                          const uint32_t *__restrict__ any_sorted,
                          const uint8_t *__restrict__ pref, uint64_t npieces, uint64_t nany,
                          uint32_t seg_max, DealPlan deal, uint32_t *comb_idx, uint32_t *comb_key,
                          Counters *C)
{
    const uint64_t nbound = npieces - nany;
    uint32_t cnt[kSlices] = {0}, lng[kSlices] = {0};
    GRID_STRIDE(t, npieces + nany)
    {
        uint32_t piece, q;
        uint64_t at;
        if (t < npieces) { // a bound piece, at its rank among the bound ones
            if (anyflag[t])
                continue;
            piece = (uint32_t)t;
            q = pqueue[t];
            at = t - anypos[t];
        } else { // the free piece of rank j
            const uint64_t j = t - npieces;
            piece = any_sorted[j];
            q = deal_queue_pref((uint32_t)j, pref[piece], deal);
            at = nbound + j;
        }
        const uint32_t l = pseg[piece].len;
        comb_idx[at] = piece;
        comb_key[at] = q * (seg_max + 1) + (seg_max - l);
#pragma unroll
        for (uint32_t k = 0; k < kSlices; ++k) {
            cnt[k] += q == k;
            lng[k] += q == k && l >= kLongSegment;
        }
    }
#pragma unroll
    for (uint32_t k = 0; k < kSlices; ++k) {
        const uint32_t c = block_sum(cnt[k]), g = block_sum(lng[k]);
        if (threadIdx.x == 0) {
            if (c)
                atomicAdd(&C->qcount[k], c);
            if (g)
                atomicAdd(&C->qlong[k], g);
        }
    }
}

struct QStart {
    uint32_t v[kSlices];
};

// Step 4: piece of rank i in queue q goes to chunk i / 64 of that queue, which is
// global chunk (i / 64) * 8 + q.
__global__ void scatter_segs_k(const Seg *__restrict__ pseg, const uint32_t *__restrict__ idx,
                               const uint32_t *__restrict__ key, uint64_t n, uint32_t seg_max,
                               QStart qstart, Seg *out)
{
    GRID_STRIDE(s, n)
    {
        const uint32_t q = key[s] / (seg_max + 1);
        const uint64_t i = s - qstart.v[q];
        out[((i / kChunk) * kSlices + q) * kChunk + i % kChunk] = pseg[idx[s]];
    }
}

// ---- localizeIndices / ReMapIndices on the device -----------------------------
// head[i] = 1 where a run of equal sorted keys starts (i == n: 0, the scan's total slot)
__global__ void heads_k(const uint32_t *__restrict__ key, uint64_t n, uint32_t *head)
{
    GRID_STRIDE(i, n + 1) head[i] = (i < n && (i == 0 || key[i] != key[i - 1])) ? 1u : 0u;
}

// For every run: the position at which its value first appears in the caller's
// array (the sort is stable, so the head of the run holds it) and the value.
__global__ void run_firsts_k(const uint32_t *__restrict__ key, const uint32_t *__restrict__ pos,
                             const uint32_t *__restrict__ head,
                             const uint32_t *__restrict__ run_of, uint64_t n, uint32_t *first_pos,
                             uint32_t *run_key)
{
    GRID_STRIDE(i, n)
    if (head[i]) {
        first_pos[run_of[i]] = pos[i];
        run_key[run_of[i]] = key[i];
    }
}

// Runs in order of first appearance: the r-th gets local id r.
__global__ void run_ranks_k(const uint32_t *__restrict__ run_order,
                            const uint32_t *__restrict__ run_key, uint64_t nruns,
                            uint32_t *rank_of, uint32_t *ltg)
{
    GRID_STRIDE(r, nruns)
    {
        rank_of[run_order[r]] = (uint32_t)r;
        ltg[r] = run_key[run_order[r]];
    }
}

__global__ void write_local_k(const uint32_t *__restrict__ pos, const uint32_t *__restrict__ head,
                              const uint32_t *__restrict__ run_of,
                              const uint32_t *__restrict__ rank_of, uint64_t n, uint32_t *idx)
{
    // run_of[] is the exclusive scan of head[]: inside a run it already counts the head
    GRID_STRIDE(i, n) idx[pos[i]] = rank_of[run_of[i] + head[i] - 1];
}

__global__ void remap_check_k(const uint32_t *__restrict__ idx, uint64_t n, uint32_t map_len,
                              Counters *C)
{
    GRID_STRIDE(e, n)
    if (idx[e] >= map_len)
        atomicMin(&C->first_bad, (uint32_t)e);
}

__global__ void remap_apply_k(uint32_t *idx, uint64_t n, const uint32_t *__restrict__ map)
{
    GRID_STRIDE(e, n) idx[e] = map[idx[e]];
}

#define HIP_OK(expr)                                                                              \
    do {                                                                                          \
        const hipError_t e_ = (expr);                                                             \
        if (e_ != hipSuccess) {                                                                   \
            err = std::string("device plan: ") + #expr + ": " + hipGetErrorString(e_);            \
            return e_ == hipErrorOutOfMemory ? SPC3D_ERR_ALLOC : SPC3D_ERR_HIP;                   \
        }                                                                                         \
    } while (0)

// Scratch for the device-wide primitives, grown on demand.
struct Temp {
    Arena &arena;
    unsigned char *p = nullptr;
    size_t cap = 0;
    explicit Temp(Arena &a) : arena(a) {}
    hipError_t need(size_t bytes)
    {
        bytes = bytes < 256 ? 256 : bytes; // never null: a null pointer asks for the size again
        if (bytes <= cap)
            return hipSuccess;
        const hipError_t e = arena.take(reinterpret_cast<void **>(&p), bytes);
        cap = e == hipSuccess ? bytes : 0;
        return e;
    }
};

template <typename T>
int exclusive_sum(Temp &tmp, const T *in, T *out, size_t n, hipStream_t st, std::string &err)
{
    size_t bytes = 0;
    HIP_OK(rocprim::exclusive_scan(nullptr, bytes, in, out, T(0), n, rocprim::plus<T>(), st));
    HIP_OK(tmp.need(bytes));
    HIP_OK(rocprim::exclusive_scan(tmp.p, bytes, in, out, T(0), n, rocprim::plus<T>(), st));
    return SPC3D_OK;
}

// Stable ascending sort of (key, value) pairs on key bits [0, bits).
template <typename KeyT>
int sort_pairs(Temp &tmp, const KeyT *kin, KeyT *kout, const uint32_t *vin, uint32_t *vout,
               uint32_t n, int bits, bool descending, hipStream_t st, std::string &err)
{
    size_t bytes = 0;
    if (descending) {
        HIP_OK(rocprim::radix_sort_pairs_desc(nullptr, bytes, kin, kout, vin, vout, (size_t)n, 0u,
                                              (unsigned)bits, st));
        HIP_OK(tmp.need(bytes));
        HIP_OK(rocprim::radix_sort_pairs_desc(tmp.p, bytes, kin, kout, vin, vout, (size_t)n, 0u,
                                              (unsigned)bits, st));
    } else {
        HIP_OK(rocprim::radix_sort_pairs(nullptr, bytes, kin, kout, vin, vout, (size_t)n, 0u,
                                         (unsigned)bits, st));
        HIP_OK(tmp.need(bytes));
        HIP_OK(rocprim::radix_sort_pairs(tmp.p, bytes, kin, kout, vin, vout, (size_t)n, 0u,
                                         (unsigned)bits, st));
    }
    return SPC3D_OK;
}

// Ascending sort of keys on key bits [0, bits).
int sort_keys(Temp &tmp, const uint32_t *kin, uint32_t *kout, uint32_t n, int bits,
              hipStream_t st, std::string &err)
{
    size_t bytes = 0;
    HIP_OK(rocprim::radix_sort_keys(nullptr, bytes, kin, kout, (size_t)n, 0u, (unsigned)bits, st));
    HIP_OK(tmp.need(bytes));
    HIP_OK(rocprim::radix_sort_keys(tmp.p, bytes, kin, kout, (size_t)n, 0u, (unsigned)bits, st));
    return SPC3D_OK;
}

#define LAUNCH(kernel, n, ...)                                                                    \
    hipLaunchKernelGGL(kernel, dim3(grid_for(n)), dim3(kTB), 0, st, __VA_ARGS__)
#define LAUNCH_SMALL(kernel, n, ...)                                                              \
    hipLaunchKernelGGL(kernel, dim3(small_grid_for(n)), dim3(kTB), 0, st, __VA_ARGS__)

#define TRY(expr)                                                                                 \
    do {                                                                                          \
        const int rc_ = (expr);                                                                   \
        if (rc_ != SPC3D_OK)                                                                      \
            return rc_;                                                                           \
    } while (0)

int fetch(hipStream_t st, void *host, const void *dev, size_t bytes, std::string &err)
{
    HIP_OK(hipGetLastError());
    HIP_OK(hipMemcpyAsync(host, dev, bytes, hipMemcpyDeviceToHost, st));
    HIP_OK(hipStreamSynchronize(st));
    return SPC3D_OK;
}

// Sorts the entries into kernel order: perm (kernel position -> caller's
// position) and col.  KeyT is wide enough for (row << 4 | group).
// by_column: the entries are first brought into ascending column order (stable), so that
// every row ends up ordered by column (col_bits: bits of the largest column id).
template <typename KeyT>
int order_entries(Arena &arena, Temp &tmp, hipStream_t st, uint64_t nnz, int key_bits, bool slices,
                  bool by_column, int col_bits, const uint32_t *d_ii, const uint32_t *d_jj,
                  const uint32_t *hubflag, const uint8_t *cls, uint32_t *perm, uint32_t *col,
                  Counters *C, std::string &err)
{
    SBuf<KeyT> key, key_out;
    SBuf<uint32_t> ident;
    HIP_OK(key.alloc(arena, nnz));
    HIP_OK(key_out.alloc(arena, nnz));
    HIP_OK(ident.alloc(arena, nnz));
    LAUNCH(iota_k, nnz, ident.p, nnz);
    const uint32_t *visit = nullptr;
    if (by_column) {
        // col and perm are free until the end: sorted columns (unused) and the visiting order
        TRY(sort_pairs<uint32_t>(tmp, d_jj, col, ident.p, perm, (uint32_t)nnz, col_bits, false, st,
                                 err));
        HIP_OK(hipMemcpyAsync(ident.p, perm, nnz * sizeof(uint32_t), hipMemcpyDeviceToDevice, st));
        visit = ident.p;
    }
    LAUNCH((keys_k<KeyT>), nnz, d_ii, d_jj, nnz, slices, hubflag, cls, visit, key.p);
    TRY(sort_pairs<KeyT>(tmp, key.p, key_out.p, ident.p, perm, (uint32_t)nnz, key_bits, false, st,
                         err));
    LAUNCH(gather_cols_k, nnz, d_jj, perm, nnz, col, C);
    HIP_OK(hipGetLastError());
    return SPC3D_OK;
}

// ---- column blocks ---------------------------------------------------------------
__global__ void block_keys_k(const uint32_t *__restrict__ jj, uint64_t nnz, uint32_t block_cols,
                             uint32_t *key)
{
    GRID_STRIDE(e, nnz) key[e] = jj[e] / block_cols;
}
__global__ void gather_u32_k(const uint32_t *__restrict__ in, const uint32_t *__restrict__ idx,
                             uint64_t n, uint32_t *out)
{
    GRID_STRIDE(e, n) out[e] = in[idx[e]];
}
// first[b] = position of the first entry of block b in the sorted keys (first[nblocks] = n)
__global__ void block_firsts_k(const uint32_t *__restrict__ sorted, uint64_t n, uint32_t nblocks,
                               uint32_t *first)
{
    GRID_STRIDE(i, n + 1)
    {
        const uint32_t lo = i == 0 ? 0u : sorted[i - 1] + 1;
        const uint32_t hi = i == n ? nblocks : sorted[i];
        for (uint32_t b = lo; b <= hi && b <= nblocks; ++b)
            first[b] = (uint32_t)i;
    }
}
// perm[q] = order[off + (perm ? perm[q] : q)]
__global__ void compose_perm_k(const uint32_t *__restrict__ order, const uint32_t *__restrict__ perm,
                               uint64_t n, uint32_t *out)
{
    GRID_STRIDE(q, n) out[q] = order[perm ? perm[q] : (uint32_t)q];
}
// out[perm[q]] = vals[q]
__global__ void scatter_u32_k(const uint32_t *__restrict__ perm, const uint32_t *__restrict__ vals,
                              uint64_t n, uint32_t *out)
{
    GRID_STRIDE(q, n) out[perm[q]] = vals[q];
}
// key[q] = rows[perm ? perm[q] : q] / rows_per_tile
__global__ void tile_keys_k(const uint32_t *__restrict__ rows, const uint32_t *__restrict__ perm,
                            uint64_t n, uint32_t rows_per_tile, uint32_t *key)
{
    GRID_STRIDE(q, n) key[q] = rows[perm ? perm[q] : (uint32_t)q] / rows_per_tile;
}
// rank[sorted[i]] = i
__global__ void ranks_k(const uint32_t *__restrict__ sorted, uint64_t n, uint32_t *rank)
{
    GRID_STRIDE(i, n) rank[sorted[i]] = (uint32_t)i;
}
__global__ void sum_sq_len_k(const Seg *__restrict__ segs, uint64_t n, unsigned long long *out)
{
    unsigned long long s = 0;
    GRID_STRIDE(i, n)
    {
        const unsigned long long l = segs[i].len;
        s += l * l;
    }
    s = block_sum(s);
    if (threadIdx.x == 0 && s)
        atomicAdd(out, s);
}

} // namespace

int build_device_plan(hipStream_t st, uint32_t nrows, uint32_t ncols, uint64_t nnz,
                      const uint32_t *d_ii, const uint32_t *d_jj, const PlanOpts &opts,
                      HostPlan &meta, DevPlanArrays &out, std::string &err)
{
    if (nnz >= (1ull << 32)) {
        err = "nnz >= 2^32 is not supported";
        return SPC3D_ERR_TOO_LARGE;
    }
    if (nnz > 0 && (d_ii == nullptr || d_jj == nullptr)) {
        err = "ii/jj is NULL with nnz > 0";
        return SPC3D_ERR_INVALID_ARG;
    }
    const uint32_t seg_max =
        clamp_seg_max(opts.seg_max ? opts.seg_max : default_seg_max(nnz, opts.row_bytes), nnz);
    const uint32_t hub_min = opts.hub_min ? opts.hub_min : kDefaultHubMin;
    const bool want_slices = opts.xcd_slices == 0 || opts.xcd_slices == kSlices;

    HostPlan P;
    P.nrows = nrows;
    P.ncols = ncols;
    P.nnz = nnz;
    P.seg_max = seg_max;
    out = DevPlanArrays{};
    if (nnz == 0) {
        meta = std::move(P);
        return SPC3D_OK;
    }

    // One block for everything whose size is known now: ten arrays per row, five and
    // a class byte per column, the sorted column ids, two keys and an index per entry,
    // the primitives' scratch.
    Arena arena;
    const size_t key_bytes = bits_for(nrows ? nrows - 1 : 0) + 4 > 32 ? 8 : 4;
    HIP_OK(arena.reserve(((size_t)nrows + 1) * 40 + (size_t)ncols * 17 + (size_t)std::max(nrows, ncols) * 4 +
                         (size_t)nnz * (2 * key_bytes + 8) + (size_t)nnz / 2 + ((size_t)8 << 20)));
    Temp tmp(arena);
    SBuf<Counters> dC;
    Counters hC;
    HIP_OK(dC.alloc(arena, 1));
    HIP_OK(hipMemsetAsync(dC.p, 0, sizeof(Counters), st));
    HIP_OK(hipMemsetAsync(&dC.p->first_bad, 0xFF, sizeof(uint32_t), st));

    // ---- histograms, validation ------------------------------------------------
    SBuf<uint32_t> rowcnt, rowptr, coldeg;
    HIP_OK(rowcnt.alloc(arena, (size_t)nrows + 1));
    HIP_OK(rowptr.alloc(arena, (size_t)nrows + 1));
    HIP_OK(coldeg.alloc(arena, ncols));
    HIP_OK(hipMemsetAsync(rowcnt.p, 0, ((size_t)nrows + 1) * sizeof(uint32_t), st));
    HIP_OK(hipMemsetAsync(coldeg.p, 0, (size_t)ncols * sizeof(uint32_t), st));
    LAUNCH_SMALL(check_k, nnz, d_ii, d_jj, nnz, nrows, ncols, dC.p);
    TRY(fetch(st, &hC, dC.p, sizeof hC, err));
    if (hC.first_bad != 0xFFFFFFFFu) {
        uint32_t r = 0, c = 0;
        TRY(fetch(st, &r, d_ii + hC.first_bad, sizeof r, err));
        TRY(fetch(st, &c, d_jj + hC.first_bad, sizeof c, err));
        char buf[160];
        std::snprintf(buf, sizeof buf, "entry %llu = (%u, %u) is outside the %u x %u pattern",
                      (unsigned long long)hC.first_bad, r, c, nrows, ncols);
        err = buf;
        return SPC3D_ERR_BAD_INDEX;
    }
    bool rows_unsorted = false;
    {
        SBuf<uint32_t> sorted, start;
        HIP_OK(sorted.alloc(arena, nnz));
        HIP_OK(start.alloc(arena, std::max<size_t>(ncols, nrows)));
        rows_unsorted = hC.rows_unsorted != 0;
        if (hC.rows_unsorted) {
            TRY(sort_keys(tmp, d_ii, sorted.p, (uint32_t)nnz, bits_for(nrows ? nrows - 1 : 0), st,
                          err));
            LAUNCH(run_bounds_k, nnz, sorted.p, nnz, nrows, start.p, rowcnt.p);
            LAUNCH(run_lengths_k, nrows, start.p, (uint64_t)nrows, rowcnt.p);
        } else {
            LAUNCH(hist_sorted_k, nnz, d_ii, nnz, rowcnt.p);
        }
        TRY(sort_keys(tmp, d_jj, sorted.p, (uint32_t)nnz, bits_for(ncols ? ncols - 1 : 0), st,
                      err));
        LAUNCH(run_bounds_k, nnz, sorted.p, nnz, ncols, start.p, coldeg.p);
        LAUNCH(run_lengths_k, ncols, start.p, (uint64_t)ncols, coldeg.p);
    }
    LAUNCH_SMALL(stats_k, nrows, rowcnt.p, (uint64_t)nrows, &dC.p->rows_touched, &dC.p->max_row);
    LAUNCH_SMALL(stats_k, ncols, coldeg.p, (uint64_t)ncols, &dC.p->cols_touched, &dC.p->max_cdeg);
    TRY(exclusive_sum(tmp, rowcnt.p, rowptr.p, (size_t)nrows + 1, st, err));
    TRY(fetch(st, &hC, dC.p, sizeof hC, err));
    P.rows_touched = hC.rows_touched;
    P.cols_touched = hC.cols_touched;
    P.max_row_nnz = hC.max_row;
    const uint32_t ctouched = hC.cols_touched, maxcdeg = hC.max_cdeg;

    // ---- column classes (XCD slicing only) ---------------------------------------
    SBuf<uint8_t> cls;
    bool slices = false;
    if (want_slices && opts.hot_cols > 0 && ctouched > opts.hot_cols) {
        const uint32_t h1 = opts.hot_cols;
        const uint32_t hrep = std::max<uint32_t>(h1 / 6, 1);
        const uint64_t htot =
            std::min<uint64_t>((uint64_t)hrep + (uint64_t)(h1 - hrep) * kSlices, ctouched);
        // Columns by degree, highest first, ties in column order (a stable sort);
        // the untouched columns end up last.
        SBuf<uint32_t> colid, order, deg_sorted;
        HIP_OK(colid.alloc(arena, ncols));
        HIP_OK(order.alloc(arena, ncols));
        HIP_OK(deg_sorted.alloc(arena, ncols));
        LAUNCH(iota_k, ncols, colid.p, (uint64_t)ncols);
        TRY(sort_pairs<uint32_t>(tmp, coldeg.p, deg_sorted.p, colid.p, order.p, ncols,
                                 bits_for(maxcdeg), true, st, err));
        LAUNCH_SMALL(sum_first_k, htot, deg_sorted.p, htot, &dC.p->covered);
        TRY(fetch(st, &hC, dC.p, sizeof hC, err));
        const uint64_t covered = hC.covered;
        const double coverage = (double)covered / (double)nnz;
        const double share = (double)htot / (double)ctouched;
        if (coverage >= 0.2 && coverage >= 2.0 * share) {
            slices = true;
            HIP_OK(cls.alloc(arena, ncols));
            LAUNCH(fill_k<uint8_t>, ncols, cls.p, (uint64_t)ncols, kClsCold);
            LAUNCH(classify_k, htot, order.p, htot, hrep, cls.p);
            P.hot_cols = (uint32_t)htot;
            P.hot_entries = covered;
        }
        HIP_OK(hipGetLastError());
    }

    // ---- hub rows: group counts ---------------------------------------------------
    SBuf<uint32_t> hubflag, hubpos, hubcnt;
    uint32_t nh = 0;
    if (slices) {
        HIP_OK(hubflag.alloc(arena, (size_t)nrows + 1));
        HIP_OK(hubpos.alloc(arena, (size_t)nrows + 1));
        LAUNCH(hubflag_k, (uint64_t)nrows + 1, rowcnt.p, nrows, hub_min, hubflag.p);
        TRY(exclusive_sum(tmp, hubflag.p, hubpos.p, (size_t)nrows + 1, st, err));
        TRY(fetch(st, &nh, hubpos.p + nrows, sizeof nh, err));
        P.hub_rows = nh;
        HIP_OK(hubcnt.alloc(arena, (size_t)nh * 9 + 1));
        HIP_OK(hipMemsetAsync(hubcnt.p, 0, ((size_t)nh * 9 + 1) * sizeof(uint32_t), st));
        LAUNCH(hubcount_k, nnz, d_ii, d_jj, nnz, hubflag.p, hubpos.p, cls.p, hubcnt.p);
    }

    // ---- stable sort into kernel order ------------------------------------------------
    DBuf<uint32_t> perm, col;
    HIP_OK(perm.alloc(nnz));
    HIP_OK(col.alloc(nnz));
    {
        const int row_bits = bits_for(nrows ? nrows - 1 : 0);
        const int key_bits = row_bits + (slices ? 4 : 0);
        const bool by_column = rows_unsorted && !opts.keep_entry_order;
        const int col_bits = bits_for(ncols ? ncols - 1 : 0);
        P.by_column_in_rows = by_column;
        if (key_bits <= 32)
            TRY(order_entries<uint32_t>(arena, tmp, st, nnz, key_bits, slices, by_column, col_bits,
                                        d_ii, d_jj, hubflag.p, cls.p, perm.p, col.p, dC.p, err));
        else
            TRY(order_entries<unsigned long long>(arena, tmp, st, nnz, key_bits, slices, by_column,
                                                  col_bits, d_ii, d_jj, hubflag.p, cls.p, perm.p,
                                                  col.p, dC.p, err));
    }

    // ---- segments --------------------------------------------------------------------
    SBuf<uint32_t> npieces, issplit, nslot, piece_off, split_off, slot_off;
    const size_t nr1 = (size_t)nrows + 1;
    HIP_OK(npieces.alloc(arena, nr1));
    HIP_OK(issplit.alloc(arena, nr1));
    HIP_OK(nslot.alloc(arena, nr1));
    HIP_OK(piece_off.alloc(arena, nr1));
    HIP_OK(split_off.alloc(arena, nr1));
    HIP_OK(slot_off.alloc(arena, nr1));
    LAUNCH(count_pieces_k, nr1, rowcnt.p, nrows, seg_max, slices, hubflag.p, hubpos.p, hubcnt.p,
           npieces.p, issplit.p, nslot.p);
    TRY(exclusive_sum(tmp, npieces.p, piece_off.p, (size_t)nrows + 1, st, err));
    TRY(exclusive_sum(tmp, issplit.p, split_off.p, (size_t)nrows + 1, st, err));
    TRY(exclusive_sum(tmp, nslot.p, slot_off.p, (size_t)nrows + 1, st, err));
    uint32_t totals[3] = {0, 0, 0};
    TRY(fetch(st, &totals[0], piece_off.p + nrows, sizeof(uint32_t), err));
    TRY(fetch(st, &totals[1], split_off.p + nrows, sizeof(uint32_t), err));
    TRY(fetch(st, &totals[2], slot_off.p + nrows, sizeof(uint32_t), err));
    const uint32_t np_total = totals[0], nsplit = totals[1];
    P.nslots = totals[2];
    P.nseg_real = np_total;

    // and one for everything sized by the number of pieces
    HIP_OK(arena.reserve((size_t)np_total * 64 + ((size_t)4 << 20)));
    SBuf<Seg> pseg;
    SBuf<uint8_t> pqueue;
    DBuf<SplitRow> splits;
    HIP_OK(pseg.alloc(arena, np_total));
    HIP_OK(pqueue.alloc(arena, np_total));
    HIP_OK(splits.alloc(nsplit));
    LAUNCH(emit_pieces_k, nrows, rowptr.p, nrows, seg_max, slices, hubflag.p, hubpos.p, hubcnt.p,
           piece_off.p, split_off.p, slot_off.p, pseg.p, pqueue.p, splits.p);

    // ---- order and deal --------------------------------------------------------------
    DBuf<Seg> segs;
    uint32_t nseg_padded = 0;
    const int len_bits = bits_for(seg_max);
    if (!slices) {
        SBuf<uint32_t> key, key_out, idx, idx_out;
        HIP_OK(key.alloc(arena, np_total));
        HIP_OK(key_out.alloc(arena, np_total));
        HIP_OK(idx.alloc(arena, np_total));
        HIP_OK(idx_out.alloc(arena, np_total));
        HIP_OK(segs.alloc(np_total));
        LAUNCH_SMALL(len_keys_k, np_total, pseg.p, (uint64_t)np_total, seg_max, key.p, dC.p);
        LAUNCH(iota_k, np_total, idx.p, (uint64_t)np_total);
        TRY(sort_pairs<uint32_t>(tmp, key.p, key_out.p, idx.p, idx_out.p, np_total, len_bits,
                                 false, st, err));
        LAUNCH(gather_segs_k, np_total, pseg.p, idx_out.p, (uint64_t)np_total, segs.p);
        TRY(fetch(st, &hC, dC.p, sizeof hC, err));
        P.nqueues = 1;
        nseg_padded = np_total;
        P.nseg_long = hC.nlong / kChunk * kChunk;
    } else {
        SBuf<uint32_t> anyflag, anypos;
        SBuf<uint8_t> pref;
        HIP_OK(anyflag.alloc(arena, (size_t)np_total + 1));
        HIP_OK(anypos.alloc(arena, (size_t)np_total + 1));
        HIP_OK(pref.alloc(arena, np_total));
        LAUNCH_SMALL(any_flags_k, (uint64_t)np_total + 1, pseg.p, pqueue.p, (uint64_t)np_total,
               anyflag.p, dC.p);
        LAUNCH_SMALL(pref_k, np_total, pseg.p, pqueue.p, (uint64_t)np_total, col.p, cls.p, pref.p,
                     dC.p);
        TRY(exclusive_sum(tmp, anyflag.p, anypos.p, (size_t)np_total + 1, st, err));
        uint32_t nany = 0;
        TRY(fetch(st, &nany, anypos.p + np_total, sizeof nany, err));
        TRY(fetch(st, &hC, dC.p, sizeof hC, err));

        SBuf<uint32_t> any_idx, any_key, any_key_out, any_sorted;
        HIP_OK(any_idx.alloc(arena, nany));
        HIP_OK(any_key.alloc(arena, nany));
        HIP_OK(any_key_out.alloc(arena, nany));
        HIP_OK(any_sorted.alloc(arena, nany));
        if (nany) {
            LAUNCH(compact_any_k, np_total, pseg.p, anyflag.p, anypos.p, (uint64_t)np_total,
                   seg_max, any_idx.p, any_key.p);
            TRY(sort_pairs<uint32_t>(tmp, any_key.p, any_key_out.p, any_idx.p, any_sorted.p, nany,
                                     len_bits, false, st, err));
        }
        uint64_t load[kDealQueues], pref_load[kDealQueues];
        for (uint32_t q = 0; q < kDealQueues; ++q) {
            load[q] = hC.load[q];
            pref_load[q] = hC.pref_load[q];
        }
        DealPlan deal;
        deal_plan(load, pref_load, hC.any_load, opts.slice_affinity, deal);

        SBuf<uint32_t> comb_idx, comb_key, comb_idx_out, comb_key_out;
        HIP_OK(comb_idx.alloc(arena, np_total));
        HIP_OK(comb_key.alloc(arena, np_total));
        HIP_OK(comb_idx_out.alloc(arena, np_total));
        HIP_OK(comb_key_out.alloc(arena, np_total));
        LAUNCH_SMALL(combine_k, (uint64_t)np_total + nany, pseg.p, pqueue.p, anyflag.p, anypos.p,
               any_sorted.p, pref.p, (uint64_t)np_total, (uint64_t)nany, seg_max, deal, comb_idx.p,
               comb_key.p, dC.p);
        const int comb_bits = bits_for((uint64_t)kSlices * ((uint64_t)seg_max + 1) - 1);
        TRY(sort_pairs<uint32_t>(tmp, comb_key.p, comb_key_out.p, comb_idx.p, comb_idx_out.p,
                                 np_total, comb_bits, false, st, err));
        TRY(fetch(st, &hC, dC.p, sizeof hC, err));
        QStart qs;
        uint32_t at = 0, nchunks = 0, rounds = 0xFFFFFFFFu;
        for (uint32_t q = 0; q < kSlices; ++q) {
            qs.v[q] = at;
            at += hC.qcount[q];
            nchunks = std::max(nchunks, (hC.qcount[q] + kChunk - 1) / kChunk);
            rounds = std::min(rounds, hC.qlong[q] / kChunk);
        }
        const uint64_t padded = (uint64_t)nchunks * kSlices * kChunk;
        if (padded >= (1ull << 32)) {
            err = "the padded segment list does not fit 32 bits";
            return SPC3D_ERR_TOO_LARGE;
        }
        nseg_padded = (uint32_t)padded;
        HIP_OK(segs.alloc(nseg_padded));
        LAUNCH(fill_k<Seg>, nseg_padded, segs.p, (uint64_t)nseg_padded, (Seg{0, 0, 0, kWholeRow}));
        LAUNCH(scatter_segs_k, np_total, pseg.p, comb_idx_out.p, comb_key_out.p,
               (uint64_t)np_total, seg_max, qs, segs.p);
        P.nqueues = kSlices;
        P.nseg_long = rounds * kSlices * kChunk;
    }
    HIP_OK(hipGetLastError());
    HIP_OK(hipStreamSynchronize(st));
    P.identity = hC.not_identity == 0;

    out.segs = segs.release();
    out.nseg_padded = nseg_padded;
    out.col = col.release();
    out.perm = P.identity ? nullptr : perm.release();
    out.splits = splits.release();
    out.nsplit = nsplit;
    meta = std::move(P);
    return SPC3D_OK;
}

int localize_device(hipStream_t st, uint64_t n, uint32_t *d_idx, uint32_t *d_ltg,
                    uint32_t *nlocal, std::string &err)
{
    *nlocal = 0;
    if (n == 0)
        return SPC3D_OK;
    if (n >= (1ull << 32)) {
        err = "more than 2^32 - 1 indices are not supported";
        return SPC3D_ERR_TOO_LARGE;
    }
    Arena arena;
    HIP_OK(arena.reserve((size_t)n * 44 + ((size_t)8 << 20))); // ten arrays of at most n + 1, scratch
    Temp tmp(arena);
    SBuf<uint32_t> ident, key, pos, head, run_of;
    HIP_OK(ident.alloc(arena, n));
    HIP_OK(key.alloc(arena, n));
    HIP_OK(pos.alloc(arena, n));
    HIP_OK(head.alloc(arena, n + 1));
    HIP_OK(run_of.alloc(arena, n + 1));
    LAUNCH(iota_k, n, ident.p, n);
    TRY(sort_pairs<uint32_t>(tmp, d_idx, key.p, ident.p, pos.p, (uint32_t)n, 32, false, st, err));
    LAUNCH(heads_k, n + 1, key.p, n, head.p);
    TRY(exclusive_sum(tmp, head.p, run_of.p, (size_t)n + 1, st, err));
    uint32_t nruns = 0;
    TRY(fetch(st, &nruns, run_of.p + n, sizeof nruns, err));

    SBuf<uint32_t> first_pos, run_key, first_sorted, run_order, rank_of;
    HIP_OK(first_pos.alloc(arena, nruns));
    HIP_OK(run_key.alloc(arena, nruns));
    HIP_OK(first_sorted.alloc(arena, nruns));
    HIP_OK(run_order.alloc(arena, nruns));
    HIP_OK(rank_of.alloc(arena, nruns));
    // run_of[i] of a head is its run's index; of the other members it is one more
    LAUNCH(run_firsts_k, n, key.p, pos.p, head.p, run_of.p, n, first_pos.p, run_key.p);
    LAUNCH(iota_k, nruns, ident.p, (uint64_t)nruns);
    TRY(sort_pairs<uint32_t>(tmp, first_pos.p, first_sorted.p, ident.p, run_order.p, nruns,
                             bits_for(n - 1), false, st, err));
    LAUNCH(run_ranks_k, nruns, run_order.p, run_key.p, (uint64_t)nruns, rank_of.p, d_ltg);
    LAUNCH(write_local_k, n, pos.p, head.p, run_of.p, rank_of.p, n, d_idx);
    HIP_OK(hipGetLastError());
    HIP_OK(hipStreamSynchronize(st));
    *nlocal = nruns;
    return SPC3D_OK;
}

int remap_device(hipStream_t st, uint64_t n, uint32_t *d_idx, const uint32_t *d_map,
                 uint32_t map_len, std::string &err)
{
    if (n == 0)
        return SPC3D_OK;
    if (n >= (1ull << 32)) {
        err = "more than 2^32 - 1 indices are not supported";
        return SPC3D_ERR_TOO_LARGE;
    }
    DBuf<Counters> dC;
    Counters hC;
    HIP_OK(dC.alloc(1));
    HIP_OK(hipMemsetAsync(dC.p, 0xFF, sizeof(Counters), st));
    LAUNCH(remap_check_k, n, d_idx, n, map_len, dC.p);
    TRY(fetch(st, &hC, dC.p, sizeof hC, err));
    if (hC.first_bad != 0xFFFFFFFFu) {
        uint32_t v = 0;
        TRY(fetch(st, &v, d_idx + hC.first_bad, sizeof v, err));
        char buf[128];
        std::snprintf(buf, sizeof buf, "index %llu = %u is outside the map of %u entries",
                      (unsigned long long)hC.first_bad, v, map_len);
        err = buf;
        return SPC3D_ERR_BAD_INDEX;
    }
    LAUNCH(remap_apply_k, n, d_idx, n, d_map);
    HIP_OK(hipGetLastError());
    HIP_OK(hipStreamSynchronize(st));
    return SPC3D_OK;
}

} // namespace spc3d

namespace spc3d {

int partition_by_col_block(hipStream_t st, uint64_t nnz, const uint32_t *d_ii, const uint32_t *d_jj,
                           uint32_t ncols, uint32_t nblocks, uint32_t *d_ii_out, uint32_t *d_jj_out,
                           uint32_t *d_order, uint32_t *first, std::string &err)
{
    for (uint32_t b = 0; b <= nblocks; ++b)
        first[b] = 0;
    if (nnz == 0 || nblocks == 0)
        return SPC3D_OK;
    const uint32_t block_cols = (ncols + nblocks - 1) / nblocks;
    Arena arena;
    HIP_OK(arena.reserve((size_t)nnz * 12 + (size_t)nblocks * 4 + ((size_t)8 << 20)));
    Temp tmp(arena);
    SBuf<uint32_t> key, key_out, ident, dfirst;
    HIP_OK(key.alloc(arena, nnz));
    HIP_OK(key_out.alloc(arena, nnz));
    HIP_OK(ident.alloc(arena, nnz));
    HIP_OK(dfirst.alloc(arena, (size_t)nblocks + 1));
    LAUNCH(block_keys_k, nnz, d_jj, nnz, block_cols, key.p);
    LAUNCH(iota_k, nnz, ident.p, nnz);
    TRY(sort_pairs<uint32_t>(tmp, key.p, key_out.p, ident.p, d_order, (uint32_t)nnz,
                             bits_for(nblocks), false, st, err));
    LAUNCH(gather_u32_k, nnz, d_ii, d_order, nnz, d_ii_out);
    LAUNCH(gather_u32_k, nnz, d_jj, d_order, nnz, d_jj_out);
    LAUNCH(block_firsts_k, nnz + 1, key_out.p, nnz, nblocks, dfirst.p);
    TRY(fetch(st, first, dfirst.p, ((size_t)nblocks + 1) * sizeof(uint32_t), err));
    return SPC3D_OK;
}

int compose_perm_device(hipStream_t st, const uint32_t *d_order, const uint32_t *d_perm, uint64_t n,
                        uint32_t *d_out, std::string &err)
{
    if (n == 0)
        return SPC3D_OK;
    LAUNCH(compose_perm_k, n, d_order, d_perm, n, d_out);
    HIP_OK(hipGetLastError());
    return SPC3D_OK;
}

int scatter_device(hipStream_t st, const uint32_t *d_perm, const uint32_t *d_vals, uint64_t n,
                   uint32_t *d_out, std::string &err)
{
    if (n == 0)
        return SPC3D_OK;
    LAUNCH(scatter_u32_k, n, d_perm, d_vals, n, d_out);
    HIP_OK(hipGetLastError());
    return SPC3D_OK;
}

int tile_keys_device(hipStream_t st, const uint32_t *d_rows, const uint32_t *d_perm, uint64_t n,
                     uint32_t rows_per_tile, uint32_t *d_key, std::string &err)
{
    if (n == 0)
        return SPC3D_OK;
    LAUNCH(tile_keys_k, n, d_rows, d_perm, n, rows_per_tile, d_key);
    HIP_OK(hipGetLastError());
    return SPC3D_OK;
}

int stable_ranks_device(hipStream_t st, const uint32_t *d_key, uint64_t n, uint32_t max_key,
                        uint32_t *d_rank, std::string &err)
{
    if (n == 0)
        return SPC3D_OK;
    Arena arena;
    HIP_OK(arena.reserve((size_t)n * 12 + ((size_t)8 << 20)));
    Temp tmp(arena);
    SBuf<uint32_t> key_out, ident, sorted;
    HIP_OK(key_out.alloc(arena, n));
    HIP_OK(ident.alloc(arena, n));
    HIP_OK(sorted.alloc(arena, n));
    LAUNCH(iota_k, n, ident.p, n);
    TRY(sort_pairs<uint32_t>(tmp, d_key, key_out.p, ident.p, sorted.p, (uint32_t)n,
                             bits_for(max_key), false, st, err));
    LAUNCH(ranks_k, n, sorted.p, n, d_rank);
    HIP_OK(hipGetLastError());
    HIP_OK(hipStreamSynchronize(st)); // the arena goes away with this call
    return SPC3D_OK;
}

// One wavefront per segment: flag[p] = 1 for every entry of a segment whose caller's
// positions are not perm[start], perm[start] + 1, ...
__global__ void staged_flags_k(const Seg *__restrict__ segs, uint32_t nseg,
                               const uint32_t *__restrict__ perm, uint32_t *__restrict__ flag)
{
    const uint32_t lane = threadIdx.x & 63u;
    for (uint64_t s = ((uint64_t)blockIdx.x * kTB + threadIdx.x) / 64; s < nseg;
         s += (uint64_t)gridDim.x * (kTB / 64)) {
        const Seg sg = segs[s];
        if (sg.len == 0)
            continue;
        const uint32_t base = perm[sg.start];
        bool bad = false;
        for (uint32_t u = lane; u < sg.len; u += 64)
            bad |= perm[sg.start + u] != base + u;
        const uint32_t any = __any(bad) ? 1u : 0u;
        for (uint32_t u = lane; u < sg.len; u += 64)
            flag[sg.start + u] = any;
    }
}

__global__ void staged_fill_k(const uint32_t *__restrict__ perm, const uint32_t *__restrict__ flag,
                              const uint32_t *__restrict__ idx, uint64_t nnz, uint32_t *perm2,
                              uint32_t *key, uint32_t *val)
{
    GRID_STRIDE(p, nnz)
    {
        if (flag[p]) {
            perm2[p] = (uint32_t)nnz + idx[p];
            key[idx[p]] = perm[p];
            val[idx[p]] = idx[p];
        } else {
            perm2[p] = perm[p];
        }
    }
}

__global__ void adjacent_k(const uint32_t *__restrict__ sorted, uint64_t n, unsigned long long *acc)
{
    unsigned long long c = 0;
    GRID_STRIDE(i, n)
    if (i + 1 < n && sorted[i + 1] == sorted[i] + 1)
        ++c;
    c = wave_sum(c);
    if ((threadIdx.x & 63u) == 0 && c)
        atomicAdd(acc, c);
}

// How many of the n staged results are read next to another one of the same wavefront of
// the final pass (64 consecutive h): src[h] - 1 is the src of another lane.
__global__ void src_neighbours_k(const uint32_t *__restrict__ src, uint64_t n, unsigned long long *acc)
{
    unsigned long long c = 0;
    const uint64_t nround = (n + 63) / 64 * 64;
    GRID_STRIDE(h, nround)
    {
        const uint32_t mine = h < n ? src[h] : 0xFFFFFFFFu;
        bool near = false;
        for (int j = 0; j < 64; ++j)
            near |= __shfl(mine, j) + 1 == mine;
        if (h < n && near)
            ++c;
    }
    c = wave_sum(c);
    if ((threadIdx.x & 63u) == 0 && c)
        atomicAdd(acc, c);
}

int build_store_staging(hipStream_t st, const Seg *d_segs, uint32_t nseg, const uint32_t *d_perm,
                        uint64_t nnz, StoreStaging &out, std::string &err)
{
    out = StoreStaging();
    if (!d_perm || nnz == 0 || nseg == 0 || nnz >= (1ull << 31))
        return SPC3D_OK;
    Arena arena;
    HIP_OK(arena.reserve((size_t)nnz * 8 + ((size_t)8 << 20)));
    Temp tmp(arena);
    SBuf<uint32_t> flag, idx;
    HIP_OK(flag.alloc(arena, nnz));
    HIP_OK(idx.alloc(arena, nnz));
    HIP_OK(hipMemsetAsync(flag.p, 0, (size_t)nnz * 4, st));
    hipLaunchKernelGGL(staged_flags_k, dim3(grid_for((uint64_t)nseg * 64)), dim3(kTB), 0, st, d_segs,
                       nseg, d_perm, flag.p);
    TRY(exclusive_sum<uint32_t>(tmp, flag.p, idx.p, (size_t)nnz, st, err));
    uint32_t last[2] = {0, 0};
    TRY(fetch(st, &last[0], idx.p + (nnz - 1), 4, err));
    TRY(fetch(st, &last[1], flag.p + (nnz - 1), 4, err));
    const uint64_t n = (uint64_t)last[0] + last[1];
    if (n == 0) {
        out.consecutive = true;
        return SPC3D_OK;
    }
    if (nnz + n >= (1ull << 32))
        return SPC3D_OK;
    DBuf<uint32_t> perm2, dst, src;
    HIP_OK(perm2.alloc(nnz));
    HIP_OK(dst.alloc(n));
    HIP_OK(src.alloc(n));
    SBuf<uint32_t> key, val;
    HIP_OK(key.alloc(arena, n));
    HIP_OK(val.alloc(arena, n));
    LAUNCH(staged_fill_k, nnz, d_perm, flag.p, idx.p, nnz, perm2.p, key.p, val.p);
    TRY(sort_pairs<uint32_t>(tmp, key.p, dst.p, val.p, src.p, (uint32_t)n, bits_for(nnz - 1), false,
                             st, err));
    // The final pass pays when it writes runs and reads near what its neighbours read; an
    // arbitrary order of the entries gives neither, and keeps its scattered stores.
    DBuf<unsigned long long> acc;
    HIP_OK(acc.alloc(2));
    HIP_OK(hipMemsetAsync(acc.p, 0, 2 * sizeof(unsigned long long), st));
    LAUNCH_SMALL(adjacent_k, n, dst.p, n, acc.p);
    LAUNCH_SMALL(src_neighbours_k, n, src.p, n, acc.p + 1);
    unsigned long long seen[2] = {0, 0};
    TRY(fetch(st, seen, acc.p, sizeof seen, err));
    if (seen[0] * 2 < n || seen[1] * 2 < n)
        return SPC3D_OK; // (the DBufs free themselves)
    out.perm2 = perm2.release();
    out.dst = dst.release();
    out.src = src.release();
    out.n = n;
    out.consecutive = true;
    return SPC3D_OK;
}

// key1 = tile of the kernel position, then bucket of the caller's position; key2 the other
// way round
__global__ void two_pass_keys_k(const uint32_t *__restrict__ perm, uint64_t n, uint32_t T,
                                uint32_t ntiles, uint32_t *key1, uint32_t *key2)
{
    GRID_STRIDE(p, n)
    {
        const uint32_t t = (uint32_t)(p / T), b = perm[p] / T;
        key1[p] = t * ntiles + b;
        key2[p] = b * ntiles + t;
    }
}

__global__ void two_pass_mid_k(const uint32_t *__restrict__ sp2, const uint32_t *__restrict__ perm,
                               uint64_t n, uint32_t T, uint32_t *mid_of, uint16_t *l2)
{
    GRID_STRIDE(m, n)
    {
        const uint32_t p = sp2[m];
        mid_of[p] = (uint32_t)m;
        l2[perm[p]] = (uint16_t)(m % T);
    }
}

__global__ void two_pass_slots_k(const uint32_t *__restrict__ sp1,
                                 const uint32_t *__restrict__ mid_of, uint64_t n, uint32_t T,
                                 uint16_t *l1, uint32_t *dst1)
{
    GRID_STRIDE(s, n)
    {
        const uint32_t p = sp1[s];
        l1[s] = (uint16_t)(p - (uint32_t)(s / T) * T); // the sort kept every tile in its place
        dst1[s] = mid_of[p];
    }
}

int build_two_pass(hipStream_t st, const uint32_t *d_perm, uint64_t nnz, uint32_t T, TwoPass &out,
                   std::string &err)
{
    out = TwoPass();
    if (!d_perm || T == 0 || T > 65536 || nnz >= (1ull << 32) || nnz < 2ull * T)
        return SPC3D_OK;
    const uint64_t ntiles64 = (nnz + T - 1) / T;
    if (ntiles64 * ntiles64 >= (1ull << 32))
        return SPC3D_OK;
    const uint32_t ntiles = (uint32_t)ntiles64;
    Arena arena;
    HIP_OK(arena.reserve((size_t)nnz * 24 + ((size_t)8 << 20)));
    Temp tmp(arena);
    SBuf<uint32_t> key1, key2, idx, key_out, sp1, sp2, mid_of;
    HIP_OK(key1.alloc(arena, nnz));
    HIP_OK(key2.alloc(arena, nnz));
    HIP_OK(idx.alloc(arena, nnz));
    HIP_OK(key_out.alloc(arena, nnz));
    HIP_OK(sp1.alloc(arena, nnz));
    HIP_OK(sp2.alloc(arena, nnz));
    LAUNCH(two_pass_keys_k, nnz, d_perm, nnz, T, ntiles, key1.p, key2.p);
    LAUNCH(iota_k, nnz, idx.p, nnz);
    const int bits = bits_for(ntiles64 * ntiles64 - 1);
    TRY(sort_pairs<uint32_t>(tmp, key1.p, key_out.p, idx.p, sp1.p, (uint32_t)nnz, bits, false, st,
                             err));
    TRY(sort_pairs<uint32_t>(tmp, key2.p, key_out.p, idx.p, sp2.p, (uint32_t)nnz, bits, false, st,
                             err));
    mid_of.p = key1.p; // the keys are no longer needed
    DBuf<uint16_t> l1, l2;
    DBuf<uint32_t> dst1;
    HIP_OK(l1.alloc(nnz));
    HIP_OK(l2.alloc(nnz));
    HIP_OK(dst1.alloc(nnz));
    LAUNCH(two_pass_mid_k, nnz, sp2.p, d_perm, nnz, T, mid_of.p, l2.p);
    LAUNCH(two_pass_slots_k, nnz, sp1.p, mid_of.p, nnz, T, l1.p, dst1.p);
    HIP_OK(hipGetLastError());
    HIP_OK(hipStreamSynchronize(st));
    out.l1 = l1.release();
    out.l2 = l2.release();
    out.dst1 = dst1.release();
    out.tile = T;
    out.n = nnz;
    return SPC3D_OK;
}

// ---- row tiles x column blocks ("sweep") ---------------------------------------------
// out[perm[q]] = base + q
__global__ void inverse_offsets_k(const uint32_t *__restrict__ perm, uint64_t n, uint32_t base,
                                  uint32_t *out)
{
    GRID_STRIDE(q, n) out[perm[q]] = base + (uint32_t)q;
}

// key[j] = (generation of rank j) << 32 | row of rank j
__global__ void sweep_gen_keys_k(const uint32_t *__restrict__ order, uint32_t nin, uint64_t per_gen,
                                 unsigned long long *key)
{
    GRID_STRIDE(j, nin) key[j] = ((unsigned long long)(j / per_gen) << 32) | order[j];
}

// Tile and local row of the j-th row of the sweep (by generation, inside a generation by row
// number): rpt consecutive rows make a tile (rpt_last in the last generation).
__global__ void sweep_rows_k(const unsigned long long *__restrict__ gen_row, uint32_t nin,
                             uint32_t P, uint32_t R, uint32_t last_gen, uint32_t rpt_last,
                             uint32_t *row_tile, uint32_t *row_local, uint32_t *tile_rows)
{
    GRID_STRIDE(j, nin)
    {
        const uint32_t row = (uint32_t)gen_row[j];
        const uint64_t per_gen = (uint64_t)P * R;
        const uint32_t gen = (uint32_t)(j / per_gen), jl = (uint32_t)(j % per_gen);
        const uint32_t rpt = gen == last_gen ? rpt_last : R;
        const uint32_t t = gen * P + jl / rpt, l = jl % rpt;
        row_tile[row] = t;
        row_local[row] = l;
        tile_rows[(uint64_t)t * R + l] = row;
    }
}

// Sort key of entry e: (tile, block, local row); one past the largest such key for an entry
// of a row outside the sweep (they sort last, in the caller's order).
__global__ void sweep_keys_k(const uint32_t *__restrict__ ii, const uint32_t *__restrict__ jj,
                             uint64_t nnz, const uint32_t *__restrict__ row_tile,
                             const uint32_t *__restrict__ row_local, uint32_t block_cols,
                             uint32_t nb, uint32_t R, unsigned long long rest_key,
                             unsigned long long *key, unsigned long long *nin)
{
    unsigned long long mine = 0;
    GRID_STRIDE(e, nnz)
    {
        const uint32_t r = ii[e], t = row_tile[r];
        if (t == 0xFFFFFFFFu) {
            key[e] = rest_key;
            continue;
        }
        key[e] = ((unsigned long long)t * nb + jj[e] / block_cols) * R + row_local[r];
        ++mine;
    }
    mine = block_sum(mine);
    if (threadIdx.x == 0 && mine)
        atomicAdd(nin, mine);
}

// Of the sorted sweep entries: column, local row, and the (tile, block) bin.
__global__ void sweep_entries_k(const unsigned long long *__restrict__ skey,
                                const uint32_t *__restrict__ perm,
                                const uint32_t *__restrict__ jj, uint64_t n, uint32_t R,
                                uint32_t *col, uint16_t *lrow, uint32_t *bin)
{
    GRID_STRIDE(k, n)
    {
        const unsigned long long key = skey[k];
        bin[k] = (uint32_t)(key / R);
        lrow[k] = (uint16_t)(key % R);
        col[k] = jj[perm[k]];
    }
}

int build_sweep(hipStream_t st, uint32_t nrows, uint32_t ncols, uint64_t nnz, const uint32_t *d_ii,
                const uint32_t *d_jj, uint32_t lanes, uint32_t R, uint32_t nb, uint32_t min_row,
                uint32_t P, SweepPlan &out, std::string &err)
{
    out = SweepPlan();
    if (nnz == 0 || nnz >= (1ull << 32) || lanes == 0 || R == 0 || R > 65536 || nb == 0 || P == 0)
        return SPC3D_OK;
    const uint32_t G = 1024 / lanes;
    if (G == 0)
        return SPC3D_OK;
    const uint32_t block_cols = (ncols + nb - 1) / nb;
    Arena arena;
    HIP_OK(arena.reserve(((size_t)nrows + 1) * 40 + (size_t)nnz * 36 + ((size_t)8 << 20)));
    Temp tmp(arena);
    // ---- rows by length ----
    SBuf<uint32_t> rowcnt, rowid, order, cnt_sorted, row_tile, row_local;
    SBuf<unsigned long long> total, gkey, gkey_sorted;
    HIP_OK(rowcnt.alloc(arena, (size_t)nrows + 1));
    HIP_OK(rowid.alloc(arena, nrows));
    HIP_OK(order.alloc(arena, nrows));
    HIP_OK(cnt_sorted.alloc(arena, nrows));
    HIP_OK(row_tile.alloc(arena, nrows));
    HIP_OK(row_local.alloc(arena, nrows));
    HIP_OK(total.alloc(arena, 1));
    HIP_OK(hipMemsetAsync(rowcnt.p, 0, ((size_t)nrows + 1) * sizeof(uint32_t), st));
    HIP_OK(hipMemsetAsync(total.p, 0, sizeof(unsigned long long), st));
    // one addition per run of equal row numbers inside a wavefront: few for rows that arrive
    // together, one per entry at worst
    LAUNCH(hist_sorted_k, nnz, d_ii, nnz, rowcnt.p);
    // rows by length, longest first, equal lengths in row order; those of at least min_row
    // entries come first and are the sweep's
    LAUNCH(iota_k, nrows, rowid.p, (uint64_t)nrows);
    TRY(sort_pairs<uint32_t>(tmp, rowcnt.p, cnt_sorted.p, rowid.p, order.p, nrows, 32, true, st, err));
    std::vector<uint32_t> lens;
    try {
        lens.resize(nrows);
    } catch (const std::bad_alloc &) {
        err = "host allocation failed";
        return SPC3D_ERR_ALLOC;
    }
    TRY(fetch(st, lens.data(), cnt_sorted.p, (size_t)nrows * sizeof(uint32_t), err));
    uint32_t nin = 0;
    while (nin < nrows && lens[nin] >= min_row && lens[nin] > 0)
        ++nin;
    if (nin == 0)
        return SPC3D_OK;
    // A generation: the next P * R rows by length, which one launch of P tiles takes.  Inside
    // a generation the rows are of similar length, and a tile takes R of them that are
    // consecutive by row number: the tiles of a launch stay level to about a percent, and
    // what a tile reads and writes (its rows of A or Y, its SDDMM results on their way to
    // the caller's order) lies together.  The last generation spreads its rows over the P
    // tiles.
    const uint64_t per_gen = (uint64_t)P * R;
    const uint64_t gens = (nin + per_gen - 1) / per_gen;
    const uint64_t last = nin - (gens - 1) * per_gen; // rows of the last generation
    const uint32_t rpt_last = (uint32_t)((last + P - 1) / P);
    const uint64_t ntiles64 = (gens - 1) * P + (last + rpt_last - 1) / rpt_last;
    if (ntiles64 * nb + 1 >= (1ull << 32))
        return SPC3D_OK;
    const uint32_t ntiles = (uint32_t)ntiles64;
    HIP_OK(gkey.alloc(arena, nin));
    HIP_OK(gkey_sorted.alloc(arena, nin));
    LAUNCH(sweep_gen_keys_k, nin, order.p, nin, per_gen, gkey.p);
    // (values unused: cnt_sorted and rowid are free by now)
    TRY(sort_pairs<unsigned long long>(tmp, gkey.p, gkey_sorted.p, rowid.p, cnt_sorted.p, nin,
                                       32 + bits_for(gens), false, st, err));
    DBuf<uint32_t> tile_rows, perm, col, ptr;
    DBuf<uint16_t> lrow;
    HIP_OK(tile_rows.alloc((size_t)ntiles * R));
    HIP_OK(hipMemsetAsync(tile_rows.p, 0xFF, (size_t)ntiles * R * sizeof(uint32_t), st));
    HIP_OK(hipMemsetAsync(row_tile.p, 0xFF, (size_t)nrows * sizeof(uint32_t), st));
    LAUNCH(sweep_rows_k, nin, gkey_sorted.p, nin, P, R, (uint32_t)(gens - 1), rpt_last, row_tile.p,
           row_local.p, tile_rows.p);
    // ---- entries ----
    SBuf<unsigned long long> key, skey;
    SBuf<uint32_t> ident, bin;
    HIP_OK(key.alloc(arena, nnz));
    HIP_OK(skey.alloc(arena, nnz));
    HIP_OK(ident.alloc(arena, nnz));
    HIP_OK(perm.alloc(nnz));
    const unsigned long long rest_key = (unsigned long long)ntiles * nb * R;
    LAUNCH_SMALL(sweep_keys_k, nnz, d_ii, d_jj, nnz, row_tile.p, row_local.p, block_cols, nb, R,
                 rest_key, key.p, total.p);
    LAUNCH(iota_k, nnz, ident.p, nnz);
    TRY(sort_pairs<unsigned long long>(tmp, key.p, skey.p, ident.p, perm.p, (uint32_t)nnz,
                                       bits_for(rest_key), false, st, err));
    unsigned long long n = 0;
    TRY(fetch(st, &n, total.p, sizeof n, err));
    if (n == 0)
        return SPC3D_OK;
    HIP_OK(col.alloc(n));
    HIP_OK(lrow.alloc(n));
    HIP_OK(bin.alloc(arena, n));
    const uint64_t nbins = (uint64_t)ntiles * nb;
    HIP_OK(ptr.alloc(nbins + 1));
    SBuf<uint32_t> bstart, bcnt;
    HIP_OK(bstart.alloc(arena, nbins));
    HIP_OK(bcnt.alloc(arena, nbins + 1));
    HIP_OK(hipMemsetAsync(bcnt.p, 0, (nbins + 1) * sizeof(uint32_t), st));
    LAUNCH(sweep_entries_k, n, skey.p, perm.p, d_jj, n, R, col.p, lrow.p, bin.p);
    LAUNCH(run_bounds_k, n, bin.p, n, (uint32_t)nbins, bstart.p, bcnt.p);
    LAUNCH(run_lengths_k, nbins, bstart.p, nbins, bcnt.p);
    TRY(exclusive_sum(tmp, bcnt.p, ptr.p, (size_t)nbins + 1, st, err));
    HIP_OK(hipGetLastError());
    HIP_OK(hipStreamSynchronize(st));
    out.perm = perm.release();
    out.col = col.release();
    out.lrow = lrow.release();
    out.ptr = ptr.release();
    out.tile_rows = tile_rows.release();
    out.n = n;
    out.ntiles = ntiles;
    out.nblocks = nb;
    out.rows_per_tile = R;
    out.groups = G;
    out.lanes = lanes;
    out.per_launch = P;
    out.nrows_in = nin;
    return SPC3D_OK;
}

// ii[perm[k]], jj[perm[k]] = row and column of sweep entry k: its tile by bisection over the
// tiles' first bounds, its row from the tile's row list.
__global__ void sweep_coords_k(const uint32_t *__restrict__ ptr, uint32_t ntiles, uint32_t nb,
                               const uint32_t *__restrict__ tile_rows, uint32_t R,
                               const uint16_t *__restrict__ lrow, const uint32_t *__restrict__ col,
                               const uint32_t *__restrict__ perm, uint64_t n, uint32_t *ii,
                               uint32_t *jj)
{
    GRID_STRIDE(k, n)
    {
        uint32_t lo = 0, hi = ntiles; // ptr[lo * nb] <= k < ptr[hi * nb]
        while (hi - lo > 1) {
            const uint32_t mid = lo + (hi - lo) / 2;
            if (ptr[(uint64_t)mid * nb] <= k)
                lo = mid;
            else
                hi = mid;
        }
        const uint32_t at = perm[k];
        ii[at] = tile_rows[(uint64_t)lo * R + lrow[k]];
        jj[at] = col[k];
    }
}

// The same for the entries of a plan in segments (perm null: kernel order is the caller's).
__global__ void seg_coords_k(const Seg *__restrict__ segs, uint64_t nseg,
                             const uint32_t *__restrict__ col, const uint32_t *__restrict__ perm,
                             uint32_t *ii, uint32_t *jj)
{
    GRID_STRIDE(sg, nseg)
    {
        const Seg g = segs[sg];
        for (uint32_t q = g.start; q < g.start + g.len; ++q) {
            const uint32_t at = perm ? perm[q] : q;
            ii[at] = g.row;
            jj[at] = col[q];
        }
    }
}

int sweep_coords_device(hipStream_t st, const SweepPlan &sw, uint32_t *d_ii, uint32_t *d_jj,
                        std::string &err)
{
    if (sw.n == 0)
        return SPC3D_OK;
    LAUNCH(sweep_coords_k, sw.n, sw.ptr, sw.ntiles, sw.nblocks, sw.tile_rows, sw.rows_per_tile,
           sw.lrow, sw.col, sw.perm, sw.n, d_ii, d_jj);
    HIP_OK(hipGetLastError());
    return SPC3D_OK;
}

int seg_coords_device(hipStream_t st, const Seg *d_segs, uint64_t nseg, const uint32_t *d_col,
                      const uint32_t *d_perm, uint32_t *d_ii, uint32_t *d_jj, std::string &err)
{
    if (nseg == 0)
        return SPC3D_OK;
    LAUNCH(seg_coords_k, nseg, d_segs, nseg, d_col, d_perm, d_ii, d_jj);
    HIP_OK(hipGetLastError());
    return SPC3D_OK;
}

int count_adjacent_device(hipStream_t st, const uint32_t *d, uint64_t n, uint64_t *out,
                          std::string &err)
{
    *out = 0;
    if (n < 2)
        return SPC3D_OK;
    DBuf<unsigned long long> acc;
    HIP_OK(acc.alloc(1));
    HIP_OK(hipMemsetAsync(acc.p, 0, sizeof(unsigned long long), st));
    LAUNCH_SMALL(adjacent_k, n, d, n, acc.p);
    unsigned long long seen = 0;
    TRY(fetch(st, &seen, acc.p, sizeof seen, err));
    *out = seen;
    return SPC3D_OK;
}

int inverse_offsets_device(hipStream_t st, const uint32_t *d_perm, uint64_t n, uint32_t base,
                           uint32_t *d_out, std::string &err)
{
    if (n == 0)
        return SPC3D_OK;
    LAUNCH(inverse_offsets_k, n, d_perm, n, base, d_out);
    HIP_OK(hipGetLastError());
    return SPC3D_OK;
}

int gather_u32_device(hipStream_t st, const uint32_t *d_in, const uint32_t *d_idx, uint64_t n,
                      uint32_t *d_out, std::string &err)
{
    if (n == 0)
        return SPC3D_OK;
    LAUNCH(gather_u32_k, n, d_in, d_idx, n, d_out);
    HIP_OK(hipGetLastError());
    return SPC3D_OK;
}

__global__ void descents_k(const uint32_t *__restrict__ d, uint64_t n, unsigned long long *acc)
{
    unsigned long long c = 0;
    GRID_STRIDE(i, n)
    if (i + 1 < n && d[i + 1] < d[i])
        ++c;
    c = wave_sum(c);
    if ((threadIdx.x & 63u) == 0 && c)
        atomicAdd(acc, c);
}

int is_nondecreasing_device(hipStream_t st, const uint32_t *d, uint64_t n, bool *out,
                            std::string &err)
{
    *out = true;
    if (n < 2)
        return SPC3D_OK;
    DBuf<unsigned long long> acc;
    HIP_OK(acc.alloc(1));
    HIP_OK(hipMemsetAsync(acc.p, 0, sizeof(unsigned long long), st));
    LAUNCH_SMALL(descents_k, n, d, n, acc.p);
    unsigned long long descents = 0;
    TRY(fetch(st, &descents, acc.p, sizeof descents, err));
    *out = descents == 0;
    return SPC3D_OK;
}

int sum_sq_seg_len_device(hipStream_t st, const Seg *d_segs, uint64_t nseg, uint64_t *out,
                          std::string &err)
{
    *out = 0;
    if (nseg == 0)
        return SPC3D_OK;
    DBuf<unsigned long long> acc;
    HIP_OK(acc.alloc(1));
    HIP_OK(hipMemsetAsync(acc.p, 0, sizeof(unsigned long long), st));
    LAUNCH_SMALL(sum_sq_len_k, nseg, d_segs, nseg, acc.p);
    unsigned long long h = 0;
    TRY(fetch(st, &h, acc.p, sizeof h, err));
    *out = h;
    return SPC3D_OK;
}

} // namespace spc3d
