// gfx950 (CDNA4, wave64) kernels for the local SDDMM and SpMM.
//
//   sddmm: C[e] = S.vv[e] * <A[ii[e],:], B[jj[e],:]>      (reference: src/core_ops.cpp:5-22)
//   spmm : Y[ii[e],:] += A.vv[e] * X[jj[e],:]             (reference: src/core_ops.cpp:24-35)
//
// Both are gather-bound (about 0.25 flop per byte): no MFMA.  The unit of work
// is a row segment (plan_host.h): at most seg_max consecutive entries of one
// row.  A dense row of K reals is nvec 16-byte vectors, covered by LPR lanes
// holding VPL vectors each (nvec = LPR * VPL with the row stride a compile-time
// constant, or nvec < LPR * VPL given at run time in the "ragged" variants, whose
// spare lanes idle, or a row that ends inside its last vector in the "odd"
// variants, or one shorter than a vector in the "thin" variant; rows over 4 KiB
// run as 4 KiB column slices, one launch each); one wavefront works on 64 / LPR
// segments at once and every global load instruction moves 64 x 16 B.  Segments
// arrive sorted longest first, so the lane groups of a wavefront run the same trip
// count.
//
// A segment is walked in batches of UB entries; what remains is one masked
// batch (the missing entries repeat the last one's loads and store nothing), or,
// in SpMM's short-segment launch, exact batches of UB/2, ..., 2, 1.  Every batch
// is straight-line code: within it all gathers are issued before any arithmetic
// (a scheduling barrier keeps the compiler from serialising them).
//
//   sddmm: the group keeps its A row slice in registers, gathers the B row
//          slices of a batch, and reduces the per-lane partial dot products
//          across the group with a halving exchange (NB-1 exchanges for NB
//          entries instead of NB*log2(LPR)); exchanges inside a 16-lane row
//          are DPP moves, those across rows the gfx950 row swaps
//          (v_permlane16_swap, v_permlane32_swap).  The lane that ends up
//          with entry u's dot product scales it by S.vv and stores it at the
//          caller's position: read per entry, or once per segment where a
//          segment's positions are consecutive; segments for which they are
//          not store in kernel order to a staging vector instead
//          (unstage_pairs_kernel brings those home), and for an arbitrary
//          entry order everything is stored in kernel order and brought home
//          by two tile-local passes through LDS (unpermute_pass1/2_kernel).
//   spmm : lane = slice of K, no cross-lane reduction; the group accumulates
//          a * X[c,:] in registers and does one read-modify-write of the Y
//          row slice.  Rows cut into several segments write partial sums that
//          spmm_fixup adds into Y in a fixed order (no atomics, results are
//          reproducible run to run).
//
// Streams that are read once (indices, sparse values, segment descriptors, A
// rows, Y rows) use non-temporal accesses so that the per-XCD L2 is left to
// the gathered B / X rows, the only operand with reuse.  The gathers themselves
// are plain loads: a non-temporal hint on the gathers of low-degree columns
// was measured to slow both kernels down by 15 to 40 %.
#include <hip/hip_runtime.h>

#include "kernels.h"

namespace spc3d {
namespace {

template <typename T> struct Vec;
template <> struct Vec<float> {
    typedef float type __attribute__((ext_vector_type(4)));
    typedef type loose __attribute__((aligned(4))); // same vector at element alignment
    static constexpr int N = 4;
};
template <> struct Vec<double> {
    typedef double type __attribute__((ext_vector_type(2)));
    typedef type loose __attribute__((aligned(8)));
    static constexpr int N = 2;
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kBlock = 256; // 4 wavefronts

template <typename P> __device__ __forceinline__ P nt_load(const P *p)
{
    return __builtin_nontemporal_load(p);
}
template <typename P> __device__ __forceinline__ void nt_store(P v, P *p)
{
    __builtin_nontemporal_store(v, p);
}

__device__ __forceinline__ constexpr int ilog2(int x) { return x <= 1 ? 0 : 1 + ilog2(x >> 1); }

// ---- lane exchange ----------------------------------------------------------
// xchg<S>(v): the value lane (id ^ S) holds.  S < 16 (the only strides the kernels
// use it for; 16 and 32 go through swap_add below) stays inside a 16-lane DPP row: xor 1 and 2 are quad permutes, xor 8 is a rotation by 8, xor 4 is
// half-row mirror (i -> 7 - i = i ^ 7) after quad reverse (i ^ 3).
template <int CTRL> __device__ __forceinline__ int dpp_mov(int v)
{
    // every lane is written (all rows and banks enabled, the patterns used here have
    // no invalid source lane): no previous value to set up
    return __builtin_amdgcn_mov_dpp(v, CTRL, 0xF, 0xF, false);
}
template <int S> __device__ __forceinline__ int xchg_i32(int v)
{
    if constexpr (S == 1)
        return dpp_mov<0xB1>(v); // quad_perm [1,0,3,2]
    else if constexpr (S == 2)
        return dpp_mov<0x4E>(v); // quad_perm [2,3,0,1]
    else if constexpr (S == 4)
        return dpp_mov<0x141>(dpp_mov<0x1B>(v)); // row_half_mirror o quad_perm [3,2,1,0]
    else if constexpr (S == 8)
        return dpp_mov<0x128>(v); // row_ror:8
    else
        return __shfl_xor(v, S, 64);
}
template <int S> __device__ __forceinline__ float xchg(float v)
{
    return __int_as_float(xchg_i32<S>(__float_as_int(v)));
}
template <int S> __device__ __forceinline__ double xchg(double v)
{
    const int lo = xchg_i32<S>(__double2loint(v));
    const int hi = xchg_i32<S>(__double2hiint(v));
    return __hiloint2double(hi, lo);
}

// Halving step across stride 16 or 32: a and b are two partial sums of which the
// lanes with bit S clear go on with a and those with bit S set with b.  One
// v_permlane16_swap / v_permlane32_swap (gfx950) exchanges the odd 16-lane rows of a
// with the even rows of b (the upper 32 lanes of a with the lower 32 of b): the two
// results, added, are a summed over the stride in the lanes with bit S clear and b
// in the others -- no selects and no second move, 2 instructions per 32-bit word
// where the DPP form takes 4.  With b == a it is the all-reduce across the stride.
template <int S> __device__ __forceinline__ void swap_rows(unsigned &a, unsigned &b)
{
    static_assert(S == 16 || S == 32, "row swaps exist for strides 16 and 32");
    if constexpr (S == 16) {
        const auto r = __builtin_amdgcn_permlane16_swap(a, b, false, false);
        a = r[0], b = r[1];
    } else {
        const auto r = __builtin_amdgcn_permlane32_swap(a, b, false, false);
        a = r[0], b = r[1];
    }
}
template <int S> __device__ __forceinline__ float swap_add(float a, float b)
{
    unsigned x = __float_as_uint(a), y = __float_as_uint(b);
    swap_rows<S>(x, y);
    return __uint_as_float(x) + __uint_as_float(y);
}
template <int S> __device__ __forceinline__ double swap_add(double a, double b)
{
    unsigned xl = (unsigned)__double2loint(a), yl = (unsigned)__double2loint(b);
    unsigned xh = (unsigned)__double2hiint(a), yh = (unsigned)__double2hiint(b);
    swap_rows<S>(xl, yl);
    swap_rows<S>(xh, yh);
    return __hiloint2double((int)xh, (int)xl) + __hiloint2double((int)yh, (int)yl);
}

// Order in which the xor strides of an LPR-lane group are used: the steps that
// move the most values come first and get the cheapest exchanges: the row swaps
// of strides 32 and 16, then the single-instruction DPP moves.
template <int LPR> struct Strides;
template <> struct Strides<4> { static constexpr int s[2] = {2, 1}; };
template <> struct Strides<8> { static constexpr int s[3] = {2, 1, 4}; };
template <> struct Strides<16> { static constexpr int s[4] = {8, 2, 1, 4}; };
template <> struct Strides<32> { static constexpr int s[5] = {16, 8, 2, 1, 4}; };
template <> struct Strides<64> { static constexpr int s[6] = {32, 16, 8, 2, 1, 4}; };

// Halving exchange + finishing all-reduce over an LPR-lane group.
// In: part[u] = this lane's partial sum for entry u, u < NB.  Out: part[0] =
// the full sum of entry entry_of<LPR, NB>(sub), identical in every lane that
// maps to that entry.
template <typename T, int LPR, int NB, int STEP = 0, int N = NB>
__device__ __forceinline__ void group_reduce(T (&part)[NB], uint32_t sub)
{
    if constexpr (STEP < ilog2(LPR)) {
        constexpr int S = Strides<LPR>::s[STEP];
        if constexpr (N > 1) {
            const bool upper = (sub & S) != 0;
#pragma unroll
            for (int i = 0; i < N / 2; ++i) {
                if constexpr (S >= 16) {
                    part[i] = swap_add<S>(part[i], part[i + N / 2]);
                } else {
                    const T keep = upper ? part[i + N / 2] : part[i];
                    const T send = upper ? part[i] : part[i + N / 2];
                    part[i] = keep + xchg<S>(send);
                }
            }
            group_reduce<T, LPR, NB, STEP + 1, N / 2>(part, sub);
        } else {
            if constexpr (S >= 16)
                part[0] = swap_add<S>(part[0], part[0]);
            else
                part[0] += xchg<S>(part[0]);
            group_reduce<T, LPR, NB, STEP + 1, 1>(part, sub);
        }
    }
}

// Entry (0 .. NB-1) whose sum lane `sub` holds after group_reduce<LPR, NB>.
template <int LPR, int NB> __device__ __forceinline__ uint32_t entry_of(uint32_t sub)
{
    uint32_t u = 0;
#pragma unroll
    for (int t = 0; t < ilog2(NB); ++t)
        u |= ((sub & Strides<LPR>::s[t]) ? 1u : 0u) << (ilog2(NB) - 1 - t);
    return u;
}

// One lane per entry stores: the lane whose bits for the finishing strides are 0.
template <int LPR, int NB> __device__ __forceinline__ bool is_writer(uint32_t sub)
{
    uint32_t mask = 0;
#pragma unroll
    for (int t = ilog2(NB); t < ilog2(LPR); ++t)
        mask |= Strides<LPR>::s[t];
    return (sub & mask) == 0;
}

// Lane (within the group) that stores entry u after group_reduce<LPR, NB>.
template <int LPR, int NB> __device__ __forceinline__ constexpr int writer_lane(int u)
{
    int lane = 0;
    for (int t = 0; t < ilog2(NB); ++t)
        if ((u >> (ilog2(NB) - 1 - t)) & 1)
            lane |= Strides<LPR>::s[t];
    return lane;
}

// Segment this lane group works on.  Segments are stored in chunks of kChunk;
// with nq == 8, chunk v belongs to queue v % 8.  The hardware deals the
// workgroups of a dispatch to the 8 XCDs round-robin by workgroup id, starting
// from an XCD that is fixed per hardware queue, so the workgroups b with equal
// (b + rot) % 8 all run on one XCD; they take the chunks of queue (b + rot) % 8
// and the dense rows of one column slice are then only ever gathered through
// one L2.  `rot` lines the queues of the auxiliary stream up with those of the
// main stream.  Any rot gives each segment to exactly one workgroup: if the
// hardware dealt workgroups differently the result would be the same, only
// slower.
template <int G> __device__ __forceinline__ uint64_t seg_index(uint32_t nq, uint32_t rot)
{
    constexpr uint32_t kSegPerBlock = (kBlock / 64) * G;
    constexpr uint32_t kBlocksPerChunk = kChunk / kSegPerBlock;
    static_assert(kChunk % kSegPerBlock == 0, "a chunk is a whole number of workgroups");
    const uint32_t b = blockIdx.x;
    uint64_t chunk;
    uint32_t inner;
    if (nq == 8) {
        const uint32_t j = b >> 3;
        chunk = (uint64_t)(j / kBlocksPerChunk) * 8 + ((b + rot) & 7u);
        inner = j % kBlocksPerChunk;
    } else {
        chunk = b / kBlocksPerChunk;
        inner = b % kBlocksPerChunk;
    }
    return chunk * kChunk + inner * kSegPerBlock + (threadIdx.x >> 6) * G +
           (threadIdx.x & 63u) / (64 / G);
}

// The short-segment launch walks a dependency chain per segment: descriptor, then
// column indices, then the gathers.  The plan keeps the first kFirstCols column indices
// of every short segment in a table addressed by the segment's position (past the
// segment's end they repeat its last column), so that they are fetched beside the
// descriptor instead of after it: two memory latencies per segment instead of three.
// Lane u of a group of LPR >= kFirstCols lanes gets the column of entry u % kFirstCols;
// a group of 4 lanes gets those of entries u and 4 + u.
// stream_c: SDDMM stores its results at permuted positions past the L2 (streaming)
// instead of with plain stores that the L2 can merge: for the blocks of a plan kept in
// column blocks, whose positions are long runs in a staging vector and whose block of
// dense rows is meant to stay in the L2s.
// stage / stage_from: SDDMM results whose position (perm) is stage_from or more go to
// place (position - stage_from) of the staging vector instead of into C (segments whose
// caller's positions are not consecutive; unstage_pairs_kernel brings them home).
// shift: added to the kernel position of an entry when no `perm` is read (a plan whose
// segments all have consecutive positions: perm[start] - start of the segment).
struct Ahead {
    uint32_t first[2] = {0, 0};
    bool stream_c = false;
    uint32_t stage_from = 0xFFFFFFFFu;
    void *stage = nullptr;
    uint32_t shift = 0;
};
constexpr uint32_t kStoreStream = 1u;  // sddmm_seg_kernel flags: Ahead::stream_c
constexpr uint32_t kStoreSegBase = 2u; // positions are perm[segment start] + offset
template <int LPR, bool WIDE>
__device__ __forceinline__ Ahead load_first_cols(const uint32_t *__restrict__ first_cols,
                                                 uint64_t sid, uint32_t sub)
{
    Ahead f;
    if constexpr (!WIDE) {
        constexpr uint32_t GL = (uint32_t)LPR < kFirstCols ? (uint32_t)LPR : kFirstCols;
        const uint32_t *at = first_cols + sid * kFirstCols + (sub & (GL - 1));
        f.first[0] = nt_load(at);
        if constexpr ((uint32_t)LPR < kFirstCols)
            f.first[1] = nt_load(at + LPR);
    }
    return f;
}

// Fills the table above for `n` short segments.
__global__ void __launch_bounds__(kBlock)
first_cols_kernel(const Seg *__restrict__ segs, uint32_t n, const uint32_t *__restrict__ col,
                  uint32_t *__restrict__ first_cols)
{
    const uint64_t t = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    const uint64_t s = t / kFirstCols;
    const uint32_t u = (uint32_t)(t % kFirstCols);
    if (s >= n)
        return;
    const Seg sg = segs[s];
    uint32_t c = 0;
    if (sg.len)
        c = col[sg.start + (u < sg.len ? u : sg.len - 1)];
    first_cols[t] = c;
}

// RG == 1 ("ragged"): a dense row is nvec 16-byte vectors with nvec < LPR * VPL,
// given at run time; lanes whose vector index is >= nvec idle.  RG == 0: nvec ==
// LPR * VPL exactly and the row stride is a compile-time constant.  RG == 2, 3: below.
template <typename T, int LPR, int VPL, int RG>
__device__ __forceinline__ const typename Vec<T>::type *row_ptr(const T *base, uint32_t row,
                                                                uint32_t sub, uint32_t nvec)
{
    const uint64_t row_bytes = RG ? (uint64_t)nvec * 16 : (uint64_t)LPR * VPL * 16;
    return reinterpret_cast<const typename Vec<T>::type *>(
               reinterpret_cast<const char *>(base) + (uint64_t)row * row_bytes) +
           sub;
}

template <int LPR, int RG>
__device__ __forceinline__ bool lane_on(uint32_t sub, int v, uint32_t nvec)
{
    return !RG || sub + (uint32_t)v * LPR < nvec;
}

// 16-byte accesses at element alignment.  (Not through nt_load / nt_store: template
// argument deduction would drop the typedef's alignment.)
template <typename T> __device__ __forceinline__ typename Vec<T>::type loose_load(const char *p)
{
    return *reinterpret_cast<const typename Vec<T>::loose *>(p);
}
template <typename T> __device__ __forceinline__ typename Vec<T>::type loose_load_nt(const char *p)
{
    return __builtin_nontemporal_load(reinterpret_cast<const typename Vec<T>::loose *>(p));
}
template <typename T>
__device__ __forceinline__ void loose_store(typename Vec<T>::type v, char *p)
{
    *reinterpret_cast<typename Vec<T>::loose *>(p) = v;
}
template <typename T>
__device__ __forceinline__ void loose_store_nt(typename Vec<T>::type v, char *p)
{
    __builtin_nontemporal_store(v, reinterpret_cast<typename Vec<T>::loose *>(p));
}

// RG == 2 ("odd"): a dense row of K reals is no whole number of 16-byte vectors
// (the kernels' `nvec` argument carries K).  Rows start at element alignment only,
// and the last vector of a row would reach past its end, so: the lane that holds the
// row's end loads the 16 bytes that END there (the leading elements of that vector
// belong to the lane before and are not counted), and lanes past the end load the
// same vector and count nothing.  Every load stays inside the row, without a
// branch.  Vector loads and stores at 4- or 8-byte alignment are what global memory
// accesses on this GPU allow.
//
// RG == 3 ("thin"): a dense row is shorter than 16 bytes (K < Vec<T>::N reals; `nvec`
// carries K again).  The row is the first K elements of one vector, loaded element by
// element (the elements past K repeat element K - 1: no branch, no access outside
// the row) and counted by the first lane of the group only; the group's other lanes
// load the same addresses and count nothing.  Runs the 4-lane shape.
template <typename T, int VPL> struct OddLanes {
    uint32_t off[VPL];             // byte offset within a row of this lane's vector v
    bool keep[VPL][Vec<T>::N];     // the elements of it that are this lane's
    bool all[VPL];                 // every element is
    uint32_t stride;               // reals from one dense row to the next (>= K: the kernel may
                                   // be working on a slice of K columns of wider rows)
    bool accum;                    // SDDMM adds to C instead of overwriting it (every slice of
                                   // wide rows but the first)
};
template <typename T, int VPL, int RG> struct Odd {};
template <typename T, int VPL> struct Odd<T, VPL, 2> : OddLanes<T, VPL> {};
template <typename T, int VPL> struct Odd<T, VPL, 3> : OddLanes<T, VPL> {};

template <typename T, int LPR, int VPL, int RG>
__device__ __forceinline__ Odd<T, VPL, RG> odd_lanes(uint32_t sub, uint32_t K, uint32_t stride,
                                                     uint32_t accum)
{
    Odd<T, VPL, RG> o;
    if constexpr (RG >= 2) {
        o.stride = stride;
        o.accum = accum != 0;
    }
    if constexpr (RG == 2) {
        const uint32_t bytes = K * (uint32_t)sizeof(T); // >= 16: see pick_shape
#pragma unroll
        for (int v = 0; v < VPL; ++v) {
            const uint32_t first = (sub + (uint32_t)v * LPR) * 16;
            const uint32_t start = first < bytes - 16 ? first : bytes - 16;
            o.off[v] = start;
            o.all[v] = start == first;
#pragma unroll
            for (int i = 0; i < Vec<T>::N; ++i)
                o.keep[v][i] = start + (uint32_t)i * sizeof(T) >= first;
        }
    } else if constexpr (RG == 3) {
#pragma unroll
        for (int v = 0; v < VPL; ++v) {
            o.off[v] = 0;
            o.all[v] = false;
#pragma unroll
            for (int i = 0; i < Vec<T>::N; ++i)
                o.keep[v][i] = v == 0 && sub == 0 && (uint32_t)i < K;
        }
    }
    return o;
}

template <typename T, int RG>
__device__ __forceinline__ const char *odd_row(const T *base, uint32_t row, uint32_t stride)
{
    static_assert(RG >= 2, "rows at element alignment, `stride` reals apart");
    return reinterpret_cast<const char *>(base) + (uint64_t)row * ((uint64_t)stride * sizeof(T));
}

// Vector v of the row at r as this lane loads it in the RG >= 2 variants (NT: a
// row that is read once).
template <typename T, int RG, int VPL, bool NT = false>
__device__ __forceinline__ typename Vec<T>::type odd_load(const char *r, int v, uint32_t K,
                                                          const Odd<T, VPL, RG> &odd)
{
    if constexpr (RG == 3) {
        typename Vec<T>::type out{};
        const T *e = reinterpret_cast<const T *>(r);
#pragma unroll
        for (int i = 0; i + 1 < Vec<T>::N; ++i) // K <= N - 1
            out[i] = e[(uint32_t)i < K ? (uint32_t)i : K - 1];
        return out;
    } else if constexpr (NT) {
        return loose_load_nt<T>(r + odd.off[v]);
    } else {
        return loose_load<T>(r + odd.off[v]);
    }
}

// out[v] = this lane's vectors of dense row `row`.  RG >= 2 loads every element of
// them; what is not the lane's to count is left out by the caller (SDDMM: in the
// dot product; SpMM: at the store).
template <typename T, int LPR, int VPL, int RG>
__device__ __forceinline__ void gather_row(typename Vec<T>::type (&out)[VPL], const T *base,
                                           uint32_t row, uint32_t sub, uint32_t nvec,
                                           const Odd<T, VPL, RG> &odd)
{
    using V = typename Vec<T>::type;
    if constexpr (RG >= 2) {
        const char *r = odd_row<T, RG>(base, row, odd.stride);
#pragma unroll
        for (int v = 0; v < VPL; ++v)
            out[v] = odd_load<T, RG, VPL>(r, v, nvec, odd);
    } else {
        const V *r = row_ptr<T, LPR, VPL, RG>(base, row, sub, nvec);
#pragma unroll
        for (int v = 0; v < VPL; ++v)
            out[v] = lane_on<LPR, RG>(sub, v, nvec) ? r[v * LPR] : V{};
    }
}

// a . b over the elements that are this lane's.
template <typename T, int VPL, int RG>
__device__ __forceinline__ T lane_dot(const typename Vec<T>::type (&a)[VPL],
                                      const typename Vec<T>::type (&b)[VPL],
                                      const Odd<T, VPL, RG> &odd)
{
    T dot = (T)0;
#pragma unroll
    for (int v = 0; v < VPL; ++v)
#pragma unroll
        for (int i = 0; i < Vec<T>::N; ++i) {
            if constexpr (RG >= 2)
                dot += a[v][i] * (odd.keep[v][i] ? b[v][i] : (T)0);
            else
                dot += a[v][i] * b[v][i];
        }
    return dot;
}

// Writes y0 + acc (whole rows of Y) or acc (partial-sum slots, read back by
// spmm_fixup right after) to this lane's part of the row at drow: one vector store
// where the whole vector is the lane's, element stores for the lane at the row's end.
template <typename T, int VPL>
__device__ __forceinline__ void odd_store(char *drow, bool whole,
                                          const typename Vec<T>::type (&y0)[VPL],
                                          const typename Vec<T>::type (&acc)[VPL],
                                          const OddLanes<T, VPL> &odd)
{
    using V = typename Vec<T>::type;
#pragma unroll
    for (int v = 0; v < VPL; ++v) {
        const V r = y0[v] + acc[v]; // y0 is zero for a slot
        if (odd.all[v]) {
            if (whole)
                loose_store_nt<T>(r, drow + odd.off[v]);
            else
                loose_store<T>(r, drow + odd.off[v]);
        } else {
            T *d = reinterpret_cast<T *>(drow + odd.off[v]);
#pragma unroll
            for (int i = 0; i < Vec<T>::N; ++i)
                if (odd.keep[v][i])
                    d[i] = r[i];
        }
    }
}

// ---------------------------------------------------------------- SDDMM ----
// One batch of NB entries from p0.  MK ("masked"): only the first n (1 <= n <= NB)
// exist; the others repeat entry n - 1 (loads without branches, from addresses
// that are being read anyway) and store nothing, so that a tail of any length
// costs one round of gathers.
//
// FZ ("fused"): the gathered B rows also feed the SpMM of the same pattern,
// acc += w_u * B[c_u,:] in kernel order, with w_u = S.vv (FZ == 1) or the SDDMM
// result just computed (FZ == 2); the weight of entry u is broadcast from the lane
// that stores it.
//
// PRE: the column indices of the batch were loaded ahead (lane u of the group holds that
// of entry u in ex.first[0], or, where the group has fewer lanes than the batch has entries,
// those of entries u and LPR + u in ex.first[0] and ex.first[1]); past the segment's end they
// repeat its last column.
//
// NG <= NB: every lane group of the wavefront has at most NG entries in this batch, so
// only the first NG gathers are issued.
template <typename T, int LPR, int VPL, int NB, int RG, bool MK, int FZ, bool PRE, int NG>
__device__ __forceinline__ void
sddmm_batch_one(const typename Vec<T>::type (&a)[VPL], typename Vec<T>::type (&acc)[VPL],
            const uint32_t *__restrict__ col, const uint32_t *__restrict__ perm,
            const T *__restrict__ sval, const T *__restrict__ B, T *__restrict__ C, uint32_t p0,
            uint32_t n, uint32_t sub, uint32_t nvec,
            const Odd<T, VPL, RG> &odd, const Ahead &ex)
{
    using V = typename Vec<T>::type;
    static_assert(NB <= LPR, "batch must fit the lane group");

    // Lane u of the group fetches the column of entry u; the writer lanes fetch
    // what they need for the store.  These head the dependency chain.
    uint32_t e = sub & (NB - 1);
    if (MK)
        e = e < n ? e : n - 1;
    const uint32_t cme = PRE ? ex.first[0] : nt_load(col + p0 + e);
    const uint32_t uo = entry_of<LPR, NB>(sub);
    const bool writer = is_writer<LPR, NB>(sub) && (!MK || uo < n);
    T sv = (T)0;
    uint32_t dst = p0 + uo + ex.shift;
    if (writer) {
        sv = nt_load(sval + p0 + uo);
        if (perm)
            dst = nt_load(perm + p0 + uo);
    }

    static_assert(NG >= 1 && NG <= NB && (MK || NG == NB), "NG < NB only in a masked batch");
    V b[NG][VPL];
#pragma unroll
    for (int u = 0; u < NG; ++u) {
        const uint32_t c = __shfl(cme, u, LPR);
        gather_row<T, LPR, VPL, RG>(b[u], B, c, sub, nvec, odd);
    }
    __builtin_amdgcn_sched_barrier(0); // all gathers in flight before the first use

    T part[NB];
#pragma unroll
    for (int u = 0; u < NB; ++u) {
        if (u < NG)
            part[u] = lane_dot<T, VPL, RG>(a, b[u], odd);
        else
            part[u] = (T)0;
    }
    group_reduce<T, LPR, NB>(part, sub);
    T result = part[0] * sv;
    // Results in the caller's order: when that is the kernel order the stores of a
    // batch fill whole lines and stream out; when it is not they are scattered, and
    // plain stores let the L2 merge neighbours into lines before writing back.
    if (writer) {
        const bool staged = dst >= ex.stage_from;
        T *out = staged ? static_cast<T *>(ex.stage) + (dst - ex.stage_from) : C + dst;
        if constexpr (RG >= 2) {
            if (odd.accum)
                result += *out;
        }
        if (perm && !ex.stream_c && !staged)
            *out = result;
        else
            nt_store(result, out);
    }
    if constexpr (FZ != 0) {
        const T mine = FZ == 2 ? result : sv; // valid on the writer lanes
#pragma unroll
        for (int u = 0; u < NG; ++u) {
            const bool on = !MK || (uint32_t)u < n;
            const T w = on ? __shfl(mine, writer_lane<LPR, NB>(u), LPR) : (T)0;
#pragma unroll
            for (int v = 0; v < VPL; ++v)
                acc[v] += (on ? b[u][v] : V{}) * w;
        }
    }
}

template <typename T, int LPR, int VPL, int NB, int RG, bool MK, int FZ, bool PRE>
__device__ __forceinline__ void
sddmm_batch_rounds(const typename Vec<T>::type (&a)[VPL], typename Vec<T>::type (&acc)[VPL],
            const uint32_t *__restrict__ col, const uint32_t *__restrict__ perm,
            const T *__restrict__ sval, const T *__restrict__ B, T *__restrict__ C, uint32_t p0,
            uint32_t n, uint32_t sub, uint32_t nvec,
            const Odd<T, VPL, RG> &odd, const Ahead &ex)
{
    using V = typename Vec<T>::type;
    // A group of LPR lanes reduces at most LPR entries at a time: the NB entries of
    // the batch are R rounds of G, all gathered before the first round is reduced, so
    // that narrow rows (LPR = 4, 8) keep as many gathers in flight as wide ones.
    constexpr int G = NB < LPR ? NB : LPR;
    constexpr int R = NB / G;
    static_assert(R * G == NB, "a batch is a whole number of rounds");
    static_assert(!PRE || R <= 2, "at most two rounds of columns are loaded ahead");

    // Lane u of the group fetches the column of entry u of each round; the writer
    // lanes fetch what they need for the store.  These head the dependency chain.
    const uint32_t uo = entry_of<LPR, G>(sub);
    const bool wlane = is_writer<LPR, G>(sub);
    uint32_t cme[R], dst[R];
    T sv[R];
    bool writer[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        uint32_t e = (uint32_t)r * G + (sub & (G - 1));
        if (MK)
            e = e < n ? e : n - 1;
        cme[r] = PRE ? ex.first[r & 1] : nt_load(col + p0 + e);
        const uint32_t mine = (uint32_t)r * G + uo;
        writer[r] = wlane && (!MK || mine < n);
        sv[r] = (T)0;
        dst[r] = p0 + mine + ex.shift;
        if (writer[r]) {
            sv[r] = nt_load(sval + p0 + mine);
            if (perm)
                dst[r] = nt_load(perm + p0 + mine);
        }
    }

    V b[NB][VPL];
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        const uint32_t c = __shfl(cme[j / G], j % G, LPR);
        gather_row<T, LPR, VPL, RG>(b[j], B, c, sub, nvec, odd);
    }
    __builtin_amdgcn_sched_barrier(0); // all gathers in flight before the first use

#pragma unroll
    for (int r = 0; r < R; ++r) {
        T part[G];
#pragma unroll
        for (int u = 0; u < G; ++u) {
            part[u] = lane_dot<T, VPL, RG>(a, b[r * G + u], odd);
        }
        group_reduce<T, LPR, G>(part, sub);
        T result = part[0] * sv[r];
        // Results in the caller's order: when that is the kernel order the stores of a
        // batch fill whole lines and stream out; when it is not they are scattered, and
        // plain stores let the L2 merge neighbours into lines before writing back.
        if (writer[r]) {
            const bool staged = dst[r] >= ex.stage_from;
            T *out = staged ? static_cast<T *>(ex.stage) + (dst[r] - ex.stage_from) : C + dst[r];
            if constexpr (RG >= 2) {
                if (odd.accum)
                    result += *out;
            }
            if (perm && !ex.stream_c && !staged)
                *out = result;
            else
                nt_store(result, out);
        }
        if constexpr (FZ != 0) {
            const T mine = FZ == 2 ? result : sv[r]; // valid on the writer lanes
#pragma unroll
            for (int u = 0; u < G; ++u) {
                const bool on = !MK || (uint32_t)(r * G + u) < n;
                const T w = on ? __shfl(mine, writer_lane<LPR, G>(u), LPR) : (T)0;
#pragma unroll
                for (int v = 0; v < VPL; ++v)
                    acc[v] += (on ? b[r * G + u][v] : V{}) * w;
            }
        }
    }
}

// A batch of NB entries: one round when the lane group can reduce them at once,
// several otherwise.  The two forms are kept apart on purpose: written as the
// R = 1 case of the rounds form, the single round compiles to 24 more VGPRs
// (100 -> 124 in the wide launch, 62 -> 74 and two wavefronts per SIMD fewer in
// the short one), which cost the 5-entry rows of a stencil 20 %.
template <typename T, int LPR, int VPL, int NB, int RG, bool MK, int FZ, bool PRE = false,
          int NG = NB>
__device__ __forceinline__ void
sddmm_batch(const typename Vec<T>::type (&a)[VPL], typename Vec<T>::type (&acc)[VPL],
            const uint32_t *__restrict__ col, const uint32_t *__restrict__ perm,
            const T *__restrict__ sval, const T *__restrict__ B, T *__restrict__ C, uint32_t p0,
            uint32_t n, uint32_t sub, uint32_t nvec,
            const Odd<T, VPL, RG> &odd, const Ahead &ex)
{
    if constexpr (NB <= LPR)
        sddmm_batch_one<T, LPR, VPL, NB, RG, MK, FZ, PRE, NG>(a, acc, col, perm, sval, B, C, p0, n,
                                                              sub, nvec, odd, ex);
    else
        sddmm_batch_rounds<T, LPR, VPL, NB, RG, MK, FZ, PRE>(a, acc, col, perm, sval, B, C, p0, n,
                                                             sub, nvec, odd, ex);
}

// n consecutive entries from p.  WIDE: full batches of UB, then one masked batch
// of the smallest size in {4, 8, 16} that holds the rest.  !WIDE (segments known
// to be short, run at twice the occupancy): masked batches of UB throughout, the
// first of them on the column indices in `ex.first` (loaded ahead, beside the segment's
// descriptor, from the plan's table of first columns: kFirstCols per short segment).
template <typename T, int LPR, int VPL, int UB, int RG, bool WIDE, int FZ>
__device__ __forceinline__ void
sddmm_walk(const typename Vec<T>::type (&a)[VPL], typename Vec<T>::type (&acc)[VPL],
           const uint32_t *__restrict__ col, const uint32_t *__restrict__ perm,
           const T *__restrict__ sval, const T *__restrict__ B, T *__restrict__ C, uint32_t p,
           uint32_t n, uint32_t sub, uint32_t nvec,
            const Odd<T, VPL, RG> &odd, const Ahead &ex)
{
    if constexpr (WIDE) {
        for (; n >= UB; n -= UB, p += UB)
            sddmm_batch<T, LPR, VPL, UB, RG, false, FZ>(a, acc, col, perm, sval, B, C, p, UB, sub, nvec, odd, ex);
        if (n == 0)
            return;
        if constexpr (UB > 8) {
            if (n > 8) {
                sddmm_batch<T, LPR, VPL, UB, RG, true, FZ>(a, acc, col, perm, sval, B, C, p, n, sub, nvec, odd, ex);
                return;
            }
        }
        if constexpr (UB > 4) {
            if (n > 4) {
                sddmm_batch<T, LPR, VPL, 8, RG, true, FZ>(a, acc, col, perm, sval, B, C, p, n, sub, nvec, odd, ex);
                return;
            }
        }
        sddmm_batch<T, LPR, VPL, (UB < 4 ? UB : 4), RG, true, FZ>(a, acc, col, perm, sval, B, C, p, n, sub, nvec, odd, ex);
    } else {
        static_assert(WIDE || UB <= (int)kFirstCols, "the first batch runs on the columns loaded ahead");
        {
            // Segments arrive sorted by length, so the groups of a wavefront mostly hold
            // the same number of entries: the batch is cut to what the longest of them
            // needs (a condition uniform over the wavefront), which spares the memory
            // pipeline the repeated gathers of a full masked batch.
            const uint32_t m = n < (uint32_t)UB ? n : (uint32_t)UB;
            if constexpr (UB == 8 && LPR >= 8) {
                if (__ballot(m > 2) == 0)
                    sddmm_batch<T, LPR, VPL, 2, RG, true, FZ, true>(a, acc, col, perm, sval, B, C, p, m, sub, nvec, odd, ex);
                else if (__ballot(m > 4) == 0)
                    sddmm_batch<T, LPR, VPL, 4, RG, true, FZ, true>(a, acc, col, perm, sval, B, C, p, m, sub, nvec, odd, ex);
                else if (__ballot(m > 5) == 0)
                    sddmm_batch<T, LPR, VPL, 8, RG, true, FZ, true, 5>(a, acc, col, perm, sval, B, C, p, m, sub, nvec, odd, ex);
                else
                    sddmm_batch<T, LPR, VPL, 8, RG, true, FZ, true>(a, acc, col, perm, sval, B, C, p, m, sub, nvec, odd, ex);
            } else {
                sddmm_batch<T, LPR, VPL, UB, RG, true, FZ, true>(a, acc, col, perm, sval, B, C, p, m, sub, nvec, odd, ex);
            }
            n -= m;
            p += m;
        }
#pragma nounroll
        while (n > 0) {
            const uint32_t m = n < (uint32_t)UB ? n : (uint32_t)UB;
            sddmm_batch<T, LPR, VPL, UB, RG, true, FZ>(a, acc, col, perm, sval, B, C, p, m, sub, nvec, odd, ex);
            n -= m;
            p += m;
        }
    }
}

// FZ != 0: also Y[row,:] += sum of the segment's w_u * B[c_u,:] (partial-sum slot for
// a cut row, as in spmm_seg_kernel); Y and partial are unused otherwise.
template <typename T, int LPR, int VPL, int UB, int RG, bool WIDE, int FZ>
__global__ void __launch_bounds__(kBlock)
sddmm_seg_kernel(const Seg *__restrict__ segs, uint32_t nseg, uint32_t nq, uint32_t rot,
                 const uint32_t *__restrict__ col, const uint32_t *__restrict__ perm,
                 const T *__restrict__ sval, const T *__restrict__ A, const T *__restrict__ B,
                 T *__restrict__ C, T *__restrict__ Y, T *__restrict__ partial, uint32_t nvec,
                 uint32_t stride, uint32_t accum, const uint32_t *__restrict__ first_cols,
                 uint32_t flags, T *__restrict__ stage, uint32_t stage_from)
{
    static_assert(UB <= 16 && LPR <= 64, "at most 16 entries in flight per lane");
    using V = typename Vec<T>::type;
    const uint32_t sub = threadIdx.x & (LPR - 1);
    const uint64_t sid = seg_index<64 / LPR>(nq, rot);
    if (sid >= nseg)
        return;
    Ahead ex = load_first_cols<LPR, WIDE>(first_cols, sid, sub);
    ex.stream_c = (flags & kStoreStream) != 0;
    ex.stage = stage;
    ex.stage_from = stage_from;
    const u32x4 sg = nt_load(reinterpret_cast<const u32x4 *>(segs) + sid); // row, start, len, slot
    if (sg[2] == 0)
        return;
    if (flags & kStoreSegBase) { // one position per segment instead of one per entry
        ex.shift = nt_load(perm + sg[1]) - sg[1];
        perm = nullptr;
    }

    const Odd<T, VPL, RG> odd = odd_lanes<T, LPR, VPL, RG>(sub, nvec, stride, accum);
    V a[VPL], acc[VPL];
    if constexpr (RG >= 2) {
        const char *arow = odd_row<T, RG>(A, sg[0], stride);
#pragma unroll
        for (int v = 0; v < VPL; ++v) {
            a[v] = odd_load<T, RG, VPL, true>(arow, v, nvec, odd);
#pragma unroll
            for (int i = 0; i < Vec<T>::N; ++i)
                a[v][i] = odd.keep[v][i] ? a[v][i] : (T)0;
            acc[v] = V{};
        }
    } else {
        const V *arow = row_ptr<T, LPR, VPL, RG>(A, sg[0], sub, nvec);
#pragma unroll
        for (int v = 0; v < VPL; ++v) {
            a[v] = lane_on<LPR, RG>(sub, v, nvec) ? nt_load(arow + v * LPR) : V{};
            acc[v] = V{};
        }
    }
    sddmm_walk<T, LPR, VPL, UB, RG, WIDE, FZ>(a, acc, col, perm, sval, B, C, sg[1], sg[2], sub,
                                              nvec, odd, ex);
    if constexpr (FZ != 0 && RG >= 2) {
        const bool whole = sg[3] == kWholeRow;
        char *drow = const_cast<char *>(whole ? odd_row<T, RG>(Y, sg[0], stride)
                                              : odd_row<T, RG>(partial, sg[3], stride));
        V y0[VPL];
#pragma unroll
        for (int v = 0; v < VPL; ++v)
            y0[v] = whole ? odd_load<T, RG, VPL, true>(drow, v, nvec, odd) : V{};
        odd_store<T, VPL>(drow, whole, y0, acc, odd);
    } else if constexpr (FZ != 0) {
        const bool whole = sg[3] == kWholeRow;
        V *dst = const_cast<V *>(whole ? row_ptr<T, LPR, VPL, RG>(Y, sg[0], sub, nvec)
                                       : row_ptr<T, LPR, VPL, RG>(partial, sg[3], sub, nvec));
#pragma unroll
        for (int v = 0; v < VPL; ++v) {
            if (!lane_on<LPR, RG>(sub, v, nvec))
                continue;
            if (whole)
                nt_store(nt_load(dst + v * LPR) + acc[v], dst + v * LPR);
            else
                dst[v * LPR] = acc[v]; // read back by spmm_fixup right after
        }
    }
}

// ----------------------------------------------------------------- SpMM ----
// MK: only the first n of the NB entries exist; the others repeat the loads of
// entry n - 1 and add zero times zero.
// Column of entry j < kFirstCols of a short segment out of the indices loaded ahead:
// lane u of the group holds that of entry u in FC[0] (groups of 4 lanes: of entries u
// and 4 + u in FC[0] and FC[1]).
template <int LPR> __device__ __forceinline__ uint32_t first_col(const uint32_t (&FC)[2], uint32_t j)
{
    if constexpr (LPR >= (int)kFirstCols)
        return __shfl(FC[0], j, LPR);
    else
        return __shfl((j & LPR) ? FC[1] : FC[0], j & (LPR - 1), LPR);
}

// PRE: the batch is entries off .. off + NB - 1 of a short segment, off + NB <=
// kFirstCols, and takes its column indices from `ex.first` (first_col).
template <typename T, int LPR, int VPL, int NB, int RG, bool MK, bool PRE>
__device__ __forceinline__ void
spmm_batch_one(typename Vec<T>::type (&acc)[VPL], const uint32_t *__restrict__ col,
           const T *__restrict__ sval, const T *__restrict__ X, uint32_t p0, uint32_t n,
           uint32_t sub, uint32_t nvec,
            const Odd<T, VPL, RG> &odd, const Ahead &ex, uint32_t off)
{
    using V = typename Vec<T>::type;
    static_assert(NB <= LPR, "batch must fit the lane group");
    uint32_t e = sub & (NB - 1);
    if (MK)
        e = e < n ? e : n - 1;
    uint32_t cme = 0;
    if constexpr (!PRE)
        cme = nt_load(col + p0 + e);
    const T vme = nt_load(sval + p0 + e);

    V x[NB][VPL];
    T av[NB];
#pragma unroll
    for (int u = 0; u < NB; ++u) {
        const uint32_t c = PRE ? first_col<LPR>(ex.first, off + u) : __shfl(cme, u, LPR);
        av[u] = __shfl(vme, u, LPR);
        gather_row<T, LPR, VPL, RG>(x[u], X, c, sub, nvec, odd);
    }
    __builtin_amdgcn_sched_barrier(0); // all gathers in flight before the first use
    // Entries are added in kernel order.
#pragma unroll
    for (int u = 0; u < NB; ++u) {
        const bool on = !MK || (uint32_t)u < n;
        const T a = on ? av[u] : (T)0;
#pragma unroll
        for (int v = 0; v < VPL; ++v)
            acc[v] += (on ? x[u][v] : V{}) * a;
    }
}

template <typename T, int LPR, int VPL, int NB, int RG, bool MK>
__device__ __forceinline__ void
spmm_batch_rounds(typename Vec<T>::type (&acc)[VPL], const uint32_t *__restrict__ col,
           const T *__restrict__ sval, const T *__restrict__ X, uint32_t p0, uint32_t n,
           uint32_t sub, uint32_t nvec,
            const Odd<T, VPL, RG> &odd)
{
    using V = typename Vec<T>::type;
    // Lane u of the group fetches column and value of entry u of each of the R rounds
    // of G <= LPR entries (see sddmm_batch).
    constexpr int G = NB < LPR ? NB : LPR;
    constexpr int R = NB / G;
    static_assert(R * G == NB, "a batch is a whole number of rounds");
    uint32_t cme[R];
    T vme[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        uint32_t e = (uint32_t)r * G + (sub & (G - 1));
        if (MK)
            e = e < n ? e : n - 1;
        cme[r] = nt_load(col + p0 + e);
        vme[r] = nt_load(sval + p0 + e);
    }

    V x[NB][VPL];
    T av[NB];
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        const uint32_t c = __shfl(cme[j / G], j % G, LPR);
        av[j] = __shfl(vme[j / G], j % G, LPR);
        gather_row<T, LPR, VPL, RG>(x[j], X, c, sub, nvec, odd);
    }
    __builtin_amdgcn_sched_barrier(0); // all gathers in flight before the first use
    // Entries are added in kernel order.
#pragma unroll
    for (int j = 0; j < NB; ++j) {
        const bool on = !MK || (uint32_t)j < n;
        const T w = on ? av[j] : (T)0;
#pragma unroll
        for (int v = 0; v < VPL; ++v)
            acc[v] += (on ? x[j][v] : V{}) * w;
    }
}

template <typename T, int LPR, int VPL, int NB, int RG, bool MK>
__device__ __forceinline__ void
spmm_batch(typename Vec<T>::type (&acc)[VPL], const uint32_t *__restrict__ col,
           const T *__restrict__ sval, const T *__restrict__ X, uint32_t p0, uint32_t n,
           uint32_t sub, uint32_t nvec,
            const Odd<T, VPL, RG> &odd)
{
    const Ahead none{};
    if constexpr (NB <= LPR)
        spmm_batch_one<T, LPR, VPL, NB, RG, MK, false>(acc, col, sval, X, p0, n, sub, nvec, odd,
                                                       none, 0u);
    else
        spmm_batch_rounds<T, LPR, VPL, NB, RG, MK>(acc, col, sval, X, p0, n, sub, nvec, odd);
}

template <typename T, int LPR, int VPL, int UB, int RG, bool WIDE>
__device__ __forceinline__ void
spmm_walk(typename Vec<T>::type (&acc)[VPL], const uint32_t *__restrict__ col,
          const T *__restrict__ sval, const T *__restrict__ X, uint32_t p, uint32_t n,
          uint32_t sub, uint32_t nvec,
            const Odd<T, VPL, RG> &odd, const Ahead &ex)
{
    // Short segments: exact batches of UB, then UB/2 ... 1 as n requires.  Measured
    // against masked batches here (which cost registers, hence occupancy): 3 % faster
    // on 5-entry rows, level elsewhere.  SpMM's short rows are bound by the Y
    // read-modify-write stream, not by rounds of gathers.  The first kFirstCols
    // entries take their column indices from `ex.first`, which was loaded ahead, beside the
    // segment's descriptor.
    if constexpr (!WIDE) {
        static_assert(WIDE || (UB <= 4 && UB <= LPR), "short batches fit the lane group");
        {
            const uint32_t m = n < kFirstCols ? n : kFirstCols;
            uint32_t off = 0;
            for (; off + UB <= m; off += UB)
                spmm_batch_one<T, LPR, VPL, UB, RG, false, true>(acc, col, sval, X, p + off, UB,
                                                                 sub, nvec, odd, ex, off);
            if constexpr (UB > 2)
                if ((m - off) & 2) {
                    spmm_batch_one<T, LPR, VPL, 2, RG, false, true>(acc, col, sval, X, p + off, 2,
                                                                    sub, nvec, odd, ex, off);
                    off += 2;
                }
            if constexpr (UB > 1)
                if ((m - off) & 1)
                    spmm_batch_one<T, LPR, VPL, 1, RG, false, true>(acc, col, sval, X, p + off, 1,
                                                                    sub, nvec, odd, ex, off);
            n -= m;
            p += m;
        }
        for (; n >= UB; n -= UB, p += UB)
            spmm_batch<T, LPR, VPL, UB, RG, false>(acc, col, sval, X, p, UB, sub, nvec, odd);
        if constexpr (UB > 8)
            if (n & 8) {
                spmm_batch<T, LPR, VPL, 8, RG, false>(acc, col, sval, X, p, 8, sub, nvec, odd);
                p += 8;
            }
        if constexpr (UB > 4)
            if (n & 4) {
                spmm_batch<T, LPR, VPL, 4, RG, false>(acc, col, sval, X, p, 4, sub, nvec, odd);
                p += 4;
            }
        if constexpr (UB > 2)
            if (n & 2) {
                spmm_batch<T, LPR, VPL, 2, RG, false>(acc, col, sval, X, p, 2, sub, nvec, odd);
                p += 2;
            }
        if constexpr (UB > 1)
            if (n & 1)
                spmm_batch<T, LPR, VPL, 1, RG, false>(acc, col, sval, X, p, 1, sub, nvec, odd);
    } else {
        for (; n >= UB; n -= UB, p += UB)
            spmm_batch<T, LPR, VPL, UB, RG, false>(acc, col, sval, X, p, UB, sub, nvec, odd);
        if (n == 0)
            return;
        if constexpr (UB > 8) {
            if (n > 8) {
                spmm_batch<T, LPR, VPL, UB, RG, true>(acc, col, sval, X, p, n, sub, nvec, odd);
                return;
            }
        }
        if constexpr (UB > 4) {
            if (n > 4) {
                spmm_batch<T, LPR, VPL, 8, RG, true>(acc, col, sval, X, p, n, sub, nvec, odd);
                return;
            }
        }
        spmm_batch<T, LPR, VPL, (UB < 4 ? UB : 4), RG, true>(acc, col, sval, X, p, n, sub, nvec, odd);
    }
}

template <typename T, int LPR, int VPL, int UB, int RG, bool WIDE>
__global__ void __launch_bounds__(kBlock)
spmm_seg_kernel(const Seg *__restrict__ segs, uint32_t nseg, uint32_t nq, uint32_t rot,
                const uint32_t *__restrict__ col, const T *__restrict__ sval,
                const T *__restrict__ X, T *__restrict__ Y, T *__restrict__ partial,
                uint32_t nvec, uint32_t stride, const uint32_t *__restrict__ first_cols)
{
    static_assert(UB <= 16 && LPR <= 64, "at most 16 entries in flight per lane");
    using V = typename Vec<T>::type;
    const uint32_t sub = threadIdx.x & (LPR - 1);
    const uint64_t sid = seg_index<64 / LPR>(nq, rot);
    if (sid >= nseg)
        return;
    const Ahead ex = load_first_cols<LPR, WIDE>(first_cols, sid, sub);
    const u32x4 sg = nt_load(reinterpret_cast<const u32x4 *>(segs) + sid); // row, start, len, slot
    if (sg[2] == 0)
        return;
    const bool whole = sg[3] == kWholeRow;
    const Odd<T, VPL, RG> odd = odd_lanes<T, LPR, VPL, RG>(sub, nvec, stride, 0u);

    V acc[VPL], y0[VPL];
#pragma unroll
    for (int v = 0; v < VPL; ++v) {
        acc[v] = V{};
        y0[v] = V{};
    }
    if constexpr (RG >= 2) {
        char *drow = const_cast<char *>(whole ? odd_row<T, RG>(Y, sg[0], stride)
                                              : odd_row<T, RG>(partial, sg[3], stride));
        if (whole) {
#pragma unroll
            for (int v = 0; v < VPL; ++v)
                y0[v] = odd_load<T, RG, VPL, true>(drow, v, nvec, odd);
        }
        spmm_walk<T, LPR, VPL, UB, RG, WIDE>(acc, col, sval, X, sg[1], sg[2], sub, nvec, odd, ex);
        odd_store<T, VPL>(drow, whole, y0, acc, odd);
    } else {
        V *dst = const_cast<V *>(whole ? row_ptr<T, LPR, VPL, RG>(Y, sg[0], sub, nvec)
                                       : row_ptr<T, LPR, VPL, RG>(partial, sg[3], sub, nvec));
        if (whole) {
#pragma unroll
            for (int v = 0; v < VPL; ++v)
                if (lane_on<LPR, RG>(sub, v, nvec))
                    y0[v] = nt_load(dst + v * LPR);
        }
        spmm_walk<T, LPR, VPL, UB, RG, WIDE>(acc, col, sval, X, sg[1], sg[2], sub, nvec, odd, ex);
#pragma unroll
        for (int v = 0; v < VPL; ++v) {
            if (!lane_on<LPR, RG>(sub, v, nvec))
                continue;
            if (whole)
                nt_store(y0[v] + acc[v], dst + v * LPR);
            else
                dst[v * LPR] = acc[v]; // read back by spmm_fixup right after
        }
    }
}

// Y[row,:] += the partial sums of a cut row, in slot order.  `lanes` (a power of
// two, <= kBlock) threads share one cut row, kBlock / lanes rows per block.
template <typename T>
__global__ void __launch_bounds__(kBlock)
spmm_fixup_kernel(const SplitRow *__restrict__ splits, uint32_t nsplit,
                  const T *__restrict__ partial, T *__restrict__ Y, uint32_t K, uint32_t lanes)
{
    const uint32_t idx = blockIdx.x * (kBlock / lanes) + threadIdx.x / lanes;
    if (idx >= nsplit)
        return;
    const SplitRow sr = splits[idx];
    for (uint32_t j = threadIdx.x % lanes; j < K; j += lanes) {
        const T *p = partial + (size_t)sr.first_slot * K + j;
        T s = (T)0;
        uint32_t q = 0;
        for (; q + 4 <= sr.nslots; q += 4) { // four loads in flight, added in slot order
            const T v0 = p[(size_t)(q + 0) * K], v1 = p[(size_t)(q + 1) * K];
            const T v2 = p[(size_t)(q + 2) * K], v3 = p[(size_t)(q + 3) * K];
            s = (((s + v0) + v1) + v2) + v3;
        }
        for (; q < sr.nslots; ++q)
            s += p[(size_t)q * K];
        Y[(size_t)sr.row * K + j] += s;
    }
}

// ------------------------------------------------- row tiles x column blocks ----
// Long rows over columns that are not skewed (a hypergraph's incidence matrix: 1024 entries
// per row, uniform over 500 k columns; 512-byte dense rows): every entry gathers a dense row
// that no cache holds unless the columns are visited block by block, and cutting a row at
// every block boundary costs its A row (SDDMM) or its Y row (SpMM) again per piece.  Here a
// workgroup keeps a TILE of rows in LDS for a whole sweep over the column blocks: kSweepRowBytes
// of A rows (SDDMM, read-only) or of Y accumulators (SpMM), one workgroup per CU, one launch
// per "generation" of as many tiles as the GPU has CUs.  The workgroups of a generation start
// together and meet the same amount of work in every block, so they walk the blocks in step,
// and a barrier per block keeps the wavefronts of one workgroup in step too (without it the
// oldest wavefronts run ahead by tens of blocks): at any time one block of dense rows is
// what an L2 sees, and the gathers hit.
//
// The plan (build_sweep in plan_device.h) orders a tile's entries by block, inside a block by
// row; ptr[tile * nb + b] .. [.. + 1) is the range of block b.  Both kernels cut that range
// into batches of UB entries and deal them to the G lane groups of the workgroup, which
// leaves the lane groups within one batch of each other in every block.
// SDDMM, where any lane group can take any entry: batch i to lane group i % G.
// SpMM: lane group g takes the contiguous batches [g per, (g + 1) per), per = ceil(nbat / G).  The sum of
// a row's run of entries is kept in registers and added to the row's accumulator in LDS when
// the run ends.  A row's entries are contiguous, so a row is shared between lane groups only
// where a boundary between two chunks falls inside it: its first part then ends a chunk (and
// is added to the accumulator by that lane group), the later parts each BEGIN a chunk.  The
// first run of every chunk therefore goes to an edge slot of its lane group instead, and
// after the block's barrier the edge slots are added to their rows in lane-group order, one
// lane group per row (the first of those that hold it); a second barrier ends the block.
// No atomics, one fixed order of additions: the same bits run to run.
constexpr int kSweepBlock = 1024;
constexpr uint32_t kSweepRowBytes = 128u << 10; // of LDS for the tile's rows
constexpr uint32_t kSweepPtrWords = 1028;       // nb + 1 range bounds of a tile, in LDS too
template <typename T, int LPR>
__device__ __forceinline__ T sweep_dot(const typename Vec<T>::type &a, const typename Vec<T>::type &b)
{
    T d = a[0] * b[0];
#pragma unroll
    for (int i = 1; i < Vec<T>::N; ++i)
        d += a[i] * b[i];
    return d;
}

// One batch of a lane group: its entries' columns, local rows and (for the lanes that need
// one) sparse values, asked for one batch ahead.
template <typename T> struct SweepIdx {
    uint32_t n = 0, col = 0, row = 0, pos = 0;
    T val = (T)0;
};

template <typename T, int LPR, int UB>
__global__ void __launch_bounds__(kSweepBlock)
sweep_sddmm_kernel(const uint32_t *__restrict__ ptr, const uint32_t *__restrict__ tile_rows,
                   const uint32_t *__restrict__ col, const uint16_t *__restrict__ lrow,
                   const T *__restrict__ sval, const uint32_t *__restrict__ pos,
                   const T *__restrict__ A, const T *__restrict__ B, T *__restrict__ C, uint32_t nb,
                   uint32_t R, uint32_t tile0)
{
    using V = typename Vec<T>::type;
    constexpr uint32_t G = kSweepBlock / LPR;
    __shared__ V tile_a[kSweepRowBytes / 16];
    __shared__ uint32_t lptr[kSweepPtrWords];
    const uint32_t tile = tile0 + blockIdx.x;
    for (uint32_t i = threadIdx.x; i < R * LPR; i += kSweepBlock) {
        const uint32_t g = tile_rows[(uint64_t)tile * R + i / LPR];
        V v{};
        if (g != 0xFFFFFFFFu)
            v = nt_load(reinterpret_cast<const V *>(A) + (uint64_t)g * LPR + i % LPR);
        tile_a[i] = v;
    }
    for (uint32_t i = threadIdx.x; i < nb + 1; i += kSweepBlock)
        lptr[i] = ptr[(uint64_t)tile * nb + i];
    __syncthreads();
    const uint32_t grp = threadIdx.x / LPR, sub = threadIdx.x % LPR;
    const uint32_t uo = entry_of<LPR, UB>(sub);
    const bool wlane = is_writer<LPR, UB>(sub);
    const V *Bv = reinterpret_cast<const V *>(B);
    auto fetch = [&](uint32_t q, uint32_t qhi) {
        SweepIdx<T> x;
        x.n = qhi - q < (uint32_t)UB ? qhi - q : (uint32_t)UB;
        uint32_t e = sub & (UB - 1);
        e = e < x.n ? e : x.n - 1;
        x.col = nt_load(col + q + e);
        x.row = nt_load(lrow + q + e);
        x.val = (wlane && uo < x.n) ? nt_load(sval + q + uo) : (T)0;
        if (pos)
            x.pos = (wlane && uo < x.n) ? nt_load(pos + q + uo) : 0u;
        return x;
    };
    // batch i of a block's range belongs to lane group i % G
    uint32_t p = lptr[0] + grp * UB, hi = lptr[1];
    SweepIdx<T> cur;
    if (p < hi)
        cur = fetch(p, hi);
    for (uint32_t b = 0; b < nb; ++b) {
        uint32_t p_nb = 0, hi_nb = 0; // the next block's range
        if (b + 1 < nb) {
            p_nb = lptr[b + 1] + grp * UB;
            hi_nb = lptr[b + 2];
        }
        const bool had = p < hi;
        while (p < hi) {
            // the next batch's indices (this block's, or the first of the next block) before
            // this batch's gathers
            const uint32_t np = p + G * UB;
            SweepIdx<T> nxt;
            if (np < hi)
                nxt = fetch(np, hi);
            else if (p_nb < hi_nb)
                nxt = fetch(p_nb, hi_nb);
            V bv[UB];
#pragma unroll
            for (int u = 0; u < UB; ++u) {
                const uint32_t c = __shfl(cur.col, u, LPR);
                bv[u] = Bv[(uint64_t)c * LPR + sub];
            }
            __builtin_amdgcn_sched_barrier(0); // all gathers in flight before the first use
            T part[UB];
#pragma unroll
            for (int u = 0; u < UB; ++u) {
                const uint32_t l = __shfl(cur.row, u, LPR);
                part[u] = sweep_dot<T, LPR>(tile_a[l * LPR + sub], bv[u]);
            }
            group_reduce<T, LPR, UB>(part, sub);
            if (wlane && uo < cur.n) {
                if (pos) // the caller's positions: pieces of lines that this workgroup's next
                         // blocks complete, so plain stores, which the L2 merges
                    C[cur.pos] = part[0] * cur.val;
                else
                    nt_store(part[0] * cur.val, C + p + uo); // kernel order: whole lines, streaming
            }
            p = np;
            cur = nxt;
        }
        p = p_nb;
        hi = hi_nb;
        if (!had && p < hi) // nothing of this group in block b: the next batch was not asked for
            cur = fetch(p, hi);
        __syncthreads(); // every lane group leaves block b before any enters block b + 1
    }
}

template <typename T, int LPR, int UB>
__global__ void __launch_bounds__(kSweepBlock)
sweep_spmm_kernel(const uint32_t *__restrict__ ptr, const uint32_t *__restrict__ tile_rows,
                  const uint32_t *__restrict__ col, const uint16_t *__restrict__ lrow,
                  const T *__restrict__ sval, const uint32_t *__restrict__ vpos,
                  const T *__restrict__ X, T *__restrict__ Y, uint32_t nb, uint32_t R, uint32_t tile0)
{
    using V = typename Vec<T>::type;
    constexpr uint32_t G = kSweepBlock / LPR;
    constexpr uint32_t kNone = 0xFFFFFFFFu;
    __shared__ V tile_y[kSweepRowBytes / 16];
    __shared__ V edge[kSweepBlock];   // the sum of the first run of every lane group's chunk
    __shared__ uint32_t edge_row[G];  // and its row (kNone: the chunk is empty)
    __shared__ uint32_t lptr[kSweepPtrWords];
    const uint32_t tile = tile0 + blockIdx.x;
    for (uint32_t i = threadIdx.x; i < R * LPR; i += kSweepBlock)
        tile_y[i] = V{};
    for (uint32_t i = threadIdx.x; i < nb + 1; i += kSweepBlock)
        lptr[i] = ptr[(uint64_t)tile * nb + i];
    __syncthreads();
    const uint32_t grp = threadIdx.x / LPR, sub = threadIdx.x % LPR;
    const V *Xv = reinterpret_cast<const V *>(X);
    auto fetch = [&](uint32_t q, uint32_t qhi) {
        SweepIdx<T> x;
        x.n = qhi - q < (uint32_t)UB ? qhi - q : (uint32_t)UB;
        uint32_t e = sub & (UB - 1);
        e = e < x.n ? e : x.n - 1;
        x.col = nt_load(col + q + e);
        x.row = nt_load(lrow + q + e);
        x.val = vpos ? sval[nt_load(vpos + q + e)] : nt_load(sval + q + e);
        return x;
    };
    // this lane group's chunk of block b: ceil(nbat / G) batches each, from lane group 0 on, so
    // that the lane groups with entries are the first ones and those that share a row are
    // neighbours
    auto chunk = [&](uint32_t b, uint32_t &lo, uint32_t &up) {
        const uint32_t s = lptr[b], e = lptr[b + 1];
        const uint32_t nbat = (e - s + UB - 1) / UB;
        const uint32_t per = (nbat + G - 1) / G;
        const uint64_t first = (uint64_t)grp * per, last = first + per;
        lo = first < nbat ? s + (uint32_t)first * UB : e;
        up = last < nbat ? s + (uint32_t)last * UB : e;
    };
    uint32_t p, hi;
    chunk(0, p, hi);
    SweepIdx<T> cur;
    if (p < hi)
        cur = fetch(p, hi);
    for (uint32_t b = 0; b < nb; ++b) {
        uint32_t p_nb = 0, hi_nb = 0;
        if (b + 1 < nb)
            chunk(b + 1, p_nb, hi_nb);
        const bool had = p < hi;
        uint32_t row = kNone;
        bool first = true; // the run in `acc` is the chunk's first
        V acc{};
        // (The accumulator is read, added to and written back: LDS additions that return
        // nothing, which need no wait, were measured 2.6 times slower for the whole call.)
        auto flush = [&]() {
            if (first)
                edge[threadIdx.x] = acc;
            else
                tile_y[row * LPR + sub] += acc;
        };
        if (sub == 0)
            edge_row[grp] = had ? cur.row : kNone; // lane 0 holds the chunk's first entry
        while (p < hi) {
            const uint32_t np = p + UB;
            SweepIdx<T> nxt;
            if (np < hi)
                nxt = fetch(np, hi);
            else if (p_nb < hi_nb)
                nxt = fetch(p_nb, hi_nb);
            V xv[UB];
#pragma unroll
            for (int u = 0; u < UB; ++u) {
                const uint32_t c = __shfl(cur.col, u, LPR);
                xv[u] = Xv[(uint64_t)c * LPR + sub];
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < UB; ++u) {
                const uint32_t l = __shfl(cur.row, u, LPR);
                const T a = (uint32_t)u < cur.n ? __shfl(cur.val, u, LPR) : (T)0;
                if (l != row) {
                    if (row != kNone) {
                        flush();
                        first = false;
                    }
                    acc = V{};
                    row = l;
                }
                acc += xv[u] * a;
            }
            p = np;
            cur = nxt;
        }
        if (row != kNone)
            flush();
        p = p_nb;
        hi = hi_nb;
        if (!had && p < hi)
            cur = fetch(p, hi);
        __syncthreads(); // the edge slots of block b are written, its direct additions done
        // one lane group per row among the edge slots: the first that holds it adds them all,
        // in lane-group order
        const uint32_t er = edge_row[grp];
        if (er != kNone && (grp == 0 || edge_row[grp - 1] != er)) {
            V sum = tile_y[er * LPR + sub];
            for (uint32_t h = grp; h < G && edge_row[h] == er; ++h)
                sum += edge[h * LPR + sub];
            tile_y[er * LPR + sub] = sum;
        }
        __syncthreads(); // before block b + 1 writes edge slots and accumulators again
    }
    for (uint32_t i = threadIdx.x; i < R * LPR; i += kSweepBlock) {
        const uint32_t g = tile_rows[(uint64_t)tile * R + i / LPR];
        if (g != 0xFFFFFFFFu) {
            V *y = reinterpret_cast<V *>(Y) + (uint64_t)g * LPR + i % LPR;
            nt_store(nt_load(y) + tile_y[i], y);
        }
    }
}

// ---------------------------------------------- row pack / unpack (comm buffers) ----
// The copies either side of the reference's sparse exchanges
// (SparseComm::copy_to_sendbuff / copy_from_recvbuff / SUM_from_recvbuff,
// src/comm.hpp:90-103,166-189): buffer slot i holds the dense row rows[i].
// W = what one lane moves (a 16-byte vector of reals when the row size allows,
// else one real); upr = units of W per row.

// buf[i, :] = panel[rows[i], :]
template <typename W>
__global__ void __launch_bounds__(kBlock)
rows_pack_kernel(const W *__restrict__ panel, const uint32_t *__restrict__ rows, uint64_t total,
                 uint32_t upr, W *__restrict__ buf)
{
    const uint64_t stride = (uint64_t)gridDim.x * kBlock;
    for (uint64_t t = (uint64_t)blockIdx.x * kBlock + threadIdx.x; t < total; t += stride) {
        const uint64_t slot = t / upr;
        const uint32_t v = (uint32_t)(t - slot * upr);
        nt_store(panel[(uint64_t)rows[slot] * upr + v], buf + t);
    }
}

// For every distinct destination row u (urows[u], buffer slots slots[ptr[u] ..
// ptr[u+1]) in ascending slot order): ADD = false: panel row = its last slot
// (what the reference's sequential copy leaves); ADD = true: panel row += each
// slot in order (the reference's sequential sum, bit for bit).
template <typename W, bool ADD>
__global__ void __launch_bounds__(kBlock)
rows_unpack_kernel(W *__restrict__ panel, const uint32_t *__restrict__ urows,
                   const uint32_t *__restrict__ ptr, const uint32_t *__restrict__ slots,
                   uint64_t total, uint32_t upr, const W *__restrict__ buf)
{
    const uint64_t stride = (uint64_t)gridDim.x * kBlock;
    for (uint64_t t = (uint64_t)blockIdx.x * kBlock + threadIdx.x; t < total; t += stride) {
        const uint64_t u = t / upr;
        const uint32_t v = (uint32_t)(t - u * upr);
        W *dst = panel + (uint64_t)urows[u] * upr + v;
        const uint32_t lo = ptr[u], hi = ptr[u + 1];
        if (!ADD) {
            *dst = nt_load(buf + (uint64_t)slots[hi - 1] * upr + v);
        } else {
            W acc = *dst;
            for (uint32_t s = lo; s < hi; ++s)
                acc += nt_load(buf + (uint64_t)slots[s] * upr + v);
            *dst = acc;
        }
    }
}

// XCD on which each workgroup of a 1-D grid runs (hardware register XCC_ID).
__global__ void __launch_bounds__(64) xcc_probe_kernel(uint32_t *__restrict__ out)
{
    // s_getreg_b32 hwreg(HW_REG_XCC_ID = 20, offset 0, width 4)
    const uint32_t id = __builtin_amdgcn_s_getreg(20 | (0 << 6) | ((4 - 1) << 11));
    if (threadIdx.x == 0)
        out[blockIdx.x] = id;
}

// ------------------------------------------------------------- utilities ----
// Measurement aid (launch_probe_cols): the column of every kernel-order entry replaced so
// that the launches keep their instruction stream, segments and queues while every gather
// hits (mode 1: base + (c - base) % modulus, a table of `modulus` dense rows) or nearly
// every gather misses (mode 2: a hash of the entry's position, uniform over ncols).
__global__ void __launch_bounds__(kBlock)
probe_cols_kernel(uint32_t *__restrict__ col, uint64_t n, uint32_t mode, uint32_t base,
                  uint32_t modulus, uint32_t ncols)
{
    const uint64_t stride = (uint64_t)gridDim.x * kBlock;
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) {
        if (mode == 1) {
            const uint32_t c = col[i];
            col[i] = c >= base ? base + (c - base) % modulus : c % modulus;
        } else {
            uint64_t x = (i + 1) * 0x9E3779B97F4A7C15ull; // splitmix64 finaliser
            x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
            x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
            x ^= x >> 31;
            col[i] = (uint32_t)(x % ncols);
        }
    }
}

template <typename T>
__global__ void __launch_bounds__(kBlock)
gather_kernel(const T *__restrict__ in, const uint32_t *__restrict__ perm, T *__restrict__ out,
              uint64_t n)
{
    const uint64_t stride = (uint64_t)gridDim.x * kBlock;
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride)
        out[i] = perm ? in[perm[i]] : in[i];
}

// out[perm[i]] = in[i] (perm null: out[i] = in[i])
template <typename T>
__global__ void __launch_bounds__(kBlock)
scatter_kernel(const T *__restrict__ in, const uint32_t *__restrict__ perm, T *__restrict__ out,
               uint64_t n)
{
    const uint64_t stride = (uint64_t)gridDim.x * kBlock;
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride)
        out[perm ? perm[i] : i] = in[i];
}

// out[i] = in[pos[i]], four results per lane: positions and results move as 16-byte
// vectors, streaming; the reads in between are whatever `pos` makes them (runs, for the
// staged results of a plan kept in column blocks).
template <typename T>
__global__ void __launch_bounds__(kBlock)
gather4_kernel(const T *__restrict__ in, const uint32_t *__restrict__ pos, T *__restrict__ out,
               uint64_t n)
{
    const uint64_t stride = (uint64_t)gridDim.x * kBlock * 4;
    const uint64_t nfull = n / 4 * 4;
    // Workgroups are dealt to the XCDs in turn: workgroup b takes the chunk that gives every
    // XCD a contiguous eighth of each round of chunks, so that neighbours in `out`, whose
    // reads tend to share lines of `in`, meet in one L2.
    uint32_t chunk = blockIdx.x;
    if (gridDim.x % 8 == 0)
        chunk = (blockIdx.x % 8) * (gridDim.x / 8) + blockIdx.x / 8;
    for (uint64_t i = ((uint64_t)chunk * kBlock + threadIdx.x) * 4; i < nfull; i += stride) {
        const u32x4 p = nt_load(reinterpret_cast<const u32x4 *>(pos + i));
        using V = typename Vec<T>::type; // 16 bytes: 4 floats or 2 doubles
        V v[4 / Vec<T>::N];
#pragma unroll
        for (int u = 0; u < 4; ++u)
            v[u / Vec<T>::N][u % Vec<T>::N] = in[p[u]];
#pragma unroll
        for (int u = 0; u < 4 / Vec<T>::N; ++u)
            nt_store(v[u], reinterpret_cast<V *>(out + i) + u);
    }
    const uint64_t t = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    if (t < n - nfull)
        out[nfull + t] = in[pos[nfull + t]];
}

// out[dst[h]] = stage[src[h]], h < n, dst ascending and mostly consecutive: four results in
// flight per lane, consecutive lanes on consecutive h.
template <typename T>
__global__ void __launch_bounds__(kBlock)
unstage_pairs_kernel(const T *__restrict__ stage, const uint32_t *__restrict__ src,
                     const uint32_t *__restrict__ dst, T *__restrict__ out, uint64_t n)
{
    constexpr uint64_t U = 4;
    const uint64_t span = (uint64_t)kBlock * U;
    uint64_t base = (uint64_t)blockIdx.x * span;
    for (; base + span <= n; base += (uint64_t)gridDim.x * span) {
        uint32_t s[U], d[U];
        T v[U];
#pragma unroll
        for (uint64_t u = 0; u < U; ++u) {
            s[u] = nt_load(src + base + u * kBlock + threadIdx.x);
            d[u] = nt_load(dst + base + u * kBlock + threadIdx.x);
        }
#pragma unroll
        for (uint64_t u = 0; u < U; ++u)
            v[u] = nt_load(stage + s[u]);
#pragma unroll
        for (uint64_t u = 0; u < U; ++u)
            nt_store(v[u], out + d[u]);
    }
    // what is left is less than one span, and one workgroup's `base` lies in it
    for (uint64_t h = base + threadIdx.x; h < n; h += kBlock)
        out[dst[h]] = stage[src[h]];
}

// ---- results of an arbitrary entry order to the caller's positions in two passes ------
// (see TwoPass in plan_device.h).  One workgroup per tile of kTwoPassBytes of results,
// held in LDS between its coalesced read and its grouped write.
constexpr uint32_t kTwoPassBytes = 160u << 10; // all of a CU's LDS
constexpr int kTwoPassBlock = 1024;
template <typename T> constexpr uint32_t two_pass_tile() { return kTwoPassBytes / sizeof(T); }

template <typename T>
__device__ __forceinline__ void tile_to_lds(T *buf, const T *__restrict__ src, uint32_t cnt)
{
    using V = typename Vec<T>::type;
    constexpr uint32_t VN = Vec<T>::N;
    constexpr uint32_t TILE = two_pass_tile<T>();
    constexpr uint32_t R = TILE / VN / kTwoPassBlock; // 16-byte loads per lane and tile: 10
    static_assert(R * VN * kTwoPassBlock == TILE, "a tile is a whole number of rounds");
    const V *in = reinterpret_cast<const V *>(src); // 16-byte aligned: a whole tile into a library buffer
    V *to = reinterpret_cast<V *>(buf);
    if (cnt == TILE) { // every load in flight before the first word is stored
        V v[R];
#pragma unroll
        for (uint32_t r = 0; r < R; ++r)
            v[r] = nt_load(in + threadIdx.x + r * kTwoPassBlock);
#pragma unroll
        for (uint32_t r = 0; r < R; ++r)
            to[threadIdx.x + r * kTwoPassBlock] = v[r];
        return;
    }
    const uint32_t nvec = cnt / VN;
    for (uint32_t i = threadIdx.x; i < nvec; i += kTwoPassBlock)
        to[i] = nt_load(in + i);
    for (uint32_t i = nvec * VN + threadIdx.x; i < cnt; i += kTwoPassBlock)
        buf[i] = src[i];
}

// Pass 1: tile blockIdx.x of `stage` (kernel order), out grouped by bucket of destination.
template <typename T>
__global__ void __launch_bounds__(kTwoPassBlock)
unpermute_pass1_kernel(const T *__restrict__ stage, const uint16_t *__restrict__ l1,
                       const uint32_t *__restrict__ dst1, T *__restrict__ mid, uint64_t n)
{
    constexpr uint32_t TILE = two_pass_tile<T>();
    __shared__ T buf[TILE];
    const uint64_t base = (uint64_t)blockIdx.x * TILE;
    if (base >= n)
        return;
    const uint32_t cnt = (uint32_t)(n - base < TILE ? n - base : TILE);
    constexpr uint32_t U = 10;
    // the first positions are asked for before the tile is: they do not depend on it
    uint32_t l[U], d[U];
    uint32_t s = threadIdx.x;
    const bool first_full = s + (U - 1) * kTwoPassBlock < cnt;
    if (first_full) {
#pragma unroll
        for (uint32_t u = 0; u < U; ++u) {
            l[u] = nt_load(l1 + base + s + u * kTwoPassBlock);
            d[u] = nt_load(dst1 + base + s + u * kTwoPassBlock);
        }
    }
    tile_to_lds(buf, stage + base, cnt);
    __syncthreads();
    if (first_full) {
#pragma unroll
        for (uint32_t u = 0; u < U; ++u)
            nt_store(buf[l[u]], mid + d[u]);
        s += U * kTwoPassBlock;
    }
    for (; s + (U - 1) * kTwoPassBlock < cnt; s += U * kTwoPassBlock) {
#pragma unroll
        for (uint32_t u = 0; u < U; ++u) {
            l[u] = nt_load(l1 + base + s + u * kTwoPassBlock);
            d[u] = nt_load(dst1 + base + s + u * kTwoPassBlock);
        }
#pragma unroll
        for (uint32_t u = 0; u < U; ++u)
            nt_store(buf[l[u]], mid + d[u]);
    }
    for (; s < cnt; s += kTwoPassBlock)
        nt_store(buf[nt_load(l1 + base + s)], mid + nt_load(dst1 + base + s));
}

// Pass 2: bucket blockIdx.x of `mid`, out to the caller's positions [base, base + cnt) in order.
template <typename T>
__global__ void __launch_bounds__(kTwoPassBlock)
unpermute_pass2_kernel(const T *__restrict__ mid, const uint16_t *__restrict__ l2,
                       T *__restrict__ C, uint64_t n)
{
    using V = typename Vec<T>::type;
    constexpr uint32_t VN = Vec<T>::N;
    constexpr uint32_t TILE = two_pass_tile<T>();
    __shared__ T buf[TILE];
    const uint64_t base = (uint64_t)blockIdx.x * TILE;
    if (base >= n)
        return;
    const uint32_t cnt = (uint32_t)(n - base < TILE ? n - base : TILE);
    typedef uint16_t Idx __attribute__((ext_vector_type(VN)));
    constexpr uint32_t R = TILE / VN / kTwoPassBlock; // 16-byte stores per lane and tile: 10
    T *out = C + base;
    const bool fast = cnt == TILE && (reinterpret_cast<uintptr_t>(out) & 15u) == 0;
    Idx li[R];
    if (fast) { // the positions do not depend on the tile: asked for first
#pragma unroll
        for (uint32_t r = 0; r < R; ++r)
            li[r] = nt_load(reinterpret_cast<const Idx *>(l2 + base) + threadIdx.x + r * kTwoPassBlock);
    }
    tile_to_lds(buf, mid + base, cnt);
    __syncthreads();
    if (fast) {
#pragma unroll
        for (uint32_t r = 0; r < R; ++r) {
            V v;
#pragma unroll
            for (uint32_t e = 0; e < VN; ++e)
                v[e] = buf[li[r][e]];
            nt_store(v, reinterpret_cast<V *>(out) + threadIdx.x + r * kTwoPassBlock);
        }
        return;
    }
    uint32_t done = 0;
    if ((reinterpret_cast<uintptr_t>(out) & 15u) == 0) { // the caller's C may be a wrapped vector
        const uint32_t nvec = cnt / VN;
        for (uint32_t i = threadIdx.x; i < nvec; i += kTwoPassBlock) {
            const Idx l = nt_load(reinterpret_cast<const Idx *>(l2 + base) + i);
            V v;
#pragma unroll
            for (uint32_t e = 0; e < VN; ++e)
                v[e] = buf[l[e]];
            nt_store(v, reinterpret_cast<V *>(out) + i);
        }
        done = nvec * VN;
    }
    for (uint32_t j = done + threadIdx.x; j < cnt; j += kTwoPassBlock)
        out[j] = buf[l2[base + j]];
}

template <typename T>
__global__ void __launch_bounds__(kBlock) fill_kernel(T *__restrict__ p, uint64_t n, T value)
{
    const uint64_t stride = (uint64_t)gridDim.x * kBlock;
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride)
        p[i] = value;
}

// Plain streaming copy: four 16-byte non-temporal loads in flight per lane, then
// four non-temporal stores (5.8 TB/s read + written on this GPU; one load per
// iteration with plain accesses gives 4.6).  The last (< 4 * block) vectors go
// one by one, the tail (< 16 bytes) bytewise by the first lanes.
__global__ void __launch_bounds__(kBlock)
copy_kernel(u32x4 *__restrict__ dst, const u32x4 *__restrict__ src, uint64_t nvec,
            uint32_t tail_bytes)
{
    constexpr uint64_t U = 4;
    const uint64_t tid = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
    const uint64_t span = (uint64_t)kBlock * U; // vectors one block moves per iteration
    const uint64_t nfull = nvec / span * span;
    for (uint64_t i = (uint64_t)blockIdx.x * span + threadIdx.x; i < nfull;
         i += (uint64_t)gridDim.x * span) {
        u32x4 v[U];
#pragma unroll
        for (uint64_t u = 0; u < U; ++u)
            v[u] = nt_load(src + i + u * kBlock);
#pragma unroll
        for (uint64_t u = 0; u < U; ++u)
            nt_store(v[u], dst + i + u * kBlock);
    }
    for (uint64_t i = nfull + tid; i < nvec; i += (uint64_t)gridDim.x * kBlock)
        dst[i] = src[i];
    if (tid < tail_bytes)
        reinterpret_cast<unsigned char *>(dst + nvec)[tid] =
            reinterpret_cast<const unsigned char *>(src + nvec)[tid];
}

// ------------------------------------------------------------- dispatch ----
struct Shape {
    int lpr, vpl;  // lpr == 0: rows over 4 KiB, run slice by slice
    int mode;      // the kernels' RG: 0 exact, 1 ragged, 2 odd, 3 thin
    uint32_t nvec; // 16-byte vectors per dense row; modes 2, 3: K, the reals per row
};

// A dense row of K reals of at most 4096 bytes runs in one launch (pair); longer ones
// go slice by slice, rows under 16 bytes take the "thin" variant of the 4-lane shape.  A whole number nvec of 16-byte
// vectors with nvec == LPR * VPL, LPR a power of two in [4, 64] and VPL in {1, 2, 4},
// runs a kernel with the row stride compiled in; other nvec run the "ragged" variant
// of the smallest shape that covers a row, in which the lanes past the row's end
// idle; rows that are no whole number of vectors, or of at most 16, run the "odd"
// variant of that shape.
Shape pick_shape(size_t elem, uint32_t K)
{
    const size_t bytes = (size_t)K * elem;
    if (K == 0 || bytes > 4096)
        return {0, 0, 0, 0};
    if (bytes < 16)
        return {4, 1, 3, K};
    const uint32_t nvec = (uint32_t)((bytes + 15) / 16);
    const bool odd = bytes % 16 != 0;
    for (int lpr = 64; lpr >= 4 && !odd; lpr >>= 1) {
        if (nvec % lpr)
            continue;
        const uint32_t vpl = nvec / lpr;
        if (vpl == 1 || vpl == 2 || vpl == 4)
            return {lpr, (int)vpl, 0, nvec};
        break;
    }
    // Narrow rows that leave lanes idle also run the odd variant: its idle lanes load a
    // vector of the row and count nothing, where the ragged variant's skip the load
    // under a branch (measured on R-MAT 20, fp32 K = 4: SDDMM 644 -> 557 us, SpMM
    // 467 -> 339 us; K = 20: 510 -> 446 and 404 -> 324; level at 9 to 16 vectors, and
    // from 17 vectors on the selects in the dot product cost SDDMM 2 to 4 %).
    const int mode = (odd || nvec <= 16) ? 2 : 1;
    const uint32_t arg = mode == 2 ? K : nvec;
    if (nvec > 128)
        return {64, 4, mode, arg};
    if (nvec > 64)
        return {64, 2, mode, arg};
    int lpr = 4;
    while ((uint32_t)lpr < nvec)
        lpr *= 2;
    return {lpr, 1, mode, arg};
}

// Workgroups needed to cover nseg segments (a whole number of chunks, and of
// rounds of 8 chunks when they are dealt to XCDs) with `groups_per_wave` segments
// per wavefront.
inline uint32_t blocks_for_groups(uint32_t nseg, uint32_t nq, int groups_per_wave)
{
    uint64_t chunks = ((uint64_t)nseg + kChunk - 1) / kChunk;
    if (nq == 8)
        chunks = (chunks + 7) / 8 * 8;
    return (uint32_t)(chunks * (kChunk / ((kBlock / 64) * groups_per_wave)));
}

// Two launches per call: the leading nseg_long segments (all at least
// kLongSegment entries long) run with UB gathers in flight per lane and
// 4 wavefronts per SIMD; the rest run the US-wide variant, whose register
// budget lets 8 wavefronts per SIMD hide the three dependent memory latencies
// of a short segment (descriptor -> indices -> gathers).  Measured: 5-entry
// rows of a stencil 1.6x faster with US = 4 than with 16, R-MAT hub segments
// 1.5x slower.  With an auxiliary stream the two run side by side.

// A pattern this small does not keep the chip busy for long enough to repay a
// second launch with its fork and join (about 20 us when the kernels are short):
// when it has segments of both kinds, all of them go to the wide launch (either
// kernel handles segments of any length; the long ones hold most of the entries).
// Measured on R-MAT 14 .. 19: one launch wins up to about 180 k segments (11 against
// 32 us at 12 k), two from 400 k on.
constexpr uint32_t kOneLaunchSegments = 196608;

// Makes the auxiliary stream wait for everything queued on the main stream so
// far.  On failure nothing was queued on aux and the caller stays on main.
inline bool fork_aux(const Streams &S)
{
    return S.aux && hipEventRecord(S.fork, S.main) == hipSuccess &&
           hipStreamWaitEvent(S.aux, S.fork, 0) == hipSuccess;
}

// Makes the main stream wait for what was queued on the auxiliary stream; if the
// events fail, waits on the host instead, so the ordering holds either way.
inline hipError_t join_aux(const Streams &S)
{
    if (hipEventRecord(S.join, S.aux) == hipSuccess &&
        hipStreamWaitEvent(S.main, S.join, 0) == hipSuccess)
        return hipSuccess;
    (void)hipGetLastError();
    return hipStreamSynchronize(S.aux);
}

inline uint32_t store_flags(const DevPlanView &P)
{
    return (P.stream_c ? kStoreStream : 0u) | (P.perm && P.seg_base ? kStoreSegBase : 0u);
}

template <typename T, int LPR, int VPL, int UB, int US, int RG, int FZ>
hipError_t run_sddmm(const DevPlanView &P, const T *A, const T *B, T *C, T *Y, const Streams &S,
                     uint32_t nvec, uint32_t stride = 0, uint32_t accum = 0)
{
    uint32_t nl = P.nseg_long, ns = P.nseg - P.nseg_long;
    if (nl && ns && P.nseg <= kOneLaunchSegments)
        nl = P.nseg, ns = 0;
    const bool both = nl && ns && fork_aux(S);
    if (nl)
        hipLaunchKernelGGL((sddmm_seg_kernel<T, LPR, VPL, UB, RG, true, FZ>),
                           dim3(blocks_for_groups(nl, P.nqueues, 64 / LPR)), dim3(kBlock), 0,
                           S.main, P.segs, nl, P.nqueues, 0u, P.col, P.perm, (const T *)P.sval,
                           A, B, C, Y, (T *)P.partial, nvec, stride ? stride : nvec, accum,
                           (const uint32_t *)nullptr, store_flags(P), (T *)P.stage,
                           P.stage_from);
    if (ns)
        hipLaunchKernelGGL((sddmm_seg_kernel<T, LPR, VPL, US, RG, false, FZ>),
                           dim3(blocks_for_groups(ns, P.nqueues, 64 / LPR)), dim3(kBlock), 0,
                           both ? S.aux : S.main, P.segs + nl, ns, P.nqueues,
                           both ? S.aux_rot : 0u, P.col, P.perm, (const T *)P.sval, A, B, C, Y,
                           (T *)P.partial, nvec, stride ? stride : nvec, accum, P.first_cols,
                           store_flags(P), (T *)P.stage, P.stage_from);
    const hipError_t launched = hipGetLastError();
    const hipError_t joined = both ? join_aux(S) : hipSuccess;
    return launched != hipSuccess ? launched : joined;
}

template <typename T, int LPR, int VPL, int UB, int US, int RG>
hipError_t run_spmm(const DevPlanView &P, const T *X, T *Y, const Streams &S, uint32_t nvec,
                    uint32_t stride = 0, size_t slice_off = 0)
{
    uint32_t nl = P.nseg_long, ns = P.nseg - P.nseg_long;
    if (nl && ns && P.nseg <= kOneLaunchSegments)
        nl = P.nseg, ns = 0;
    const bool both = nl && ns && fork_aux(S);
    if (nl)
        hipLaunchKernelGGL((spmm_seg_kernel<T, LPR, VPL, UB, RG, true>),
                           dim3(blocks_for_groups(nl, P.nqueues, 64 / LPR)), dim3(kBlock), 0,
                           S.main, P.segs, nl, P.nqueues, 0u, P.col, (const T *)P.sval, X, Y,
                           (T *)P.partial + slice_off, nvec, stride ? stride : nvec,
                           (const uint32_t *)nullptr);
    if (ns)
        hipLaunchKernelGGL((spmm_seg_kernel<T, LPR, VPL, US, RG, false>),
                           dim3(blocks_for_groups(ns, P.nqueues, 64 / LPR)), dim3(kBlock), 0,
                           both ? S.aux : S.main, P.segs + nl, ns, P.nqueues,
                           both ? S.aux_rot : 0u, P.col, (const T *)P.sval, X, Y,
                           (T *)P.partial + slice_off, nvec, stride ? stride : nvec, P.first_cols);
    const hipError_t launched = hipGetLastError();
    const hipError_t joined = both ? join_aux(S) : hipSuccess;
    return launched != hipSuccess ? launched : joined;
}

// (LPR, VPL, UB, US_SDDMM, US_SPMM): UB * VPL 16-byte gathers are in flight per
// lane in the long-segment launch, US * VPL in the short-segment one.
#define SPC3D_FOR_SHAPES(X)                                                                       \
    X(4, 1, 16, 8, 4) X(8, 1, 16, 8, 4) X(16, 1, 16, 8, 4) X(32, 1, 16, 8, 4) X(64, 1, 16, 8, 4)  \
    X(4, 2, 8, 4, 2) X(8, 2, 8, 4, 2) X(16, 2, 8, 4, 2) X(32, 2, 8, 4, 2) X(64, 2, 8, 4, 2)       \
    X(4, 4, 4, 2, 1) X(8, 4, 4, 2, 1) X(16, 4, 4, 2, 1) X(32, 4, 4, 2, 1) X(64, 4, 4, 2, 1)
// Rows that do not fill a shape: the smallest power-of-two LPR covering the row,
// then 64 lanes with 2 or 4 vectors each.  The ragged variants are only used from
// 17 vectors per row on.
#define SPC3D_FOR_ODD_SHAPES(X)                                                                   \
    X(4, 1, 16, 8, 4) X(8, 1, 16, 8, 4) X(16, 1, 16, 8, 4) X(32, 1, 16, 8, 4) X(64, 1, 16, 8, 4)  \
    X(64, 2, 8, 4, 2) X(64, 4, 4, 2, 1)
#define SPC3D_FOR_RAGGED_SHAPES(X) X(32, 1, 16, 8, 4) X(64, 1, 16, 8, 4) X(64, 2, 8, 4, 2) X(64, 4, 4, 2, 1)

template <typename T>
hipError_t launch_fixup(const DevPlanView &P, T *Y, uint32_t K, hipStream_t st)
{
    if (!P.nsplit)
        return hipSuccess;
    uint32_t lanes = 4;
    while (lanes < (uint32_t)kBlock && lanes < K)
        lanes *= 2;
    const uint32_t rows_per_block = kBlock / lanes;
    hipLaunchKernelGGL((spmm_fixup_kernel<T>),
                       dim3((P.nsplit + rows_per_block - 1) / rows_per_block), dim3(kBlock), 0, st,
                       P.splits, P.nsplit, (const T *)P.partial, Y, K, lanes);
    return hipGetLastError();
}

// The shape of rows that end inside a vector (mode 2) or are shorter than one (mode
// 3), for a slice of sh.nvec columns of rows `stride` reals apart.
Shape odd_shape(size_t elem, uint32_t K)
{
    const size_t bytes = (size_t)K * elem;
    if (bytes < 16)
        return {4, 1, 3, K};
    const uint32_t nvec = (uint32_t)((bytes + 15) / 16);
    if (nvec > 128)
        return {64, 4, 2, K};
    if (nvec > 64)
        return {64, 2, 2, K};
    int lpr = 4;
    while ((uint32_t)lpr < nvec)
        lpr *= 2;
    return {lpr, 1, 2, K};
}

template <typename T, int FZ>
hipError_t run_sddmm_odd(const Shape &sh, const DevPlanView &P, const T *A, const T *B, T *C,
                         T *Y, const Streams &SS, uint32_t stride, uint32_t accum)
{
#define X(L, V, U, S, S2)                                                                         \
    if (sh.mode == 2 && sh.lpr == L && sh.vpl == V)                                               \
        return run_sddmm<T, L, V, U, S, 2, FZ>(P, A, B, C, Y, SS, sh.nvec, stride, accum);
    SPC3D_FOR_ODD_SHAPES(X)
#undef X
    if (sh.mode == 3)
        return run_sddmm<T, 4, 1, 16, 8, 3, FZ>(P, A, B, C, Y, SS, sh.nvec, stride, accum);
    return hipErrorInvalidValue;
}

// Rows over 4 KiB go slice by slice: whole 4 KiB slices of columns first (all 256
// vector slots of the 64 x 4 shape busy), then what is left of the row, each slice a
// launch over the whole pattern that adds its part of the dot products to C.
constexpr uint32_t kSliceBytes = 4096;

// FZ == 0: SDDMM.  FZ == 1, 2: SDDMM fused with the SpMM of the same pattern over
// the same B (hipErrorNotSupported for rows over 4 KiB).
template <typename T, int FZ>
hipError_t sddmm_typed(const DevPlanView &P, const void *A, const void *B, void *C, void *Y,
                       uint32_t K, const Streams &SS)
{
    const hipStream_t st = SS.main;
    if (P.nseg == 0)
        return hipSuccess;
    const Shape sh = pick_shape(sizeof(T), K);
    bool done = false;
    hipError_t e = hipSuccess;
#define X(L, V, U, S, S2)                                                                         \
    if (!done && sh.mode == 0 && sh.lpr == L && sh.vpl == V) {                                    \
        e = run_sddmm<T, L, V, U, S, 0, FZ>(P, (const T *)A, (const T *)B, (T *)C, (T *)Y, SS,    \
                                            sh.nvec);                                             \
        done = true;                                                                              \
    }
    SPC3D_FOR_SHAPES(X)
#undef X
#define X(L, V, U, S, S2)                                                                         \
    if (!done && sh.mode == 1 && sh.lpr == L && sh.vpl == V) {                                    \
        e = run_sddmm<T, L, V, U, S, 1, FZ>(P, (const T *)A, (const T *)B, (T *)C, (T *)Y, SS,    \
                                            sh.nvec);                                             \
        done = true;                                                                              \
    }
    SPC3D_FOR_RAGGED_SHAPES(X)
#undef X
    if (!done && sh.mode >= 2) {
        e = run_sddmm_odd<T, FZ>(sh, P, (const T *)A, (const T *)B, (T *)C, (T *)Y, SS, K, 0u);
        done = true;
    }
    if (!done) {
        if constexpr (FZ != 0) {
            return hipErrorNotSupported;
        } else {
            const uint32_t per = kSliceBytes / (uint32_t)sizeof(T);
            for (uint32_t at = 0; at < K && e == hipSuccess; at += per) {
                const uint32_t w = K - at < per ? K - at : per;
                e = run_sddmm_odd<T, 0>(odd_shape(sizeof(T), w), P, (const T *)A + at,
                                        (const T *)B + at, (T *)C, nullptr, SS, K, at != 0);
            }
        }
    }
    const hipError_t last = hipGetLastError();
    if (e != hipSuccess || last != hipSuccess)
        return e != hipSuccess ? e : last;
    return FZ != 0 ? launch_fixup<T>(P, (T *)Y, K, st) : hipSuccess;
}

template <typename T>
hipError_t run_spmm_odd(const Shape &sh, const DevPlanView &P, const T *X, T *Y,
                        const Streams &SS, uint32_t stride, size_t slice_off)
{
#define X(L, V, U, S, S2)                                                                         \
    if (sh.mode == 2 && sh.lpr == L && sh.vpl == V)                                               \
        return run_spmm<T, L, V, U, S2, 2>(P, X, Y, SS, sh.nvec, stride, slice_off);
    SPC3D_FOR_ODD_SHAPES(X)
#undef X
    if (sh.mode == 3)
        return run_spmm<T, 4, 1, 16, 4, 3>(P, X, Y, SS, sh.nvec, stride, slice_off);
    return hipErrorInvalidValue;
}

template <typename T>
hipError_t spmm_typed(const DevPlanView &P, const void *X_, void *Y, uint32_t K,
                      const Streams &SS)
{
    const hipStream_t st = SS.main;
    if (P.nseg == 0)
        return hipSuccess;
    const Shape sh = pick_shape(sizeof(T), K);
    bool done = false;
    hipError_t e = hipSuccess;
#define X(L, V, U, S, S2)                                                                         \
    if (!done && sh.mode == 0 && sh.lpr == L && sh.vpl == V) {                                    \
        e = run_spmm<T, L, V, U, S2, 0>(P, (const T *)X_, (T *)Y, SS, sh.nvec);                   \
        done = true;                                                                              \
    }
    SPC3D_FOR_SHAPES(X)
#undef X
#define X(L, V, U, S, S2)                                                                         \
    if (!done && sh.mode == 1 && sh.lpr == L && sh.vpl == V) {                                    \
        e = run_spmm<T, L, V, U, S2, 1>(P, (const T *)X_, (T *)Y, SS, sh.nvec);                   \
        done = true;                                                                              \
    }
    SPC3D_FOR_RAGGED_SHAPES(X)
#undef X
    if (!done && sh.mode >= 2) {
        e = run_spmm_odd<T>(sh, P, (const T *)X_, (T *)Y, SS, K, 0);
        done = true;
    }
    if (!done) {
        // rows over 4 KiB, slice by slice (see sddmm_typed); the slices of Y and of the
        // partial-sum rows are disjoint
        const uint32_t per = kSliceBytes / (uint32_t)sizeof(T);
        for (uint32_t at = 0; at < K && e == hipSuccess; at += per) {
            const uint32_t w = K - at < per ? K - at : per;
            e = run_spmm_odd<T>(odd_shape(sizeof(T), w), P, (const T *)X_ + at, (T *)Y + at, SS, K,
                                at);
        }
    }
    if (e == hipSuccess)
        e = hipGetLastError();
    if (e != hipSuccess)
        return e;
    return launch_fixup<T>(P, (T *)Y, K, st);
}

inline uint32_t stream_grid(uint64_t n)
{
    const uint64_t want = (n + kBlock - 1) / kBlock;
    const uint64_t cap = 256 * 32; // 32 blocks per CU keeps a grid-stride loop busy
    return (uint32_t)(want < 1 ? 1 : (want > cap ? cap : want));
}

} // namespace

hipError_t launch_sddmm(int dtype, const DevPlanView &P, const void *A, const void *B, void *C,
                        uint32_t K, const Streams &stream)
{
    return dtype == 1 ? sddmm_typed<double, 0>(P, A, B, C, nullptr, K, stream)
                      : sddmm_typed<float, 0>(P, A, B, C, nullptr, K, stream);
}

hipError_t launch_sddmm_spmm(int dtype, int chained, const DevPlanView &P, const void *A,
                             const void *B, void *C, void *Y, uint32_t K, const Streams &stream)
{
    if (dtype == 1)
        return chained ? sddmm_typed<double, 2>(P, A, B, C, Y, K, stream)
                       : sddmm_typed<double, 1>(P, A, B, C, Y, K, stream);
    return chained ? sddmm_typed<float, 2>(P, A, B, C, Y, K, stream)
                   : sddmm_typed<float, 1>(P, A, B, C, Y, K, stream);
}

hipError_t launch_spmm(int dtype, const DevPlanView &P, const void *X, void *Y, uint32_t K,
                       const Streams &stream)
{
    return dtype == 1 ? spmm_typed<double>(P, X, Y, K, stream)
                      : spmm_typed<float>(P, X, Y, K, stream);
}

uint32_t sweep_lanes(int dtype, uint32_t K)
{
    const uint64_t bytes = (uint64_t)K * (dtype == 1 ? 8 : 4);
    return bytes == 256 ? 16u : (bytes == 512 ? 32u : (bytes == 1024 ? 64u : 0u));
}
uint32_t sweep_groups(uint32_t lanes) { return lanes ? kSweepBlock / lanes : 0; }
uint32_t sweep_rows_per_tile(uint32_t lanes) { return lanes ? kSweepRowBytes / (lanes * 16) : 0; }
uint32_t sweep_max_blocks(uint32_t lanes) { return lanes ? kSweepPtrWords - 1 : 0; }

namespace {
template <typename T, int LPR>
void sweep_launch(bool spmm, const SweepView &S, const T *A, const T *B, T *out, uint32_t tile0,
                  uint32_t ntiles, hipStream_t stream)
{
    if (spmm)
        hipLaunchKernelGGL((sweep_spmm_kernel<T, LPR, 16>), dim3(ntiles), dim3(kSweepBlock), 0,
                           stream, S.ptr, S.tile_rows, S.col, S.lrow, (const T *)S.sval, S.pos, B,
                           out, S.nblocks, S.rows_per_tile, tile0);
    else
        hipLaunchKernelGGL((sweep_sddmm_kernel<T, LPR, 16>), dim3(ntiles), dim3(kSweepBlock), 0,
                           stream, S.ptr, S.tile_rows, S.col, S.lrow, (const T *)S.sval, S.pos, A,
                           B, out, S.nblocks, S.rows_per_tile, tile0);
}
template <typename T>
hipError_t sweep_run(bool spmm, const SweepView &S, const T *A, const T *B, T *out, hipStream_t stream)
{
    if (S.ntiles == 0)
        return hipSuccess;
    // what the kernels assume of the plan: the tile's rows and range bounds fit their LDS
    if ((S.lanes != 16 && S.lanes != 32 && S.lanes != 64) || S.per_launch == 0 ||
        S.rows_per_tile * S.lanes * 16 > kSweepRowBytes ||
        (uint64_t)S.nblocks + 1 > kSweepPtrWords)
        return hipErrorInvalidValue;
    for (uint32_t t0 = 0; t0 < S.ntiles; t0 += S.per_launch) { // one generation per launch
        const uint32_t n = S.ntiles - t0 < S.per_launch ? S.ntiles - t0 : S.per_launch;
        if (S.lanes == 16)
            sweep_launch<T, 16>(spmm, S, A, B, out, t0, n, stream);
        else if (S.lanes == 32)
            sweep_launch<T, 32>(spmm, S, A, B, out, t0, n, stream);
        else
            sweep_launch<T, 64>(spmm, S, A, B, out, t0, n, stream);
    }
    return hipGetLastError();
}
} // namespace

hipError_t launch_sweep_sddmm(int dtype, const SweepView &S, const void *A, const void *B, void *C,
                              hipStream_t stream)
{
    return dtype == 1 ? sweep_run<double>(false, S, (const double *)A, (const double *)B, (double *)C, stream)
                      : sweep_run<float>(false, S, (const float *)A, (const float *)B, (float *)C, stream);
}

hipError_t launch_sweep_spmm(int dtype, const SweepView &S, const void *X, void *Y, hipStream_t stream)
{
    return dtype == 1 ? sweep_run<double>(true, S, nullptr, (const double *)X, (double *)Y, stream)
                      : sweep_run<float>(true, S, nullptr, (const float *)X, (float *)Y, stream);
}

hipError_t launch_first_cols(const Seg *segs, uint32_t n, const uint32_t *col, uint32_t *first_cols,
                             hipStream_t stream)
{
    if (n == 0)
        return hipSuccess;
    const uint64_t threads = (uint64_t)n * kFirstCols;
    hipLaunchKernelGGL(first_cols_kernel, dim3((uint32_t)((threads + kBlock - 1) / kBlock)),
                       dim3(kBlock), 0, stream, segs, n, col, first_cols);
    return hipGetLastError();
}

hipError_t launch_unstage(int dtype, const void *in, const uint32_t *pos, void *out, uint64_t n,
                          hipStream_t stream)
{
    if (n == 0)
        return hipSuccess;
    const uint32_t grid = stream_grid((n + 3) / 4);
    if (dtype == 1)
        hipLaunchKernelGGL((gather4_kernel<double>), dim3(grid), dim3(kBlock), 0, stream,
                           (const double *)in, pos, (double *)out, n);
    else
        hipLaunchKernelGGL((gather4_kernel<float>), dim3(grid), dim3(kBlock), 0, stream,
                           (const float *)in, pos, (float *)out, n);
    return hipGetLastError();
}

hipError_t launch_unstage_pairs(int dtype, const void *stage, const uint32_t *src,
                                const uint32_t *dst, void *out, uint64_t n, hipStream_t stream)
{
    if (n == 0)
        return hipSuccess;
    const uint64_t want = (n + (uint64_t)kBlock * 4 - 1) / ((uint64_t)kBlock * 4);
    const uint32_t grid = (uint32_t)(want > 65536 ? 65536 : want);
    if (dtype == 1)
        hipLaunchKernelGGL((unstage_pairs_kernel<double>), dim3(grid), dim3(kBlock), 0, stream,
                           (const double *)stage, src, dst, (double *)out, n);
    else
        hipLaunchKernelGGL((unstage_pairs_kernel<float>), dim3(grid), dim3(kBlock), 0, stream,
                           (const float *)stage, src, dst, (float *)out, n);
    return hipGetLastError();
}

uint32_t two_pass_lds_bytes() { return kTwoPassBytes; }

uint32_t two_pass_tile_elems(int dtype)
{
    return dtype == 1 ? two_pass_tile<double>() : two_pass_tile<float>();
}

hipError_t launch_unpermute_two_pass(int dtype, const void *stage, void *mid, const uint16_t *l1,
                                     const uint32_t *dst1, const uint16_t *l2, void *out, uint64_t n,
                                     hipStream_t stream)
{
    if (n == 0)
        return hipSuccess;
    const uint64_t T = two_pass_tile_elems(dtype);
    const uint32_t grid = (uint32_t)((n + T - 1) / T);
    if (dtype == 1) {
        hipLaunchKernelGGL((unpermute_pass1_kernel<double>), dim3(grid), dim3(kTwoPassBlock), 0,
                           stream, (const double *)stage, l1, dst1, (double *)mid, n);
        hipLaunchKernelGGL((unpermute_pass2_kernel<double>), dim3(grid), dim3(kTwoPassBlock), 0,
                           stream, (const double *)mid, l2, (double *)out, n);
    } else {
        hipLaunchKernelGGL((unpermute_pass1_kernel<float>), dim3(grid), dim3(kTwoPassBlock), 0,
                           stream, (const float *)stage, l1, dst1, (float *)mid, n);
        hipLaunchKernelGGL((unpermute_pass2_kernel<float>), dim3(grid), dim3(kTwoPassBlock), 0,
                           stream, (const float *)mid, l2, (float *)out, n);
    }
    return hipGetLastError();
}

hipError_t launch_scatter_vals(int dtype, const void *in, const uint32_t *perm, void *out,
                               uint64_t n, hipStream_t stream)
{
    if (n == 0)
        return hipSuccess;
    if (dtype == 1)
        hipLaunchKernelGGL((scatter_kernel<double>), dim3(stream_grid(n)), dim3(kBlock), 0, stream,
                           (const double *)in, perm, (double *)out, n);
    else
        hipLaunchKernelGGL((scatter_kernel<float>), dim3(stream_grid(n)), dim3(kBlock), 0, stream,
                           (const float *)in, perm, (float *)out, n);
    return hipGetLastError();
}

hipError_t launch_gather_vals(int dtype, const void *in, const uint32_t *perm, void *out,
                              uint64_t n, hipStream_t stream)
{
    if (n == 0)
        return hipSuccess;
    if (dtype == 1)
        hipLaunchKernelGGL((gather_kernel<double>), dim3(stream_grid(n)), dim3(kBlock), 0, stream,
                           (const double *)in, perm, (double *)out, n);
    else
        hipLaunchKernelGGL((gather_kernel<float>), dim3(stream_grid(n)), dim3(kBlock), 0, stream,
                           (const float *)in, perm, (float *)out, n);
    return hipGetLastError();
}

namespace {
template <typename W>
hipError_t rows_typed(int op, void *panel, const RowMapView &M, uint32_t upr, void *buf,
                      hipStream_t st)
{
    if (op == 0) {
        const uint64_t total = (uint64_t)M.nslots * upr;
        hipLaunchKernelGGL((rows_pack_kernel<W>), dim3(stream_grid(total)), dim3(kBlock), 0, st,
                           (const W *)panel, M.rows, total, upr, (W *)buf);
    } else {
        const uint64_t total = (uint64_t)M.nuniq * upr;
        if (op == 1)
            hipLaunchKernelGGL((rows_unpack_kernel<W, false>), dim3(stream_grid(total)),
                               dim3(kBlock), 0, st, (W *)panel, M.urows, M.ptr, M.slots, total, upr,
                               (const W *)buf);
        else
            hipLaunchKernelGGL((rows_unpack_kernel<W, true>), dim3(stream_grid(total)),
                               dim3(kBlock), 0, st, (W *)panel, M.urows, M.ptr, M.slots, total, upr,
                               (const W *)buf);
    }
    return hipGetLastError();
}
} // namespace

hipError_t launch_rows(int op, int dtype, void *panel, const RowMapView &M, uint32_t K, void *buf,
                       hipStream_t stream)
{
    if (M.nslots == 0 || K == 0)
        return hipSuccess;
    const size_t row_bytes = (size_t)K * (dtype == 1 ? 8 : 4);
    if (row_bytes % 16 == 0) {
        const uint32_t upr = (uint32_t)(row_bytes / 16);
        return dtype == 1 ? rows_typed<Vec<double>::type>(op, panel, M, upr, buf, stream)
                          : rows_typed<Vec<float>::type>(op, panel, M, upr, buf, stream);
    }
    return dtype == 1 ? rows_typed<double>(op, panel, M, K, buf, stream)
                      : rows_typed<float>(op, panel, M, K, buf, stream);
}

hipError_t launch_xcc_probe(uint32_t *out, uint32_t nblocks, hipStream_t stream)
{
    if (nblocks == 0)
        return hipSuccess;
    hipLaunchKernelGGL(xcc_probe_kernel, dim3(nblocks), dim3(64), 0, stream, out);
    return hipGetLastError();
}

hipError_t launch_probe_cols(uint32_t *col, uint64_t n, uint32_t mode, uint32_t base,
                             uint32_t modulus, uint32_t ncols, hipStream_t stream)
{
    if (n == 0)
        return hipSuccess;
    hipLaunchKernelGGL(probe_cols_kernel, dim3(stream_grid(n)), dim3(kBlock), 0, stream, col, n,
                       mode, base, modulus, ncols);
    return hipGetLastError();
}

hipError_t launch_copy(void *dst, const void *src, uint64_t bytes, hipStream_t stream)
{
    if (bytes == 0)
        return hipSuccess;
    const uint64_t nvec = bytes / 16;
    hipLaunchKernelGGL(copy_kernel, dim3(stream_grid((nvec + 3) / 4 + 1)), dim3(kBlock), 0, stream,
                       (u32x4 *)dst, (const u32x4 *)src, nvec, (uint32_t)(bytes % 16));
    return hipGetLastError();
}

hipError_t launch_fill(int dtype, void *p, uint64_t n, double value, hipStream_t stream)
{
    if (n == 0)
        return hipSuccess;
    if (dtype == 1)
        hipLaunchKernelGGL((fill_kernel<double>), dim3(stream_grid(n)), dim3(kBlock), 0, stream,
                           (double *)p, n, value);
    else
        hipLaunchKernelGGL((fill_kernel<float>), dim3(stream_grid(n)), dim3(kBlock), 0, stream,
                           (float *)p, n, (float)value);
    return hipGetLastError();
}

const char *kernel_variant(int dtype, uint32_t K)
{
    static thread_local char buf[64];
    const Shape sh = pick_shape(dtype == 1 ? 8 : 4, K);
    if (K == 0)
        snprintf(buf, sizeof buf, "none (no columns)");
    else if (sh.lpr == 0)
        snprintf(buf, sizeof buf, "seg<%s,LPR=64,VPL=4,odd> per 4 KiB slice",
                 dtype == 1 ? "f64" : "f32");
    else
        snprintf(buf, sizeof buf, "seg<%s,LPR=%d,VPL=%d%s>", dtype == 1 ? "f64" : "f32", sh.lpr,
                 sh.vpl, sh.mode == 1 ? ",ragged" : (sh.mode == 2 ? ",odd" : (sh.mode == 3 ? ",thin" : "")));
    return buf;
}

} // namespace spc3d
