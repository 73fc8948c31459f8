// gfx950 (CDNA4, wave64) kernels for the local SDDMM and SpMM.
//
//   sddmm: C[e] = S.vv[e] * <A[ii[e],:], B[jj[e],:]>      (reference: src/core_ops.cpp:5-22)
//   spmm : Y[ii[e],:] += A.vv[e] * X[jj[e],:]             (reference: src/core_ops.cpp:24-35)
//
// Both are gather-bound (about 0.25 flop per byte): no MFMA.  The unit of work
// is a row segment (plan_host.h): at most seg_max consecutive entries of one
// row.  A dense row of K reals is covered by LPR lanes holding VPL 16-byte
// vectors each (K * sizeof(T) = LPR * VPL * 16), so one wavefront works on
// 64 / LPR segments at once and every global load instruction moves
// 64 x 16 B.  Segments arrive sorted longest first, so the lane groups of a
// wavefront run the same trip count.
//
//   sddmm: the group keeps its A row slice in registers, gathers B row slices
//          for UB entries at a time, and reduces the UB per-lane partial dot
//          products across the group with a halving exchange (UB-1 shuffles
//          for UB entries instead of UB*log2(LPR)), leaving entry u's dot
//          product in lane u*(LPR/UB); that lane scales by S.vv and stores to
//          the caller's position.
//   spmm : lane = slice of K, no cross-lane reduction; the group accumulates
//          a * X[c,:] in registers and does one read-modify-write of the Y
//          row slice.  Rows cut into several segments write partial sums that
//          spmm_fixup adds into Y in a fixed order (no atomics, results are
//          reproducible run to run).
#include <hip/hip_runtime.h>

#include "kernels.h"

namespace spc3d {
namespace {

template <typename T> struct Vec;
template <> struct Vec<float> {
    typedef float type __attribute__((ext_vector_type(4)));
    static constexpr int N = 4;
};
template <> struct Vec<double> {
    typedef double type __attribute__((ext_vector_type(2)));
    static constexpr int N = 2;
};

template <typename T>
__device__ __forceinline__ T vdot(const typename Vec<T>::type &a, const typename Vec<T>::type &b,
                                  T acc)
{
#pragma unroll
    for (int i = 0; i < Vec<T>::N; ++i)
        acc += a[i] * b[i];
    return acc;
}

constexpr int kBlock = 256; // 4 wavefronts

// ---------------------------------------------------------------- SDDMM ----
template <typename T, int LPR, int VPL, int UB, bool TAIL>
__device__ __forceinline__ void
sddmm_batch(const typename Vec<T>::type (&a)[VPL], const uint32_t *__restrict__ col,
            const uint32_t *__restrict__ perm, const T *__restrict__ sval,
            const T *__restrict__ B, T *__restrict__ C, uint32_t K, uint32_t p0, uint32_t nb,
            uint32_t sub)
{
    using V = typename Vec<T>::type;
    constexpr int RED = LPR / UB;
    const uint32_t ul = sub & (UB - 1);
    const uint32_t uo = sub / RED;

    // Indices and the output lane's operands first: they head the dependency chain.
    const uint32_t cme = col[p0 + (TAIL ? (ul < nb ? ul : nb - 1) : ul)];
    T sv = (T)0;
    uint32_t dst = 0;
    const bool writer = (sub % RED) == 0 && (!TAIL || uo < nb);
    if (writer) {
        sv = sval[p0 + uo];
        dst = perm ? perm[p0 + uo] : p0 + uo;
    }

    V b[UB][VPL];
#pragma unroll
    for (int u = 0; u < UB; ++u) {
        const uint32_t c = __shfl(cme, u, LPR);
        const V *brow = reinterpret_cast<const V *>(B + (size_t)c * K);
        if (!TAIL || (uint32_t)u < nb) {
#pragma unroll
            for (int v = 0; v < VPL; ++v)
                b[u][v] = brow[sub + v * LPR];
        } else {
#pragma unroll
            for (int v = 0; v < VPL; ++v)
                b[u][v] = V{};
        }
    }
    T part[UB];
#pragma unroll
    for (int u = 0; u < UB; ++u) {
        T acc = (T)0;
#pragma unroll
        for (int v = 0; v < VPL; ++v)
            acc = vdot<T>(a[v], b[u][v], acc);
        part[u] = acc;
    }
    // Halving exchange: after the step with stride s a lane keeps the half of
    // its values selected by (sub & s); UB values shrink to 1 in log2(UB) steps
    // and lane `sub` ends with the sum, over its RED-aligned partners so far
    // excluded, of entry sub / RED.
#pragma unroll
    for (int s = LPR / 2, n = UB; n > 1; s >>= 1, n >>= 1) {
        const bool upper = (sub & s) != 0;
#pragma unroll
        for (int i = 0; i < n / 2; ++i) {
            const T keep = upper ? part[i + n / 2] : part[i];
            const T send = upper ? part[i] : part[i + n / 2];
            part[i] = keep + __shfl_xor(send, s, LPR);
        }
    }
#pragma unroll
    for (int s = RED / 2; s >= 1; s >>= 1)
        part[0] += __shfl_xor(part[0], s, LPR);

    if (writer)
        C[dst] = part[0] * sv;
}

template <typename T, int LPR, int VPL, int UB>
__global__ void __launch_bounds__(kBlock)
sddmm_seg_kernel(const Seg *__restrict__ segs, uint32_t nseg, const uint32_t *__restrict__ col,
                 const uint32_t *__restrict__ perm, const T *__restrict__ sval,
                 const T *__restrict__ A, const T *__restrict__ B, T *__restrict__ C, uint32_t K)
{
    static_assert(UB <= LPR && LPR <= 64, "batch must fit the lane group");
    using V = typename Vec<T>::type;
    constexpr int G = 64 / LPR;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t sub = lane & (LPR - 1);
    const uint64_t wave = (uint64_t)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
    const uint64_t sid = wave * G + lane / LPR;
    if (sid >= nseg)
        return;
    const Seg sg = segs[sid];

    V a[VPL];
    {
        const V *arow = reinterpret_cast<const V *>(A + (size_t)sg.row * K);
#pragma unroll
        for (int v = 0; v < VPL; ++v)
            a[v] = arow[sub + v * LPR];
    }
    uint32_t base = 0;
    for (; base + UB <= sg.len; base += UB)
        sddmm_batch<T, LPR, VPL, UB, false>(a, col, perm, sval, B, C, K, sg.start + base, UB, sub);
    if (base < sg.len)
        sddmm_batch<T, LPR, VPL, UB, true>(a, col, perm, sval, B, C, K, sg.start + base,
                                           sg.len - base, sub);
}

// Any K: one wavefront per segment, lanes stride over K, scalar loads.
template <typename T>
__global__ void __launch_bounds__(kBlock)
sddmm_generic_kernel(const Seg *__restrict__ segs, uint32_t nseg, const uint32_t *__restrict__ col,
                     const uint32_t *__restrict__ perm, const T *__restrict__ sval,
                     const T *__restrict__ A, const T *__restrict__ B, T *__restrict__ C,
                     uint32_t K)
{
    const uint32_t lane = threadIdx.x & 63u;
    const uint64_t sid = (uint64_t)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
    if (sid >= nseg)
        return;
    const Seg sg = segs[sid];
    const T *arow = A + (size_t)sg.row * K;
    for (uint32_t i = 0; i < sg.len; ++i) {
        const uint32_t p = sg.start + i;
        const T *brow = B + (size_t)col[p] * K;
        T acc = (T)0;
        for (uint32_t j = lane; j < K; j += 64)
            acc += arow[j] * brow[j];
#pragma unroll
        for (int s = 32; s >= 1; s >>= 1)
            acc += __shfl_xor(acc, s, 64);
        if (lane == 0)
            C[perm ? perm[p] : p] = acc * sval[p];
    }
}

// ----------------------------------------------------------------- SpMM ----
template <typename T, int LPR, int VPL, int UB, bool TAIL>
__device__ __forceinline__ void
spmm_batch(typename Vec<T>::type (&acc)[VPL], const uint32_t *__restrict__ col,
           const T *__restrict__ sval, const T *__restrict__ X, uint32_t K, uint32_t p0,
           uint32_t nb, uint32_t sub)
{
    using V = typename Vec<T>::type;
    const uint32_t ul = sub & (UB - 1);
    const uint32_t pl = p0 + (TAIL ? (ul < nb ? ul : nb - 1) : ul);
    const uint32_t cme = col[pl];
    const T vme = sval[pl];

    V x[UB][VPL];
    T av[UB];
#pragma unroll
    for (int u = 0; u < UB; ++u) {
        const uint32_t c = __shfl(cme, u, LPR);
        av[u] = __shfl(vme, u, LPR);
        const V *xrow = reinterpret_cast<const V *>(X + (size_t)c * K);
        if (!TAIL || (uint32_t)u < nb) {
#pragma unroll
            for (int v = 0; v < VPL; ++v)
                x[u][v] = xrow[sub + v * LPR];
        } else {
            av[u] = (T)0;
#pragma unroll
            for (int v = 0; v < VPL; ++v)
                x[u][v] = V{};
        }
    }
    // Entries are added in kernel order, which within a row is the caller's order.
#pragma unroll
    for (int u = 0; u < UB; ++u)
#pragma unroll
        for (int v = 0; v < VPL; ++v)
            acc[v] += x[u][v] * av[u];
}

template <typename T, int LPR, int VPL, int UB>
__global__ void __launch_bounds__(kBlock)
spmm_seg_kernel(const Seg *__restrict__ segs, uint32_t nseg, const uint32_t *__restrict__ col,
                const T *__restrict__ sval, const T *__restrict__ X, T *__restrict__ Y,
                T *__restrict__ partial, uint32_t K)
{
    static_assert(UB <= LPR && LPR <= 64, "batch must fit the lane group");
    using V = typename Vec<T>::type;
    constexpr int G = 64 / LPR;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t sub = lane & (LPR - 1);
    const uint64_t wave = (uint64_t)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
    const uint64_t sid = wave * G + lane / LPR;
    if (sid >= nseg)
        return;
    const Seg sg = segs[sid];
    const bool whole = sg.slot == kWholeRow;
    V *dst = reinterpret_cast<V *>(whole ? Y + (size_t)sg.row * K : partial + (size_t)sg.slot * K);

    V acc[VPL], y0[VPL];
#pragma unroll
    for (int v = 0; v < VPL; ++v) {
        acc[v] = V{};
        y0[v] = V{};
    }
    if (whole) {
#pragma unroll
        for (int v = 0; v < VPL; ++v)
            y0[v] = dst[sub + v * LPR];
    }
    uint32_t base = 0;
    for (; base + UB <= sg.len; base += UB)
        spmm_batch<T, LPR, VPL, UB, false>(acc, col, sval, X, K, sg.start + base, UB, sub);
    if (base < sg.len)
        spmm_batch<T, LPR, VPL, UB, true>(acc, col, sval, X, K, sg.start + base, sg.len - base,
                                          sub);
#pragma unroll
    for (int v = 0; v < VPL; ++v)
        dst[sub + v * LPR] = y0[v] + acc[v];
}

template <typename T>
__global__ void __launch_bounds__(kBlock)
spmm_generic_kernel(const Seg *__restrict__ segs, uint32_t nseg, const uint32_t *__restrict__ col,
                    const T *__restrict__ sval, const T *__restrict__ X, T *__restrict__ Y,
                    T *__restrict__ partial, uint32_t K)
{
    const uint32_t lane = threadIdx.x & 63u;
    const uint64_t sid = (uint64_t)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
    if (sid >= nseg)
        return;
    const Seg sg = segs[sid];
    const bool whole = sg.slot == kWholeRow;
    T *dst = whole ? Y + (size_t)sg.row * K : partial + (size_t)sg.slot * K;
    for (uint32_t j = lane; j < K; j += 64) {
        T acc = (T)0;
        for (uint32_t i = 0; i < sg.len; ++i) {
            const uint32_t p = sg.start + i;
            acc += sval[p] * X[(size_t)col[p] * K + j];
        }
        dst[j] = whole ? dst[j] + acc : acc;
    }
}

// One block per cut row: Y[row,:] += partial sums in slot order.
template <typename T>
__global__ void __launch_bounds__(kBlock)
spmm_fixup_kernel(const SplitRow *__restrict__ splits, const T *__restrict__ partial,
                  T *__restrict__ Y, uint32_t K)
{
    const SplitRow sr = splits[blockIdx.x];
    for (uint32_t j = threadIdx.x; j < K; j += kBlock) {
        T s = (T)0;
        for (uint32_t q = 0; q < sr.nslots; ++q)
            s += partial[(size_t)(sr.first_slot + q) * K + j];
        Y[(size_t)sr.row * K + j] += s;
    }
}

// ------------------------------------------------------------- utilities ----
template <typename T>
__global__ void __launch_bounds__(kBlock)
gather_kernel(const T *__restrict__ in, const uint32_t *__restrict__ perm, T *__restrict__ out,
              uint64_t n)
{
    const uint64_t stride = (uint64_t)gridDim.x * kBlock;
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride)
        out[i] = perm ? in[perm[i]] : in[i];
}

template <typename T>
__global__ void __launch_bounds__(kBlock) fill_kernel(T *__restrict__ p, uint64_t n, T value)
{
    const uint64_t stride = (uint64_t)gridDim.x * kBlock;
    for (uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride)
        p[i] = value;
}

// ------------------------------------------------------------- dispatch ----
struct Shape {
    int lpr, vpl, ub; // lpr == 0: generic kernel
};

// K * sizeof(T) must be LPR * VPL * 16 bytes with LPR a power of two in
// [4, 64] and VPL in {1, 2, 4}; anything else takes the generic kernels.
Shape pick_shape(size_t elem, uint32_t K)
{
    const size_t bytes = (size_t)K * elem;
    if (K == 0 || bytes % 16)
        return {0, 0, 0};
    const size_t nvec = bytes / 16;
    for (int lpr = 64; lpr >= 4; lpr >>= 1) {
        if (nvec % lpr)
            continue;
        const size_t vpl = nvec / lpr;
        if (vpl == 1)
            return {lpr, 1, lpr < 16 ? lpr : 16};
        if (vpl == 2)
            return {lpr, 2, lpr < 8 ? lpr : 8};
        if (vpl == 4)
            return {lpr, 4, 4};
        return {0, 0, 0};
    }
    return {0, 0, 0};
}

inline uint32_t blocks_for_groups(uint32_t nseg, int groups_per_wave)
{
    const uint64_t waves = ((uint64_t)nseg + groups_per_wave - 1) / groups_per_wave;
    return (uint32_t)((waves + kBlock / 64 - 1) / (kBlock / 64));
}

template <typename T, int LPR, int VPL, int UB>
void run_sddmm(const DevPlanView &P, const T *A, const T *B, T *C, uint32_t K, hipStream_t st)
{
    const uint32_t grid = blocks_for_groups(P.nseg, 64 / LPR);
    hipLaunchKernelGGL((sddmm_seg_kernel<T, LPR, VPL, UB>), dim3(grid), dim3(kBlock), 0, st, P.segs,
                       P.nseg, P.col, P.perm, (const T *)P.sval, A, B, C, K);
}

template <typename T, int LPR, int VPL, int UB>
void run_spmm(const DevPlanView &P, const T *X, T *Y, uint32_t K, hipStream_t st)
{
    const uint32_t grid = blocks_for_groups(P.nseg, 64 / LPR);
    hipLaunchKernelGGL((spmm_seg_kernel<T, LPR, VPL, UB>), dim3(grid), dim3(kBlock), 0, st, P.segs,
                       P.nseg, P.col, (const T *)P.sval, X, Y, (T *)P.partial, K);
}

#define SPC3D_FOR_SHAPES(X)                                                                       \
    X(4, 1, 4) X(8, 1, 8) X(16, 1, 16) X(32, 1, 16) X(64, 1, 16)                                  \
    X(4, 2, 4) X(8, 2, 8) X(16, 2, 8) X(32, 2, 8) X(64, 2, 8)                                     \
    X(4, 4, 4) X(8, 4, 4) X(16, 4, 4) X(32, 4, 4) X(64, 4, 4)

template <typename T>
hipError_t sddmm_typed(const DevPlanView &P, const void *A, const void *B, void *C, uint32_t K,
                       hipStream_t st)
{
    if (P.nseg == 0)
        return hipSuccess;
    const Shape sh = pick_shape(sizeof(T), K);
    bool done = false;
#define X(L, V, U)                                                                                \
    if (!done && sh.lpr == L && sh.vpl == V) {                                                    \
        run_sddmm<T, L, V, U>(P, (const T *)A, (const T *)B, (T *)C, K, st);                      \
        done = true;                                                                              \
    }
    SPC3D_FOR_SHAPES(X)
#undef X
    if (!done) {
        const uint32_t grid = blocks_for_groups(P.nseg, 1);
        hipLaunchKernelGGL((sddmm_generic_kernel<T>), dim3(grid), dim3(kBlock), 0, st, P.segs,
                           P.nseg, P.col, P.perm, (const T *)P.sval, (const T *)A, (const T *)B,
                           (T *)C, K);
    }
    return hipGetLastError();
}

template <typename T>
hipError_t spmm_typed(const DevPlanView &P, const void *X_, void *Y, uint32_t K, hipStream_t st)
{
    if (P.nseg == 0)
        return hipSuccess;
    const Shape sh = pick_shape(sizeof(T), K);
    bool done = false;
#define X(L, V, U)                                                                                \
    if (!done && sh.lpr == L && sh.vpl == V) {                                                    \
        run_spmm<T, L, V, U>(P, (const T *)X_, (T *)Y, K, st);                                    \
        done = true;                                                                              \
    }
    SPC3D_FOR_SHAPES(X)
#undef X
    if (!done) {
        const uint32_t grid = blocks_for_groups(P.nseg, 1);
        hipLaunchKernelGGL((spmm_generic_kernel<T>), dim3(grid), dim3(kBlock), 0, st, P.segs,
                           P.nseg, P.col, (const T *)P.sval, (const T *)X_, (T *)Y,
                           (T *)P.partial, K);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess)
        return e;
    if (P.nsplit) {
        hipLaunchKernelGGL((spmm_fixup_kernel<T>), dim3(P.nsplit), dim3(kBlock), 0, st, P.splits,
                           (const T *)P.partial, (T *)Y, K);
        e = hipGetLastError();
    }
    return e;
}

inline uint32_t stream_grid(uint64_t n)
{
    const uint64_t want = (n + kBlock - 1) / kBlock;
    const uint64_t cap = 256 * 32; // 32 blocks per CU keeps a grid-stride loop busy
    return (uint32_t)(want < 1 ? 1 : (want > cap ? cap : want));
}

} // namespace

hipError_t launch_sddmm(int dtype, const DevPlanView &P, const void *A, const void *B, void *C,
                        uint32_t K, hipStream_t stream)
{
    return dtype == 1 ? sddmm_typed<double>(P, A, B, C, K, stream)
                      : sddmm_typed<float>(P, A, B, C, K, stream);
}

hipError_t launch_spmm(int dtype, const DevPlanView &P, const void *X, void *Y, uint32_t K,
                       hipStream_t stream)
{
    return dtype == 1 ? spmm_typed<double>(P, X, Y, K, stream)
                      : spmm_typed<float>(P, X, Y, K, stream);
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
    if (sh.lpr == 0)
        snprintf(buf, sizeof buf, "generic<%s>", dtype == 1 ? "f64" : "f32");
    else
        snprintf(buf, sizeof buf, "seg<%s,LPR=%d,VPL=%d,UB=%d>", dtype == 1 ? "f64" : "f32",
                 sh.lpr, sh.vpl, sh.ub);
    return buf;
}

} // namespace spc3d
