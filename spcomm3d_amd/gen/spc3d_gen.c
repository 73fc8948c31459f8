/*
 * Seeded, counter-based generators for the synthetic workloads the local
 * SDDMM / SpMM kernels are tested and timed on.  Host code, plain C + OpenMP.
 *
 * Every value is a pure function of (seed, stream, index), so the same arrays
 * come out on any machine, with any thread count, for the CPU checker and the
 * GPU path alike.  The reference ships no usable generator (its only one,
 * COOMatrix::self_generate_random, seeds from the clock:
 * src/SparseMatrix.hpp:49-67) and no input matrices.
 *
 * Bit generator: SplitMix64 (Steele, Lea, Flood 2014).  draw(key, i) is the
 * i-th output of a SplitMix64 stream whose initial state is key;
 * key = mix(mix(seed) ^ stream-constant) separates streams.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define GEN_API __attribute__((visibility("default")))
#define GOLDEN 0x9E3779B97F4A7C15ULL

static inline uint64_t mix64(uint64_t z)
{
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    return z ^ (z >> 31);
}

/* i-th output (i = 0,1,...) of SplitMix64 started from state `key`. */
static inline uint64_t draw(uint64_t key, uint64_t i)
{
    return mix64(key + (i + 1) * GOLDEN);
}

static inline uint64_t stream_key(uint64_t seed, uint64_t stream)
{
    return mix64(mix64(seed + GOLDEN) ^ (stream * 0xD1342543DE82EF95ULL + 1));
}

static inline double to_unit(uint64_t x) /* [0,1) with 53 bits */
{
    return (double)(x >> 11) * (1.0 / 9007199254740992.0);
}

/* Exposed so the tests can pin the bit generator against published vectors. */
GEN_API uint64_t spc3d_gen_splitmix64(uint64_t state0, uint64_t i)
{
    return draw(state0, i);
}

GEN_API uint64_t spc3d_gen_stream_key(uint64_t seed, uint64_t stream)
{
    return stream_key(seed, stream);
}

/* out[i] = lo + (hi-lo) * u(seed, stream, first+i); dtype 0 = f32, 1 = f64.
 * The f32 value is the f64 value rounded once. */
GEN_API int spc3d_gen_uniform(uint64_t seed, uint64_t stream, uint64_t first,
                              uint64_t count, double lo, double hi, int dtype,
                              void *out)
{
    const uint64_t key = stream_key(seed, stream);
    const double w = hi - lo;
    if (dtype == 1) {
        double *o = (double *)out;
#pragma omp parallel for schedule(static)
        for (uint64_t i = 0; i < count; ++i)
            o[i] = lo + w * to_unit(draw(key, first + i));
    } else if (dtype == 0) {
        float *o = (float *)out;
#pragma omp parallel for schedule(static)
        for (uint64_t i = 0; i < count; ++i)
            o[i] = (float)(lo + w * to_unit(draw(key, first + i)));
    } else {
        return -1;
    }
    return 0;
}

/* keys[i] = draw(stream_key(seed,stream), i): sort keys to get a permutation. */
GEN_API int spc3d_gen_keys(uint64_t seed, uint64_t stream, uint64_t count,
                           uint64_t *keys)
{
    const uint64_t key = stream_key(seed, stream);
#pragma omp parallel for schedule(static)
    for (uint64_t i = 0; i < count; ++i)
        keys[i] = draw(key, i);
    return 0;
}

/*
 * R-MAT edge e (Chakrabarti, Zhan, Faloutsos 2004): `scale` quadrant choices
 * with probabilities (a, b, c, 1-a-b-c) = (top-left, top-right, bottom-left,
 * bottom-right); the most significant bit is chosen first.  Two levels are
 * taken from each 64-bit draw (one 32-bit half per level).
 */
static inline void rmat_edge(uint64_t key, uint64_t e, int scale, uint32_t ta,
                             uint32_t tab, uint32_t tabc, uint32_t *row,
                             uint32_t *col)
{
    uint32_t r = 0, c = 0;
    const uint64_t draws_per_edge = (uint64_t)(scale + 1) / 2;
    uint64_t bits = 0;
    for (int l = 0; l < scale; ++l) {
        uint32_t u;
        if ((l & 1) == 0) {
            bits = draw(key, e * draws_per_edge + (uint64_t)(l >> 1));
            u = (uint32_t)(bits >> 32);
        } else {
            u = (uint32_t)bits;
        }
        uint32_t rb, cb;
        if (u < ta) {
            rb = 0; cb = 0;
        } else if (u < tab) {
            rb = 0; cb = 1;
        } else if (u < tabc) {
            rb = 1; cb = 0;
        } else {
            rb = 1; cb = 1;
        }
        r = (r << 1) | rb;
        c = (c << 1) | cb;
    }
    *row = r;
    *col = c;
}

static inline void rmat_thresholds(double a, double b, double c, uint32_t *ta,
                                   uint32_t *tab, uint32_t *tabc)
{
    const double two32 = 4294967296.0;
    *ta = (uint32_t)(a * two32);
    *tab = (uint32_t)((a + b) * two32);
    *tabc = (uint32_t)((a + b + c) * two32);
}

/* All `nedges` raw edges (duplicates included), edge e at position e. */
GEN_API int spc3d_gen_rmat_edges(uint64_t seed, int scale, uint64_t nedges,
                                 double a, double b, double c, uint32_t *rows,
                                 uint32_t *cols)
{
    if (scale < 1 || scale > 31)
        return -1;
    const uint64_t key = stream_key(seed, 0);
    uint32_t ta, tab, tabc;
    rmat_thresholds(a, b, c, &ta, &tab, &tabc);
#pragma omp parallel for schedule(static)
    for (uint64_t e = 0; e < nedges; ++e)
        rmat_edge(key, e, scale, ta, tab, tabc, &rows[e], &cols[e]);
    return 0;
}

/*
 * One block of a 2D partition of an R-MAT graph, following the reference's
 * rule (src/parallel_io.hpp:64-76): rows are randomly permuted and dealt
 * round-robin to `px` row groups (group = position % px), columns likewise to
 * `py` groups.  pos_r[v] / pos_c[v] give the position of global row / column v
 * in those permutations.  Keeps the edges whose (row group, col group) is
 * (gx, gy), renumbered to block-local ids position / px and position / py, in
 * edge order.  Call with rows == NULL to count; returns the number kept, or -1.
 */
GEN_API int64_t spc3d_gen_rmat_block(uint64_t seed, int scale, uint64_t nedges,
                                     double a, double b, double c,
                                     const uint32_t *pos_r,
                                     const uint32_t *pos_c, uint32_t px,
                                     uint32_t py, uint32_t gx, uint32_t gy,
                                     uint32_t *rows, uint32_t *cols,
                                     uint64_t capacity)
{
    if (scale < 1 || scale > 31 || px == 0 || py == 0)
        return -1;
    const uint64_t key = stream_key(seed, 0);
    uint32_t ta, tab, tabc;
    rmat_thresholds(a, b, c, &ta, &tab, &tabc);
    enum { NCHUNK = 1024 };
    uint64_t *cnt = (uint64_t *)calloc(NCHUNK + 1, sizeof(uint64_t));
    if (!cnt)
        return -1;
    const uint64_t per = (nedges + NCHUNK - 1) / NCHUNK;
#pragma omp parallel for schedule(dynamic, 4)
    for (int ch = 0; ch < NCHUNK; ++ch) {
        uint64_t lo = (uint64_t)ch * per, hi = lo + per;
        if (hi > nedges)
            hi = nedges;
        uint64_t n = 0;
        for (uint64_t e = lo; e < hi; ++e) {
            uint32_t r, cc;
            rmat_edge(key, e, scale, ta, tab, tabc, &r, &cc);
            if (pos_r[r] % px == gx && pos_c[cc] % py == gy)
                ++n;
        }
        cnt[ch + 1] = n;
    }
    for (int ch = 0; ch < NCHUNK; ++ch)
        cnt[ch + 1] += cnt[ch];
    const uint64_t total = cnt[NCHUNK];
    if (rows == NULL || cols == NULL) {
        free(cnt);
        return (int64_t)total;
    }
    if (total > capacity) {
        free(cnt);
        return -1;
    }
#pragma omp parallel for schedule(dynamic, 4)
    for (int ch = 0; ch < NCHUNK; ++ch) {
        uint64_t lo = (uint64_t)ch * per, hi = lo + per;
        if (hi > nedges)
            hi = nedges;
        uint64_t w = cnt[ch];
        for (uint64_t e = lo; e < hi; ++e) {
            uint32_t r, cc;
            rmat_edge(key, e, scale, ta, tab, tabc, &r, &cc);
            if (pos_r[r] % px == gx && pos_c[cc] % py == gy) {
                rows[w] = pos_r[r] / px;
                cols[w] = pos_c[cc] / py;
                ++w;
            }
        }
    }
    free(cnt);
    return (int64_t)total;
}

/*
 * deg[i] = min(Z, cap) with Z ~ Zipf(s) on {1,2,...} (P(k) = k^-s / zeta(s)),
 * by inverse CDF: the mass above cap-1 all lands on cap.
 */
GEN_API int spc3d_gen_zipf_capped(uint64_t seed, uint64_t stream, uint64_t count,
                                  double s, uint32_t cap, uint32_t *deg)
{
    if (cap < 1 || s <= 1.0)
        return -1;
    /* zeta(s) = sum_{k<N} k^-s + Euler-Maclaurin tail from N */
    const int N = 100000;
    double z = 0.0;
    for (int k = N - 1; k >= 1; --k)
        z += pow((double)k, -s);
    const double Nd = (double)N;
    z += pow(Nd, 1.0 - s) / (s - 1.0) + 0.5 * pow(Nd, -s) +
         s * pow(Nd, -s - 1.0) / 12.0;
    double *cdf = (double *)malloc(sizeof(double) * cap);
    if (!cdf)
        return -1;
    double acc = 0.0;
    for (uint32_t k = 1; k < cap; ++k) {
        acc += pow((double)k, -s) / z;
        cdf[k] = acc; /* P(Z <= k) */
    }
    const uint64_t key = stream_key(seed, stream);
#pragma omp parallel for schedule(static)
    for (uint64_t i = 0; i < count; ++i) {
        const double u = to_unit(draw(key, i));
        /* smallest k in [1,cap) with u < cdf[k], else cap */
        uint32_t lo = 1, hi = cap;
        while (lo < hi) {
            uint32_t mid = lo + (hi - lo) / 2;
            if (u < cdf[mid])
                hi = mid;
            else
                lo = mid + 1;
        }
        deg[i] = lo;
    }
    free(cdf);
    return 0;
}

/*
 * For each row i, deg_i distinct columns uniform in [0, ncols), written in
 * draw order to cols[rowptr[i] .. rowptr[i+1]).  Row i draws from its own
 * stream (seed, i); a candidate already taken by the row is skipped.
 * deg_i must not exceed ncols or 4096.
 */
GEN_API int spc3d_gen_distinct_cols(uint64_t seed, uint64_t nrows, uint32_t ncols,
                                    const uint64_t *rowptr, uint32_t *cols)
{
    int bad = 0;
#pragma omp parallel for schedule(dynamic, 1024)
    for (uint64_t i = 0; i < nrows; ++i) {
        const uint64_t d = rowptr[i + 1] - rowptr[i];
        if (d > ncols || d > 4096) {
            bad = 1;
            continue;
        }
        uint32_t tab[16384];
        uint32_t mask = 15;
        while (mask + 1 < 4 * d)
            mask = mask * 2 + 1;
        memset(tab, 0xFF, (size_t)(mask + 1) * sizeof(uint32_t));
        const uint64_t key = stream_key(seed, i);
        uint32_t *out = cols + rowptr[i];
        uint64_t got = 0, t = 0;
        while (got < d) {
            /* unbiased enough for ncols << 2^64: multiply-shift of 64 bits */
            const uint64_t x = draw(key, t++);
            const uint32_t c =
                (uint32_t)(((unsigned __int128)x * (unsigned __int128)ncols) >> 64);
            uint32_t h = (uint32_t)(c * 2654435761u) & mask;
            int dup = 0;
            while (tab[h] != 0xFFFFFFFFu) {
                if (tab[h] == c) {
                    dup = 1;
                    break;
                }
                h = (h + 1) & mask;
            }
            if (dup)
                continue;
            tab[h] = c;
            out[got++] = c;
        }
    }
    return bad ? -1 : 0;
}
