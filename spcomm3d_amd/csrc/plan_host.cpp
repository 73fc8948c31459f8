// Host-side plan construction: validation, row grouping, segmentation.
#include "plan_host.h"

#include <algorithm>
#include <cstdio>

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

int build_host_plan(uint32_t nrows, uint32_t ncols, uint64_t nnz, const uint32_t *ii,
                    const uint32_t *jj, uint32_t seg_max, HostPlan &out, std::string &err)
{
    int rc = validate_coo(nrows, ncols, nnz, ii, jj, err);
    if (rc != SPC3D_OK)
        return rc;
    if (seg_max == 0)
        seg_max = kDefaultSegMax;

    HostPlan P;
    P.nrows = nrows;
    P.ncols = ncols;
    P.nnz = nnz;
    P.seg_max = seg_max;
    try {
        // Row histogram -> exclusive prefix.
        std::vector<uint32_t> rowptr((size_t)nrows + 1, 0);
        for (uint64_t e = 0; e < nnz; ++e)
            ++rowptr[(size_t)ii[e] + 1];
        uint32_t touched = 0, maxlen = 0;
        for (uint32_t r = 0; r < nrows; ++r) {
            const uint32_t len = rowptr[(size_t)r + 1];
            touched += len != 0;
            maxlen = std::max(maxlen, len);
            rowptr[(size_t)r + 1] += rowptr[r];
        }
        P.rows_touched = touched;
        P.max_row_nnz = maxlen;

        // Stable scatter into row groups.
        P.col.resize(nnz);
        P.perm.resize(nnz);
        {
            std::vector<uint32_t> cursor(rowptr.begin(), rowptr.end() - 1);
            std::vector<uint8_t> seen((size_t)ncols, 0);
            uint32_t notid = 0;
            for (uint64_t e = 0; e < nnz; ++e) {
                const uint32_t p = cursor[ii[e]]++;
                P.perm[p] = (uint32_t)e;
                P.col[p] = jj[e];
                notid |= (uint32_t)(p != (uint32_t)e);
                seen[jj[e]] = 1;
            }
            P.identity = notid == 0;
            uint32_t ct = 0;
            for (uint32_t c = 0; c < ncols; ++c)
                ct += seen[c];
            P.cols_touched = ct;
        }

        // Segments in row order.
        std::vector<Seg> segs;
        segs.reserve((size_t)touched + nnz / seg_max + 1);
        uint32_t nslots = 0;
        for (uint32_t r = 0; r < nrows; ++r) {
            const uint32_t s = rowptr[r], len = rowptr[(size_t)r + 1] - s;
            if (len == 0)
                continue;
            if (len <= seg_max) {
                segs.push_back(Seg{r, s, len, kWholeRow});
                continue;
            }
            const uint32_t parts = (len + seg_max - 1) / seg_max;
            const uint32_t base = len / parts, rem = len % parts;
            P.splits.push_back(SplitRow{r, nslots, parts, 0});
            uint32_t at = s;
            for (uint32_t q = 0; q < parts; ++q) {
                const uint32_t l = base + (q < rem ? 1u : 0u);
                segs.push_back(Seg{r, at, l, nslots++});
                at += l;
            }
        }
        P.nslots = nslots;

        // Longest first (lane groups of one wavefront then run the same trip
        // count); equal lengths keep row order (neighbouring rows of banded
        // patterns share dense rows).  Counting sort on len in [1, seg_max].
        std::vector<uint32_t> bucket((size_t)seg_max + 2, 0);
        for (const Seg &g : segs)
            ++bucket[seg_max - g.len + 1];
        for (uint32_t i = 0; i <= seg_max; ++i)
            bucket[i + 1] += bucket[i];
        P.segs.resize(segs.size());
        for (const Seg &g : segs)
            P.segs[bucket[seg_max - g.len]++] = g;
    } catch (const std::bad_alloc &) {
        err = "host allocation failed while building the plan";
        return SPC3D_ERR_ALLOC;
    }
    out = std::move(P);
    return SPC3D_OK;
}

} // namespace spc3d
