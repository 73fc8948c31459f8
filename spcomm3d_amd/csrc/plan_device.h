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

} // namespace spc3d
