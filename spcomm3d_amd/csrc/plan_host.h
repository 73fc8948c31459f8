// Host-side construction of the kernel-order form of a COO pattern.
// Pure C++ (no HIP): testable and usable without a GPU.
#pragma once
#include <cstdint>
#include <string>
#include <vector>

namespace spc3d {

// One unit of work for a lane group: `len` consecutive entries of one row in
// kernel order.  slot == kWholeRow: the segment is the whole row (SpMM adds
// its sum straight into Y); otherwise the row was cut and the segment's sum
// goes to partial-sum row `slot`.
struct Seg {
    uint32_t row;
    uint32_t start;
    uint32_t len;
    uint32_t slot;
};
constexpr uint32_t kWholeRow = 0xFFFFFFFFu;

// A row cut into several segments: its partial sums are slots
// [first_slot, first_slot + nslots).
struct SplitRow {
    uint32_t row;
    uint32_t first_slot;
    uint32_t nslots;
    uint32_t pad;
};

struct HostPlan {
    uint32_t nrows = 0, ncols = 0;
    uint64_t nnz = 0;
    uint32_t rows_touched = 0, cols_touched = 0;
    uint32_t max_row_nnz = 0;
    uint32_t seg_max = 0;
    uint32_t nslots = 0;
    bool identity = true;          // perm[p] == p for all p
    std::vector<uint32_t> col;     // [nnz] column of kernel-order entry p
    std::vector<uint32_t> perm;    // [nnz] caller's position of kernel-order entry p
    std::vector<Seg> segs;         // longest first; equal lengths keep row order
    std::vector<SplitRow> splits;
};

constexpr uint32_t kDefaultSegMax = 128;

// Returns 0, or an spc3d_status value with `err` filled.
int validate_coo(uint32_t nrows, uint32_t ncols, uint64_t nnz, const uint32_t *ii,
                 const uint32_t *jj, std::string &err);

// Validates, then builds.  Entries are grouped by row with a stable counting
// sort, so within a row the caller's order (the order the reference
// accumulates in, core_ops.cpp:26-34) is kept.
int build_host_plan(uint32_t nrows, uint32_t ncols, uint64_t nnz, const uint32_t *ii,
                    const uint32_t *jj, uint32_t seg_max, HostPlan &out, std::string &err);

} // namespace spc3d
