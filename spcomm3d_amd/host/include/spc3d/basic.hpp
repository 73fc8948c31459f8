// Host-side types of the local compute step, with the reference's names and
// member layout so that code written against src/basic.hpp compiles against
// this header unchanged.
//
// Mirrors (reference paths): src/basic.hpp:16-18 (idx_t / real_t /
// idx_large_t), :20-22 (parallelTiming), :24-28 (triplet), :30-44
// (denseMatrix).  Differences, all deliberate:
//   - the scalar types are real typedefs, not #defines, and real_t can be
//     switched to float with -DSPC3D_REAL=float (the reference is double only);
//   - denseMatrix::at computes its offset in 64 bits (the reference's 32-bit
//     x*n+y wraps for m*n >= 2^32).
#pragma once

#include <cstddef>
#include <cstdint>
#include <iostream>
#include <vector>

#ifndef SPC3D_REAL
#define SPC3D_REAL double
#endif

namespace SpKernels {

using idx_t = std::uint32_t;
using real_t = SPC3D_REAL;
using idx_large_t = std::uint64_t;

static_assert(sizeof(real_t) == 4 || sizeof(real_t) == 8, "real_t must be float or double");

// Per-call phase times in whole milliseconds, as the reference reports them
// (five idx_t, the reference's layout).
struct parallelTiming {
    idx_t comm1Time = 0, comm2Time = 0, commcpyTime = 0, compTime = 0, totalTime = 0;
};

struct triplet {
    idx_t row;
    idx_t col;
    real_t val;
};

// Dense panel: m x n, row-major, n contiguous.  ltg / gtl are the local<->global
// row maps the distribution code fills; the kernels do not read them.
struct denseMatrix {
    idx_t m = 0, n = 0;
    std::vector<real_t> data;
    std::vector<idx_t> ltg;
    std::vector<idx_t> gtl;

    real_t &at(idx_t x, idx_t y) { return data.at(static_cast<std::size_t>(x) * n + y); }
    const real_t &at(idx_t x, idx_t y) const
    {
        return data.at(static_cast<std::size_t>(x) * n + y);
    }

    // "row col value" per line; count != 0 limits the output to count / n rows.
    void printMatrix(idx_t count = 0) const
    {
        const idx_t rows = count ? count / (n ? n : 1) : m;
        for (idx_t i = 0; i < rows; ++i)
            for (idx_t j = 0; j < n; ++j)
                std::cout << i << " " << j << " " << at(i, j) << std::endl;
    }
};

} // namespace SpKernels
