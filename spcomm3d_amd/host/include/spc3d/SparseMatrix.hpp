// Sparse operand types with the reference's names and members
// (src/SparseMatrix.hpp:12-29 SparseMatrix, :31-109 COOMatrix, :133-135
// aliases).  The reference's CSRMatrix (:110-132) is a stub that does not
// compile when instantiated and has no user; it is not mirrored.
//
// Index transforms that run before the kernels are kept with their exact
// results:
//   localizeIndices (:69-99): a global id gets the next local id the first
//     time it appears in the entry stream; only touched rows / columns get
//     ids; ltgR / ltgC invert the maps.
//   ReMapIndices (:100-106): ii[i] = mapR[ii[i]], jj[i] = mapC[jj[i]].
//   self_generate_random (:49-67): distinct random positions, value 1.
#pragma once

#include <chrono>
#include <cstdint>
#include <iostream>
#include <random>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <vector>

#include "basic.hpp"

namespace SpKernels {

template <typename T, typename IdxT> class SparseMatrix {
  public:
    std::vector<IdxT> ltgR, ltgC;               // local -> global row / column id
    std::vector<T> ownedVals;                   // this rank's share after the Z reduction
    std::unordered_map<IdxT, IdxT> gtlR, gtlC;  // global -> local
    std::string mtxName;
    int rank = 0, xyrank = 0, zrank = 0;
    IdxT nrows = 0, ncols = 0, ownedNnz = 0, gnrows = 0, gncols = 0;
    idx_large_t nnz = 0, gnnz = 0;

    virtual ~SparseMatrix() = default;
    virtual void localizeIndices() {}
    virtual void delocalizeIndices() {}
    virtual void ReMapIndices(std::vector<IdxT>, std::vector<IdxT>) {}
};

template <typename T, typename IdxT> class COOMatrix : public SparseMatrix<T, IdxT> {
  public:
    std::vector<IdxT> ii, jj;
    std::vector<T> vv;

    // Appends to the arrays only; nnz is the caller's to keep (as in the reference).
    void addEntry(IdxT row, IdxT col, T val)
    {
        ii.push_back(row);
        jj.push_back(col);
        vv.push_back(val);
    }

    void printMatrix(int count = 0) const
    {
        const idx_large_t n = count == 0 ? this->nnz : static_cast<idx_large_t>(count);
        for (idx_large_t i = 0; i < n; ++i)
            std::cout << ii[i] << " " << jj[i] << " " << vv[i] << std::endl;
    }

    // Appends count entries of value 1 at distinct random positions of the
    // gnrows x gncols pattern (SparseMatrix.hpp:49-67 seeds from the clock; a seed can
    // be given here so that a run can be repeated).  nnz stays the caller's to set.
    void self_generate_random(IdxT count, std::uint64_t seed = 0)
    {
        const std::uint64_t cells = (std::uint64_t)this->gnrows * this->gncols;
        if (count > cells)
            throw std::out_of_range("self_generate_random: more entries than cells");
        std::mt19937_64 rng(seed ? seed
                                 : (std::uint64_t)std::chrono::steady_clock::now()
                                       .time_since_epoch()
                                       .count());
        std::unordered_set<std::uint64_t> used;
        used.reserve(count * 2);
        for (IdxT made = 0; made < count;) {
            const std::uint64_t cell = rng() % cells;
            if (!used.insert(cell).second)
                continue; // a position is used once
            addEntry((IdxT)(cell / this->gncols), (IdxT)(cell % this->gncols), (T)1);
            ++made;
        }
    }

    void localizeIndices() override
    {
        this->ltgR.clear();
        this->ltgC.clear();
        this->nrows = 0;
        this->ncols = 0;
        for (idx_large_t i = 0; i < this->nnz; ++i) {
            if (this->gtlR.emplace(ii.at(i), this->nrows).second)
                ++this->nrows;
            if (this->gtlC.emplace(jj.at(i), this->ncols).second)
                ++this->ncols;
        }
        this->ltgR.resize(this->nrows);
        this->ltgC.resize(this->ncols);
        for (const auto &kv : this->gtlR)
            this->ltgR[kv.second] = kv.first;
        for (const auto &kv : this->gtlC)
            this->ltgC[kv.second] = kv.first;
        for (idx_large_t i = 0; i < this->nnz; ++i) {
            ii[i] = this->gtlR.at(ii[i]);
            jj[i] = this->gtlC.at(jj[i]);
        }
    }

    void ReMapIndices(std::vector<IdxT> mapR, std::vector<IdxT> mapC) override
    {
        for (idx_large_t i = 0; i < this->nnz; ++i) {
            ii[i] = mapR.at(ii[i]);
            jj[i] = mapC.at(jj[i]);
        }
    }
};

using SpMat = SparseMatrix<real_t, idx_t>;
using cooMat = COOMatrix<real_t, idx_t>;

} // namespace SpKernels
