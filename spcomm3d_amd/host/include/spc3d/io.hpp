// The two on-disk formats the reference's drivers read, with the reference's
// names: the MatrixMarket reader `SpKernels::mm` (src/mm.hpp:13-80) and the
// binary triplet file of tools/read_convert_mm.cpp.
//
// Binary layout (tools/read_convert_mm.cpp:81-94, read side :96-115 and
// src/parallel_io.hpp:61-63,91-94): little-endian, no padding,
//     uint32 rows, uint32 cols, uint64 nnz,
//     nnz x { uint32 row, uint32 col, float64 value }      (16 bytes each)
// indices 0-based.  Values are float64 on disk whatever real_t is in memory.
#pragma once

#include <algorithm>
#include <charconv>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <random>
#include <stdexcept>
#include <string>
#include <vector>

#include "SparseMatrix.hpp"
#include "basic.hpp"

namespace SpKernels {

// Whitespace-separated tokens of a text file, read in large blocks and converted
// with std::from_chars: the same numbers `stream >> x` gives (both round decimal text
// correctly) in 0.38 of the time of formatted stream extraction (4 M entries, 134 MB of
// text: 0.75 s against 1.96 s).  A leading '+' is accepted as stream extraction
// accepts it.
class TokenReader {
  public:
    // `block`: bytes read at a time (the tests make it tiny to put tokens across blocks)
    explicit TokenReader(std::ifstream &f, std::size_t block = (std::size_t)32 << 20)
        : f_(f), block_(block), buf_(block + kCarry)
    {
    }

    // The next token as an unsigned integer / a double; false at the end of the
    // file or when the token is not such a number.
    bool next(std::uint64_t &v)
    {
        const char *b, *e;
        if (!token(b, e))
            return false;
        if (b != e && *b == '+')
            ++b;
        const auto r = std::from_chars(b, e, v);
        return r.ec == std::errc() && r.ptr == e;
    }
    bool next(double &v)
    {
        const char *b, *e;
        if (!token(b, e))
            return false;
        if (b != e && *b == '+')
            ++b;
        const auto r = std::from_chars(b, e, v);
        // "inf" and "nan" are no numbers to stream extraction; from_chars would take them
        return r.ec == std::errc() && r.ptr == e && std::isfinite(v);
    }

  private:
    static constexpr std::size_t kCarry = 4096;
    static bool space(char c) { return c == ' ' || c == '\n' || c == '\t' || c == '\r' || c == '\v' || c == '\f'; }

    // Moves the unread tail to the front and reads on; false when nothing is left.
    bool refill()
    {
        const std::size_t tail = end_ - pos_;
        if (tail > kCarry)
            return false; // a "token" longer than any number: give up on it
        std::memmove(buf_.data(), buf_.data() + pos_, tail);
        pos_ = 0;
        end_ = tail;
        if (!f_.eof()) {
            f_.read(buf_.data() + end_, (std::streamsize)block_);
            end_ += (std::size_t)f_.gcount();
        }
        return end_ > tail;
    }
    bool token(const char *&b, const char *&e)
    {
        for (;;) { // skip whitespace
            while (pos_ < end_ && space(buf_[pos_]))
                ++pos_;
            if (pos_ < end_)
                break;
            if (!refill())
                return false;
        }
        std::size_t q = pos_;
        for (;;) { // the token may run into the end of the block
            while (q < end_ && !space(buf_[q]))
                ++q;
            if (q < end_ || f_.eof())
                break;
            const std::size_t len = q - pos_;
            const bool more = refill(); // the token now starts the buffer
            q = pos_ == 0 ? len : q;
            if (!more)
                break;
        }
        b = buf_.data() + pos_;
        e = buf_.data() + q;
        pos_ = q;
        return b != e;
    }

    std::ifstream &f_;
    std::size_t block_;
    std::vector<char> buf_;
    std::size_t pos_ = 0, end_ = 0;
};

// MatrixMarket coordinate reader.  What it does with the file is what the
// reference does, quirks included:
//   - "pattern", "symmetric", "complex" are recognised anywhere in the banner;
//   - entries become 0-based; a pattern entry gets value 1; the imaginary part
//     of a complex entry is dropped;
//   - a symmetric file yields 2 x (stored entries): entry i is mirrored into
//     position i + stored, diagonal entries included (so a diagonal entry
//     appears twice, src/mm.hpp:53-57);
//   - nnz = gnnz, nrows = gnrows, ncols = gncols are set from the size line.
// Unlike the reference it reports a file that cannot be opened or that ends
// early (std::runtime_error) instead of returning garbage.
class mm {
  public:
    explicit mm(std::string FN) : _FN(std::move(FN)) {}
    virtual ~mm() = default;

    void read_mm(std::string FN, cooMat &M)
    {
        std::ifstream f(FN.c_str());
        if (!f)
            throw std::runtime_error("read_mm: cannot open " + FN);
        std::string banner;
        std::getline(f, banner);
        const bool pattern = banner.find("pattern") != std::string::npos;
        const bool symm = banner.find("symmetric") != std::string::npos;
        const bool cplx = banner.find("complex") != std::string::npos;
        while (f.peek() == '%')
            f.ignore(1 << 20, '\n');
        TokenReader tok(f);
        std::uint64_t rows64 = 0, cols64 = 0, stored64 = 0;
        if (!tok.next(rows64) || !tok.next(cols64) || !tok.next(stored64) ||
            rows64 > 0xFFFFFFFFull || cols64 > 0xFFFFFFFFull)
            throw std::runtime_error("read_mm: no size line in " + FN);
        const idx_t rows = (idx_t)rows64, cols = (idx_t)cols64;
        const idx_large_t stored = stored64;
        const idx_large_t total = symm ? 2 * stored : stored;
        M.ii.assign(total, 0);
        M.jj.assign(total, 0);
        M.vv.assign(total, (real_t)0);
        M.gnnz = M.nnz = total;
        M.gnrows = M.nrows = rows;
        M.gncols = M.ncols = cols;
        for (idx_large_t i = 0; i < stored; ++i) {
            std::uint64_t r = 0, c = 0;
            double v = 1.0, im = 0.0;
            bool ok = tok.next(r) && tok.next(c);
            if (ok && !pattern) {
                ok = tok.next(v);
                if (ok && cplx)
                    ok = tok.next(im);
            }
            if (!ok)
                throw std::runtime_error("read_mm: " + FN + " ends before its last entry");
            M.ii[i] = (idx_t)(r - 1);
            M.jj[i] = (idx_t)(c - 1);
            M.vv[i] = (real_t)v;
            if (symm) {
                M.ii[i + stored] = (idx_t)(c - 1);
                M.jj[i + stored] = (idx_t)(r - 1);
                M.vv[i + stored] = (real_t)v;
            }
        }
    }

  private:
    std::string _FN;
};

// tools/read_convert_mm.cpp:81-94: header from gnrows / gncols / gnnz, then the
// first gnnz triplets.
inline void convert_to_binary(const cooMat &C, const std::string &outputFN)
{
    if (C.ii.size() < C.gnnz || C.jj.size() < C.gnnz || C.vv.size() < C.gnnz)
        throw std::out_of_range("convert_to_binary: fewer than gnnz entries");
    std::ofstream o(outputFN, std::ios::binary | std::ios::trunc);
    if (!o)
        throw std::runtime_error("convert_to_binary: cannot open " + outputFN);
    const std::uint32_t r = C.gnrows, c = C.gncols;
    const std::uint64_t n = C.gnnz;
    o.write(reinterpret_cast<const char *>(&r), 4);
    o.write(reinterpret_cast<const char *>(&c), 4);
    o.write(reinterpret_cast<const char *>(&n), 8);
    std::vector<char> block;
    const idx_large_t kChunk = 1 << 16;
    for (idx_large_t at = 0; at < n; at += kChunk) {
        const idx_large_t m = std::min<idx_large_t>(kChunk, n - at);
        block.resize(m * 16);
        for (idx_large_t i = 0; i < m; ++i) {
            const std::uint32_t ri = C.ii[at + i], ci = C.jj[at + i];
            const double v = (double)C.vv[at + i];
            std::memcpy(&block[i * 16], &ri, 4);
            std::memcpy(&block[i * 16 + 4], &ci, 4);
            std::memcpy(&block[i * 16 + 8], &v, 8);
        }
        o.write(block.data(), (std::streamsize)block.size());
    }
    if (!o)
        throw std::runtime_error("convert_to_binary: write to " + outputFN + " failed");
}

// The serial reader (tools/read_convert_mm.cpp:96-115): fills gnrows, gncols,
// gnnz and the three arrays.  With single_rank = true it also sets nnz, nrows,
// ncols to the global sizes, which is what one rank ends up holding after
// read_bin_parallel_distribute_coo (src/parallel_io.hpp:132-190) before
// localizeIndices.
inline void read_binary(const std::string &inFN, cooMat &C, bool single_rank = true)
{
    std::ifstream f(inFN, std::ios::binary);
    if (!f)
        throw std::runtime_error("read_binary: cannot open " + inFN);
    std::uint32_t r = 0, c = 0;
    std::uint64_t n = 0;
    f.read(reinterpret_cast<char *>(&r), 4);
    f.read(reinterpret_cast<char *>(&c), 4);
    f.read(reinterpret_cast<char *>(&n), 8);
    if (!f)
        throw std::runtime_error("read_binary: " + inFN + " has no header");
    // a header that promises more triplets than the file holds must not size the arrays
    f.seekg(0, std::ios::end);
    const std::uint64_t file_bytes = (std::uint64_t)f.tellg();
    f.seekg(16, std::ios::beg);
    if (n > (file_bytes - 16) / 16)
        throw std::runtime_error("read_binary: " + inFN + " ends before its last entry");
    C.gnrows = r;
    C.gncols = c;
    C.gnnz = n;
    C.ii.resize(n);
    C.jj.resize(n);
    C.vv.resize(n);
    std::vector<char> block;
    const idx_large_t kChunk = 1 << 16;
    for (idx_large_t at = 0; at < n; at += kChunk) {
        const idx_large_t m = std::min<idx_large_t>(kChunk, n - at);
        block.resize(m * 16);
        f.read(block.data(), (std::streamsize)block.size());
        if (!f)
            throw std::runtime_error("read_binary: " + inFN + " ends before its last entry");
        for (idx_large_t i = 0; i < m; ++i) {
            double v;
            std::memcpy(&C.ii[at + i], &block[i * 16], 4);
            std::memcpy(&C.jj[at + i], &block[i * 16 + 4], 4);
            std::memcpy(&v, &block[i * 16 + 8], 8);
            C.vv[at + i] = (real_t)v;
        }
    }
    if (single_rank) {
        C.nnz = n;
        C.nrows = r;
        C.ncols = c;
        C.ownedNnz = (idx_t)n;
    }
}

// The 2D block of one rank, from a binary file, in a single process: what
// read_bin_parallel_distribute_coo (src/parallel_io.hpp:132-190) leaves in Sloc on the rank
// with coordinates (gx, gy, gz) of an X x Y x Z mesh, ready for localizeIndices()
// (miniapp/bench_both.cpp:156-158).  The rule (src/parallel_io.hpp:64-76,98-105): the row
// ids are permuted at random and dealt to the X row groups round-robin, the i-th row of the
// permuted order to group i mod X; the column ids likewise to the Y column groups; entry
// (r, c) belongs to the rank at (rpvec2D[r], cpvec2D[c]).  A rank ends up with its entries
// in file order: every reader forwards its contiguous share of the file in order, and the
// shares arrive in reader order (:86-94,107-123).  All Z ranks of a fibre hold the same block
// (:150-163) and own lnnz / Z of its values, the first lnnz mod Z of them one more (:166-169).
//
// The reference shuffles with std::random_shuffle and no seed, so its partition differs from
// run to run; here the permutation is a Fisher-Yates shuffle driven by std::mt19937_64(seed)
// (position i swapped with position rng() mod (i + 1), from the back), the same on every
// platform.  rpvec2D / cpvec2D return the group of every row and column as the reference's
// reader does; the partitioner that runs next reads them (src/distribute.cpp:152,197,204).
//
// The file is streamed: memory is the two group vectors plus the block.
inline void read_binary_block(const std::string &inFN, cooMat &C, int X, int Y, int gx, int gy,
                              std::uint64_t seed, std::vector<int> &rpvec2D,
                              std::vector<int> &cpvec2D, int Z = 1, int gz = 0)
{
    if (X < 1 || Y < 1 || Z < 1 || gx < 0 || gx >= X || gy < 0 || gy >= Y || gz < 0 || gz >= Z)
        throw std::out_of_range("read_binary_block: no such rank in the mesh");
    std::ifstream f(inFN, std::ios::binary);
    if (!f)
        throw std::runtime_error("read_binary_block: cannot open " + inFN);
    std::uint32_t r = 0, c = 0;
    std::uint64_t n = 0;
    f.read(reinterpret_cast<char *>(&r), 4);
    f.read(reinterpret_cast<char *>(&c), 4);
    f.read(reinterpret_cast<char *>(&n), 8);
    if (!f)
        throw std::runtime_error("read_binary_block: " + inFN + " has no header");
    f.seekg(0, std::ios::end);
    const std::uint64_t file_bytes = (std::uint64_t)f.tellg();
    f.seekg(16, std::ios::beg);
    if (n > (file_bytes - 16) / 16)
        throw std::runtime_error("read_binary_block: " + inFN + " ends before its last entry");

    std::mt19937_64 rng(seed);
    auto deal = [&rng](std::uint32_t count, int groups, std::vector<int> &group_of) {
        std::vector<idx_t> order(count);
        for (std::uint32_t i = 0; i < count; ++i)
            order[i] = i;
        for (std::uint32_t i = count; i > 1; --i)
            std::swap(order[i - 1], order[rng() % i]);
        group_of.assign(count, 0);
        for (std::uint32_t i = 0; i < count; ++i)
            group_of[order[i]] = (int)(i % (std::uint32_t)groups);
    };
    deal(r, X, rpvec2D); // rows first, then columns, as the reference draws them
    deal(c, Y, cpvec2D);

    C.gnrows = r;
    C.gncols = c;
    C.gnnz = n;
    C.ii.clear();
    C.jj.clear();
    C.vv.clear();
    std::vector<char> block;
    const idx_large_t kChunk = 1 << 16;
    for (idx_large_t at = 0; at < n; at += kChunk) {
        const idx_large_t m = std::min<idx_large_t>(kChunk, n - at);
        block.resize(m * 16);
        f.read(block.data(), (std::streamsize)block.size());
        if (!f)
            throw std::runtime_error("read_binary_block: " + inFN + " ends before its last entry");
        for (idx_large_t i = 0; i < m; ++i) {
            std::uint32_t ri, ci;
            double v;
            std::memcpy(&ri, &block[i * 16], 4);
            std::memcpy(&ci, &block[i * 16 + 4], 4);
            if (ri >= r || ci >= c)
                throw std::out_of_range("read_binary_block: entry outside the matrix in " + inFN);
            if (rpvec2D[ri] != gx || cpvec2D[ci] != gy)
                continue;
            std::memcpy(&v, &block[i * 16 + 8], 8);
            C.ii.push_back(ri);
            C.jj.push_back(ci);
            C.vv.push_back((real_t)v);
        }
    }
    const idx_large_t lnnz = C.ii.size();
    C.nnz = lnnz;
    C.ownedNnz = (idx_t)(lnnz / (idx_large_t)Z + ((idx_large_t)gz < lnnz % (idx_large_t)Z ? 1 : 0));
    C.ownedVals.assign(C.ownedNnz, (real_t)0);
}

} // namespace SpKernels
