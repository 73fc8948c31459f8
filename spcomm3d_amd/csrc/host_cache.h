// Content keys of host operands, for the one-shot entry points over host memory
// (spc3d_sddmm_host / spc3d_spmm_host).  The reference's drivers call the kernel several
// times over one pattern and the same dense panels (miniapp/bench_both.cpp:202-203,
// bench_spmm.cpp:185-186), and rewrite indices in place at the same addresses between
// groups of calls (ReMapIndices, bench_both.cpp:200-205): what a call may reuse from the
// one before is decided by what the operands hold, never by where they are.
//
// An operand is keyed block by block (4 MiB): a block whose key is unchanged is not sent
// again, a changed one is.  Every byte goes into the key, over several threads (reading
// host memory with a few threads is faster than sending it: the point of the exercise).
#pragma once

#include <cstddef>
#include <cstdint>
#include <vector>

namespace spc3d {

// Key of one block: four interleaved CRC-32C streams over its 8-byte words (crc01,
// crc23), their plain sum and a rotate-xor fold.  A change of one word always changes
// the sum; several changes have to cancel in the sum, the fold and their CRC streams at once.
struct BlockKey {
    uint64_t crc01 = 0, crc23 = 0, sum = 0, fold = 0;
    bool operator==(const BlockKey &o) const
    {
        return crc01 == o.crc01 && crc23 == o.crc23 && sum == o.sum && fold == o.fold;
    }
    bool operator!=(const BlockKey &o) const { return !(*this == o); }
};

constexpr size_t kKeyBlockBytes = (size_t)4 << 20;

BlockKey key_of_block(const void *data, size_t bytes);
// The form used on hosts without the CRC-32C instruction (multiply-xorshift chains in place
// of the CRC streams); exposed so that it is tested on hosts that have the instruction.
BlockKey key_of_block_portable(const void *data, size_t bytes);

// Keys of every kKeyBlockBytes block of `data` (the last one may be short), computed on up
// to `threads` threads (0: a default from the machine, at most 8).
void keys_of(const void *data, size_t bytes, std::vector<BlockKey> &out, unsigned threads = 0);

} // namespace spc3d
