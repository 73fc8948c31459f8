// Content keys of host operands (see host_cache.h).  Host code only.
#include "host_cache.h"

#include <algorithm>
#include <atomic>
#include <cstring>
#include <system_error>
#include <thread>

#if defined(__x86_64__)
#include <nmmintrin.h>
#endif

namespace spc3d {

namespace {

inline uint64_t rotl(uint64_t x, int r) { return (x << r) | (x >> (64 - r)); }

// Portable form: the CRC streams become multiply-xorshift chains.
void key_plain(const unsigned char *p, size_t bytes, BlockKey &k)
{
    uint64_t h[4] = {bytes, ~(uint64_t)bytes, 0x9E3779B97F4A7C15ull, 0xD6E8FEB86659FD93ull};
    uint64_t sum = 0, fold = 0;
    size_t i = 0;
    for (; i + 32 <= bytes; i += 32) {
        uint64_t w[4];
        std::memcpy(w, p + i, 32);
        for (int l = 0; l < 4; ++l) {
            h[l] = (h[l] ^ w[l]) * 0xBF58476D1CE4E5B9ull;
            h[l] ^= h[l] >> 29;
            sum += w[l];
            fold = rotl(fold, 5) ^ w[l];
        }
    }
    uint64_t tail[4] = {0, 0, 0, 0};
    std::memcpy(tail, p + i, bytes - i);
    for (int l = 0; l < 4; ++l) {
        h[l] = (h[l] ^ tail[l]) * 0x94D049BB133111EBull;
        sum += tail[l];
        fold = rotl(fold, 5) ^ tail[l];
    }
    k.crc01 = h[0] ^ (h[1] >> 31);
    k.crc23 = h[2] ^ (h[3] >> 31);
    k.sum = sum;
    k.fold = fold;
}

#if defined(__x86_64__)
__attribute__((target("sse4.2"))) void key_crc(const unsigned char *p, size_t bytes, BlockKey &k)
{
    uint64_t h[4] = {bytes & 0xFFFFFFFFu, 0x1F3D5B79u, 0x2E4C6A80u, 0x3D5B798Fu};
    uint64_t sum = 0, fold = 0;
    size_t i = 0;
    for (; i + 32 <= bytes; i += 32) {
        uint64_t w[4];
        std::memcpy(w, p + i, 32);
        h[0] = _mm_crc32_u64(h[0], w[0]);
        h[1] = _mm_crc32_u64(h[1], w[1]);
        h[2] = _mm_crc32_u64(h[2], w[2]);
        h[3] = _mm_crc32_u64(h[3], w[3]);
        sum += (w[0] + w[1]) + (w[2] + w[3]);
        fold = rotl(fold, 5) ^ (w[0] ^ rotl(w[1], 17) ^ rotl(w[2], 31) ^ rotl(w[3], 47));
    }
    uint64_t tail[4] = {0, 0, 0, 0};
    std::memcpy(tail, p + i, bytes - i);
    for (int l = 0; l < 4; ++l) {
        h[l] = _mm_crc32_u64(h[l], tail[l]);
        sum += tail[l];
    }
    fold = rotl(fold, 5) ^ (tail[0] ^ rotl(tail[1], 17) ^ rotl(tail[2], 31) ^ rotl(tail[3], 47));
    k.crc01 = h[0] | (h[1] << 32);
    k.crc23 = h[2] | (h[3] << 32);
    k.sum = sum;
    k.fold = fold;
}
#endif

} // namespace

BlockKey key_of_block_portable(const void *data, size_t bytes)
{
    BlockKey k;
    key_plain(static_cast<const unsigned char *>(data), bytes, k);
    return k;
}

BlockKey key_of_block(const void *data, size_t bytes)
{
    BlockKey k;
    const unsigned char *p = static_cast<const unsigned char *>(data);
#if defined(__x86_64__)
    static const bool crc = __builtin_cpu_supports("sse4.2");
    if (crc) {
        key_crc(p, bytes, k);
        return k;
    }
#endif
    key_plain(p, bytes, k);
    return k;
}

void keys_of(const void *data, size_t bytes, std::vector<BlockKey> &out, unsigned threads)
{
    const size_t nblocks = (bytes + kKeyBlockBytes - 1) / kKeyBlockBytes;
    out.assign(nblocks, BlockKey());
    if (nblocks == 0)
        return;
    if (threads == 0) {
        const unsigned hw = std::thread::hardware_concurrency();
        threads = std::min(8u, hw ? hw : 1u);
    }
    threads = (unsigned)std::min<size_t>(threads, nblocks);
    const unsigned char *p = static_cast<const unsigned char *>(data);
    std::atomic<size_t> next{0};
    auto work = [&]() {
        for (;;) {
            const size_t b = next.fetch_add(1, std::memory_order_relaxed);
            if (b >= nblocks)
                return;
            const size_t off = b * kKeyBlockBytes;
            out[b] = key_of_block(p + off, std::min(kKeyBlockBytes, bytes - off));
        }
    };
    if (threads <= 1) {
        work();
        return;
    }
    std::vector<std::thread> pool;
    pool.reserve(threads - 1);
    try {
        for (unsigned t = 1; t < threads; ++t)
            pool.emplace_back(work);
    } catch (const std::system_error &) {
        // no more threads to be had: those that started and this one share the blocks
    }
    work();
    for (std::thread &t : pool)
        t.join();
}

} // namespace spc3d
