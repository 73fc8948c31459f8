// Host-only test of the content keys behind the one-shot host calls
// (spcomm3d_amd/csrc/host_cache.cpp): what decides whether a plan or a device panel may
// be reused.  A key must never be the same for two contents that differ in one word, in
// the order of two words, or in length; and it must not depend on how many threads made it.
#include <cstdio>
#include <cstring>
#include <random>
#include <vector>

#include "../../spcomm3d_amd/csrc/host_cache.h"

using namespace spc3d;

static int g_fail = 0;
#define CHECK(cond)                                                                               \
    do {                                                                                          \
        if (!(cond)) {                                                                            \
            std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond);                           \
            ++g_fail;                                                                             \
        }                                                                                         \
    } while (0)

template <typename KeyFn> static void single_block_properties(KeyFn key_of_block, std::mt19937_64 &g)
{
    // ---- one block, every length around the 32-byte stride and the tail -------------------
    for (size_t bytes : {(size_t)0, (size_t)1, (size_t)7, (size_t)8, (size_t)31, (size_t)32, (size_t)33, (size_t)63,
                         (size_t)64, (size_t)100, (size_t)4096, (size_t)4099}) {
        std::vector<unsigned char> a(bytes + 8);
        for (auto &x : a)
            x = (unsigned char)g();
        const BlockKey k0 = key_of_block(a.data(), bytes);
        CHECK(k0 == key_of_block(a.data(), bytes));
        // a byte more is another content, also when the byte is zero
        std::vector<unsigned char> z(bytes + 1, 0), z2(bytes + 2, 0);
        CHECK(key_of_block(z.data(), bytes) != key_of_block(z.data(), bytes + 1));
        for (size_t at = 0; at < bytes; ++at) { // every single byte matters
            a[at] ^= 0x10;
            CHECK(key_of_block(a.data(), bytes) != k0);
            a[at] ^= 0x10;
        }
        CHECK(key_of_block(a.data(), bytes) == k0);
    }
    // ---- words that trade places, or change so that their sum stays ------------------------
    {
        std::vector<uint64_t> w(1 << 12);
        for (auto &x : w)
            x = g();
        const size_t bytes = w.size() * 8;
        const BlockKey k0 = key_of_block(w.data(), bytes);
        for (int rep = 0; rep < 2000; ++rep) {
            const size_t i = g() % w.size(), j = g() % w.size();
            if (w[i] == w[j])
                continue;
            std::swap(w[i], w[j]); // the sum of the words is what it was
            CHECK(key_of_block(w.data(), bytes) != k0);
            std::swap(w[i], w[j]);
            const uint64_t d = g() | 1;
            w[i] += d, w[j] -= d; // so is it here
            CHECK(key_of_block(w.data(), bytes) != k0);
            w[i] -= d, w[j] += d;
        }
        // index arrays as ReMapIndices leaves them: a permutation of the same values
        std::vector<uint32_t> idx(1 << 16), back;
        for (size_t i = 0; i < idx.size(); ++i)
            idx[i] = (uint32_t)(g() % 1000);
        back = idx;
        const BlockKey ki = key_of_block(idx.data(), idx.size() * 4);
        for (auto &x : idx)
            x = (x * 7 + 3) % 1000; // a bijection of 0..999
        CHECK(key_of_block(idx.data(), idx.size() * 4) != ki);
        CHECK(key_of_block(back.data(), back.size() * 4) == ki);
    }
}

int main()
{
    std::mt19937_64 g(3);
    single_block_properties(key_of_block, g);
    single_block_properties(key_of_block_portable, g); // the form for hosts without CRC-32C
    // ---- many blocks: split at 4 MiB, the same on any number of threads ---------------------
    {
        const size_t bytes = 3 * kKeyBlockBytes + 12345;
        std::vector<unsigned char> a(bytes);
        uint64_t x = 88172645463325252ull;
        for (size_t i = 0; i + 8 <= bytes; i += 8) {
            x ^= x << 13, x ^= x >> 7, x ^= x << 17;
            std::memcpy(&a[i], &x, 8);
        }
        std::vector<BlockKey> k1, k8, kd;
        keys_of(a.data(), bytes, k1, 1);
        keys_of(a.data(), bytes, k8, 8);
        keys_of(a.data(), bytes, kd);
        CHECK(k1.size() == 4 && k1 == k8 && k1 == kd);
        for (size_t b = 0; b < 4; ++b) {
            const size_t off = b * kKeyBlockBytes;
            CHECK(k1[b] == key_of_block(a.data() + off, b < 3 ? kKeyBlockBytes : bytes - off));
        }
        // a change shows in its block and in no other
        for (size_t at : {(size_t)0, kKeyBlockBytes - 1, kKeyBlockBytes, 2 * kKeyBlockBytes + 77, bytes - 1}) {
            a[at] ^= 1;
            keys_of(a.data(), bytes, k8, 8);
            for (size_t b = 0; b < 4; ++b)
                CHECK((k8[b] != k1[b]) == (at / kKeyBlockBytes == b));
            a[at] ^= 1;
        }
        std::vector<BlockKey> none;
        keys_of(a.data(), 0, none);
        CHECK(none.empty());
    }
    std::printf("%s (%d failures)\n", g_fail ? "FAILED" : "PASSED", g_fail);
    return g_fail ? 1 : 0;
}
