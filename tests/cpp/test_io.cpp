// Host-only test of spc3d/io.hpp against golden files written by the reference's
// own converter (tests/golden/io/*.bin, made by tests/golden/make_golden_io.py
// from the .mtx files beside them): reading a .mtx and converting it must give
// the reference's bytes; reading the reference's .bin must give the same matrix.
//
//   test_io <dir with the golden files>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <iterator>
#include <string>
#include <vector>

#include "spc3d/io.hpp"

using namespace SpKernels;

static int g_fail = 0;
#define CHECK(cond)                                                                               \
    do {                                                                                          \
        if (!(cond)) {                                                                            \
            std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond);                           \
            ++g_fail;                                                                             \
        }                                                                                         \
    } while (0)

static std::vector<char> slurp(const std::string &fn)
{
    std::ifstream f(fn, std::ios::binary);
    return std::vector<char>((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
}

static void check_file(const std::string &dir, const char *stem, idx_large_t want_nnz)
{
    const std::string mtx = dir + "/" + stem + ".mtx", bin = dir + "/" + stem + ".bin";
    cooMat M;
    mm reader(mtx);
    reader.read_mm(mtx, M);
    CHECK(M.nnz == want_nnz && M.gnnz == want_nnz);
    const std::string tmp = std::string("/tmp/spc3d_test_io_") + stem + ".bin";
    convert_to_binary(M, tmp);
    const std::vector<char> mine = slurp(tmp), ref = slurp(bin);
    CHECK(!ref.empty());
    if (sizeof(real_t) == 8)
        CHECK(mine == ref); // byte for byte what the reference's converter wrote
    else
        CHECK(mine.size() == ref.size());
    cooMat R;
    read_binary(bin, R);
    CHECK(R.gnrows == M.gnrows && R.gncols == M.gncols && R.gnnz == M.gnnz && R.nnz == M.nnz);
    CHECK(R.ii == M.ii && R.jj == M.jj && R.vv == M.vv);
    std::remove(tmp.c_str());
}

// read_binary_block: one rank's 2D block in a single process.  The reference's shuffle is
// unseeded, so there is no reference output to compare with; what is held to are the
// properties its partition has by construction (src/parallel_io.hpp:64-76,98-105) and the
// ones its partitioner relies on (src/distribute.cpp:152,197,204: every entry of a block has
// the block's row group and column group).
static void check_blocks(const std::string &bin, int X, int Y, int Z, std::uint64_t seed)
{
    cooMat W;
    read_binary(bin, W);
    std::vector<int> rp0, cp0;
    std::vector<char> seen(W.nnz, 0);
    idx_large_t total = 0;
    for (int gx = 0; gx < X; ++gx)
        for (int gy = 0; gy < Y; ++gy) {
            cooMat Bk;
            std::vector<int> rp, cp;
            read_binary_block(bin, Bk, X, Y, gx, gy, seed, rp, cp, Z, Z - 1);
            if (gx == 0 && gy == 0) {
                rp0 = rp;
                cp0 = cp;
                // round-robin over a permutation: group sizes differ by at most one
                std::vector<idx_t> nr(X, 0), nc(Y, 0);
                for (int g : rp) {
                    CHECK(g >= 0 && g < X);
                    ++nr[g];
                }
                for (int g : cp) {
                    CHECK(g >= 0 && g < Y);
                    ++nc[g];
                }
                for (int g = 0; g < X; ++g)
                    CHECK(nr[g] == W.gnrows / X + ((idx_t)g < W.gnrows % X ? 1 : 0));
                for (int g = 0; g < Y; ++g)
                    CHECK(nc[g] == W.gncols / Y + ((idx_t)g < W.gncols % Y ? 1 : 0));
            }
            CHECK(rp == rp0 && cp == cp0); // one partition for all ranks
            CHECK(Bk.gnrows == W.gnrows && Bk.gncols == W.gncols && Bk.gnnz == W.gnnz);
            CHECK(Bk.nnz == Bk.ii.size() && Bk.jj.size() == Bk.nnz && Bk.vv.size() == Bk.nnz);
            CHECK(Bk.ownedNnz == Bk.nnz / Z && Bk.ownedVals.size() == Bk.ownedNnz); // last Z rank
            // the block is the file filtered, in file order
            idx_large_t at = 0;
            for (idx_large_t e = 0; e < W.nnz; ++e) {
                if (rp[W.ii[e]] != gx || cp[W.jj[e]] != gy)
                    continue;
                CHECK(at < Bk.nnz && Bk.ii[at] == W.ii[e] && Bk.jj[at] == W.jj[e] &&
                      Bk.vv[at] == W.vv[e]);
                CHECK(!seen[e]); // every entry lands in exactly one block
                seen[e] = 1;
                ++at;
            }
            CHECK(at == Bk.nnz);
            total += Bk.nnz;
            // what the drivers do next (miniapp/bench_both.cpp:158)
            const std::vector<idx_t> gi = Bk.ii, gj = Bk.jj;
            Bk.localizeIndices();
            for (idx_large_t e = 0; e < Bk.nnz; ++e)
                CHECK(Bk.ltgR[Bk.ii[e]] == gi[e] && Bk.ltgC[Bk.jj[e]] == gj[e]);
        }
    CHECK(total == W.nnz); // the union of the blocks is the file
    for (idx_large_t e = 0; e < W.nnz; ++e)
        CHECK(seen[e]);
}

static void test_blocks(const std::string &dir)
{
    for (const char *stem : {"general", "symmetric", "pattern_symmetric", "complex", "integer"})
        for (int X : {1, 2, 3})
            for (int Y : {1, 2})
                check_blocks(dir + "/" + stem + ".bin", X, Y, 1, 11);
    // a larger file with repeated entries, written by this build's converter
    const std::string big = "/tmp/spc3d_test_io_big.bin";
    cooMat G;
    G.gnrows = 1000;
    G.gncols = 700;
    unsigned long long x = 0x9E3779B97F4A7C15ull;
    for (int i = 0; i < 30000; ++i) {
        x ^= x << 13, x ^= x >> 7, x ^= x << 17;
        G.addEntry((idx_t)(x % 1000), (idx_t)((x >> 24) % 700), (real_t)((double)(x >> 40) / 1e6));
    }
    G.gnnz = G.nnz = 30000;
    convert_to_binary(G, big);
    check_blocks(big, 4, 4, 4, 1);
    check_blocks(big, 3, 5, 2, 2);
    check_blocks(big, 1, 1, 1, 3);
    // 1 x 1: the whole file, as read_binary gives it
    {
        cooMat A, B;
        std::vector<int> rp, cp;
        read_binary(big, A);
        read_binary_block(big, B, 1, 1, 0, 0, 5, rp, cp);
        CHECK(A.ii == B.ii && A.jj == B.jj && A.vv == B.vv && B.nnz == A.nnz && B.ownedNnz == A.nnz);
    }
    // the seed decides the partition, and nothing else does
    {
        cooMat A, B, C2;
        std::vector<int> rpa, cpa, rpb, cpb, rpc, cpc;
        read_binary_block(big, A, 4, 4, 1, 2, 77, rpa, cpa);
        read_binary_block(big, B, 4, 4, 1, 2, 77, rpb, cpb);
        read_binary_block(big, C2, 4, 4, 1, 2, 78, rpc, cpc);
        CHECK(rpa == rpb && cpa == cpb && A.ii == B.ii && A.jj == B.jj);
        CHECK(rpa != rpc && cpa != cpc);
    }
    // Z shares of the owned values: lnnz / Z each, the first lnnz mod Z ranks one more
    {
        idx_large_t owned = 0, lnnz = 0;
        for (int gz = 0; gz < 3; ++gz) {
            cooMat A;
            std::vector<int> rp, cp;
            read_binary_block(big, A, 2, 2, 0, 1, 9, rp, cp, 3, gz);
            lnnz = A.nnz;
            CHECK(A.ownedNnz == lnnz / 3 + ((idx_large_t)gz < lnnz % 3 ? 1 : 0));
            owned += A.ownedNnz;
        }
        CHECK(owned == lnnz);
    }
    bool threw = false;
    try {
        cooMat A;
        std::vector<int> rp, cp;
        read_binary_block(big, A, 2, 2, 2, 0, 1, rp, cp);
    } catch (const std::out_of_range &) {
        threw = true;
    }
    CHECK(threw);
    std::remove(big.c_str());
}

int main(int argc, char **argv)
{
    if (argc < 2) {
        std::printf("usage: test_io <golden dir>\n");
        return 2;
    }
    const std::string dir = argv[1];
    check_file(dir, "general", 9);
    check_file(dir, "symmetric", 12);        // mirrored, the two diagonal entries twice
    check_file(dir, "pattern_symmetric", 8); // values 1
    check_file(dir, "complex", 3);           // imaginary parts dropped
    check_file(dir, "integer", 2);
    test_blocks(dir);

    // content of one file, spelled out (src/mm.hpp:45-57 semantics)
    {
        cooMat M;
        mm reader(dir + "/symmetric.mtx");
        reader.read_mm(dir + "/symmetric.mtx", M);
        CHECK(M.gnrows == 5 && M.gncols == 5);
        const idx_t wi[] = {0, 1, 2, 3, 4, 4, 0, 0, 1, 3, 0, 3};
        const idx_t wj[] = {0, 0, 1, 3, 0, 3, 0, 1, 2, 3, 4, 4};
        const double wv[] = {2, -1, .5, 3, 1e10, -.125, 2, -1, .5, 3, 1e10, -.125};
        for (int i = 0; i < 12; ++i)
            CHECK(M.ii[i] == wi[i] && M.jj[i] == wj[i] && M.vv[i] == (real_t)wv[i]);
        cooMat P;
        mm r2(dir + "/pattern_symmetric.mtx");
        r2.read_mm(dir + "/pattern_symmetric.mtx", P);
        for (idx_large_t i = 0; i < P.nnz; ++i)
            CHECK(P.vv[i] == (real_t)1);
        CHECK(P.ii[3] == 3 && P.jj[3] == 3 && P.ii[7] == 3 && P.jj[7] == 3); // diagonal twice
    }
    // failures are reported, not swallowed
    bool threw = false;
    try {
        cooMat M;
        mm r(dir + "/does_not_exist.mtx");
        r.read_mm(dir + "/does_not_exist.mtx", M);
    } catch (const std::runtime_error &) {
        threw = true;
    }
    CHECK(threw);
    threw = false;
    try {
        cooMat R;
        const std::string cut = "/tmp/spc3d_test_io_cut.bin";
        std::vector<char> ref = slurp(dir + "/general.bin");
        std::ofstream(cut, std::ios::binary).write(ref.data(), 100);
        read_binary(cut, R);
    } catch (const std::runtime_error &) {
        threw = true;
    }
    CHECK(threw);
    // a header that promises 2^40 triplets is refused before anything is sized by it
    threw = false;
    try {
        cooMat R;
        const std::string lie = "/tmp/spc3d_test_io_lie.bin";
        std::vector<char> ref = slurp(dir + "/general.bin");
        const std::uint64_t huge = 1ull << 40;
        std::memcpy(&ref[8], &huge, 8);
        std::ofstream(lie, std::ios::binary).write(ref.data(), (std::streamsize)ref.size());
        read_binary(lie, R);
    } catch (const std::runtime_error &) {
        threw = true;
    }
    CHECK(threw);
    // the block-buffered number reader against formatted stream extraction, token by
    // token, on text with every kind of spacing and number spelling, read in blocks so
    // small that tokens straddle them
    {
        const std::string path = "/tmp/spc3d_test_io_tokens.txt";
        {
            std::ofstream o(path);
            o << "  12\t+7 \r\n\n3.25 -1e-3\t+2.5E+2 .5 7. 1.7976931348623157e308 4.9e-324\n";
            unsigned long long x = 88172645463325252ull;
            for (int i = 0; i < 5000; ++i) {
                x ^= x << 13, x ^= x >> 7, x ^= x << 17;
                char line[96];
                std::snprintf(line, sizeof line, "%llu %llu %.17g%s", x % 100000 + 1, (x >> 20) % 100000 + 1,
                              (double)(long long)(x >> 11) / 9007199254740992.0 - 0.5, i % 3 ? "\n" : " \r\n");
                o << line;
            }
        }
        for (std::size_t block : {(std::size_t)7, (std::size_t)64, (std::size_t)1000, (std::size_t)1 << 20}) {
            std::ifstream a(path), b(path);
            TokenReader tok(a, block);
            std::uint64_t u = 0, v = 0;
            double x = 0, y = 0;
            CHECK(tok.next(u) && (b >> v) && u == v && u == 12);
            CHECK(tok.next(u) && (b >> v) && u == v && u == 7);
            std::size_t n = 0;
            while (tok.next(x)) {
                if (!(b >> y))
                    break;
                if (std::memcmp(&x, &y, 8) != 0)
                    break;
                ++n;
            }
            CHECK(n == 7 + 3 * 5000);
            CHECK(!(b >> y)); // both at the end of the file
        }
        // what is no number is refused, not skipped
        {
            std::ofstream(path) << "12 abc 3";
            std::ifstream a(path);
            TokenReader tok(a);
            std::uint64_t u = 0;
            CHECK(tok.next(u) && u == 12);
            CHECK(!tok.next(u));
        }
        for (const char *word : {"inf", "-inf", "nan", "+Infinity", "NaN"}) {
            std::ofstream(path) << word << " 1";
            std::ifstream a(path), b(path);
            TokenReader tok(a);
            double x = 0, y = 0;
            CHECK(!tok.next(x) && !(b >> y)); // as stream extraction
        }
    }
    std::printf("%s (%d failures, real_t = %s)\n", g_fail ? "FAILED" : "PASSED", g_fail,
                sizeof(real_t) == 8 ? "double" : "float");
    return g_fail ? 1 : 0;
}
