"""CPU-only checks of the seeded workload generators."""
import numpy as np

from spcomm3d_amd import workloads as W


def test_splitmix64_published_vectors():
    # first outputs of SplitMix64 from state 1234567 (Vigna's reference implementation)
    want = [6457827717110365317, 3203168211198807973, 9817491932198370423,
            4593380528125082431, 16408922859458223821]
    assert [W.splitmix64(1234567, i) for i in range(5)] == want


def test_uniform_is_counter_based_and_in_range():
    a = W.uniform(3, 0, 1000, -1.0, 1.0, "f64")
    b = W.uniform(3, 0, 400, -1.0, 1.0, "f64", first=600)
    assert np.array_equal(a[600:], b)  # element i depends on (seed, stream, i) only
    assert a.min() >= -1.0 and a.max() < 1.0 and abs(a.mean()) < 0.1
    f = W.uniform(3, 0, 1000, -1.0, 1.0, "f32")
    assert f.dtype == np.float32 and np.array_equal(f, a.astype(np.float32))
    assert not np.array_equal(a, W.uniform(4, 0, 1000, -1.0, 1.0, "f64"))
    assert not np.array_equal(a, W.uniform(3, 1, 1000, -1.0, 1.0, "f64"))


def test_erdos_renyi_config_shape():
    w = W.erdos_renyi(16384, 16, 32)
    assert w.nnz == 262144 and w.nrows == w.ncols == 16384 and w.k == 32
    assert np.array_equal(np.bincount(w.ii), np.full(16384, 16))
    key = w.ii.astype(np.uint64) << np.uint64(32) | w.jj
    assert np.unique(key).size == w.nnz  # distinct columns per row
    assert w.jj.max() < 16384 and 0 <= w.vv64.min() and w.vv64.max() < 1
    w2 = W.erdos_renyi(16384, 16, 32)
    assert np.array_equal(w.jj, w2.jj) and np.array_equal(w.vv64, w2.vv64)


def test_rmat_small_is_sorted_unique_and_skewed():
    w = W.rmat(12, 16, 64)
    n = 1 << 12
    key = w.ii.astype(np.uint64) << np.uint64(32) | w.jj
    assert np.all(np.diff(key.astype(np.int64)) > 0)
    assert w.nnz <= 16 * n and w.nnz > 8 * n
    # quadrant mass of the top level follows (a, b, c, d) = (.57, .19, .19, .05) before
    # dedup; after dedup the dense top-left corner loses most, so only order is checked
    top = (w.ii >= n // 2).astype(int) * 2 + (w.jj >= n // 2)
    q = np.bincount(top, minlength=4) / w.nnz
    assert q[0] > q[1] > q[3] and q[0] > q[2] > q[3] and abs(q[1] - q[2]) < 0.03
    assert np.bincount(w.ii).max() > 50 * (w.nnz / n)  # hub rows


def test_rmat_raw_quadrant_probabilities():
    import ctypes
    lib = W._load()
    ne = 400000
    r = np.empty(ne, np.uint32)
    c = np.empty(ne, np.uint32)
    assert lib.spc3d_gen_rmat_edges(1, 10, ne, 0.57, 0.19, 0.19, r.ctypes.data_as(ctypes.c_void_p),
                                    c.ctypes.data_as(ctypes.c_void_p)) == 0
    for bit in (9, 4, 0):  # every level uses the same quadrant law
        q = np.bincount(((r >> bit) & 1) * 2 + ((c >> bit) & 1), minlength=4) / ne
        assert np.allclose(q, [0.57, 0.19, 0.19, 0.05], atol=0.004)


def test_shuffled_is_the_same_matrix():
    w = W.rmat(10, 8, 16)
    s = w.shuffled()
    assert s.order == "shuffled" and not np.array_equal(s.ii, w.ii)
    k1 = np.sort(w.ii.astype(np.uint64) << np.uint64(32) | w.jj)
    o = np.argsort(s.ii.astype(np.uint64) << np.uint64(32) | s.jj)
    assert np.array_equal(k1, (s.ii.astype(np.uint64) << np.uint64(32) | s.jj)[o])
    assert np.array_equal(w.vv64, s.vv64[o])


def test_rmat_block_small():
    w = W.rmat_block(14, 16, 64, 4, 4, 0, 0)
    assert w.nrows == w.ncols == (1 << 14) // 4
    assert w.ii.max() < w.nrows and w.jj.max() < w.ncols
    full = W.rmat(14, 16, 64)
    assert 0.03 < w.nnz / full.nnz < 0.11  # about 1/16 of the edges, more after dedup


def test_stencil_counts_and_values():
    w = W.stencil5(64, 48, 32)
    assert w.nnz == 5 * 64 * 48 - 2 * 64 - 2 * 48
    diag = w.ii == w.jj
    assert np.all(w.vv64[diag] == 1.0) and np.all(w.vv64[~diag] == -0.25)
    d = np.abs(w.ii.astype(np.int64) - w.jj.astype(np.int64))
    assert set(np.unique(d)) == {0, 1, 64}
    # no wrap-around across grid rows
    x = w.ii % 64
    assert not np.any((x == 0) & (w.jj.astype(np.int64) == w.ii.astype(np.int64) - 1))
    assert 5 * 4096 * 4096 - 4 * 4096 == 83869696


def test_hypergraph_zipf_capped():
    w = W.hypergraph_zipf(40000, 10000, 128)
    deg = np.bincount(w.ii, minlength=40000)
    assert deg.min() >= 1 and deg.max() == 1024
    assert 240 < deg.mean() < 330  # E[min(Zipf(1.2), 1024)] is about 286
    assert abs((deg == 1).mean() - 1 / 5.5916) < 0.01  # P(1) = 1/zeta(1.2)
    r = 12345
    cols = w.jj[w.ii == r]
    assert np.unique(cols).size == cols.size
