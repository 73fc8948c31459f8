"""Seeded synthetic workloads for the local SDDMM / SpMM path.

The reference ships no input matrices and no reproducible generator
(``COOMatrix::self_generate_random`` seeds from the clock,
``src/SparseMatrix.hpp:49-67``; its benches read SuiteSparse files converted
by ``tools/read_convert_mm.cpp``).  Everything here is synthetic and a pure
function of the seeds, produced by the counter-based generators in
``gen/spc3d_gen.c``.

Fixed streams: pattern seed 1, sparse values seed 2, A seed 3, B/X seed 4,
Y0 seed 5, presentation-order shuffle seed 6, partition permutations seed 7/8.

Each workload is a :class:`Workload`: unsorted-or-sorted COO ``ii, jj, vv``
(``uint32`` indices as in ``src/basic.hpp:16``), the panel shapes and K.
Dense panels are generated separately with :func:`dense_panel` so that large
configurations do not hold fp32 and fp64 copies at once.
"""
from __future__ import annotations

import ctypes
import os
from dataclasses import dataclass, field

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "gen", "libspc3d_gen.so")
_lib = None

SEED_PATTERN, SEED_VALUES, SEED_A, SEED_B, SEED_Y0, SEED_ORDER = 1, 2, 3, 4, 5, 6
SEED_PERM_R, SEED_PERM_C = 7, 8

_u64, _u32, _i32, _f64 = ctypes.c_uint64, ctypes.c_uint32, ctypes.c_int, ctypes.c_double
_vp = ctypes.c_void_p


def _load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise RuntimeError(
            f"{_LIB_PATH} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
            "or `make -C spcomm3d_amd/gen`")
    lib = ctypes.CDLL(_LIB_PATH)
    lib.spc3d_gen_splitmix64.restype = _u64
    lib.spc3d_gen_splitmix64.argtypes = [_u64, _u64]
    lib.spc3d_gen_stream_key.restype = _u64
    lib.spc3d_gen_stream_key.argtypes = [_u64, _u64]
    lib.spc3d_gen_uniform.restype = _i32
    lib.spc3d_gen_uniform.argtypes = [_u64, _u64, _u64, _u64, _f64, _f64, _i32, _vp]
    lib.spc3d_gen_keys.restype = _i32
    lib.spc3d_gen_keys.argtypes = [_u64, _u64, _u64, _vp]
    lib.spc3d_gen_rmat_edges.restype = _i32
    lib.spc3d_gen_rmat_edges.argtypes = [_u64, _i32, _u64, _f64, _f64, _f64, _vp, _vp]
    lib.spc3d_gen_rmat_block.restype = ctypes.c_int64
    lib.spc3d_gen_rmat_block.argtypes = [_u64, _i32, _u64, _f64, _f64, _f64, _vp, _vp,
                                         _u32, _u32, _u32, _u32, _vp, _vp, _u64]
    lib.spc3d_gen_zipf_capped.restype = _i32
    lib.spc3d_gen_zipf_capped.argtypes = [_u64, _u64, _u64, _f64, _u32, _vp]
    lib.spc3d_gen_distinct_cols.restype = _i32
    lib.spc3d_gen_distinct_cols.argtypes = [_u64, _u64, _u32, _vp, _vp]
    _lib = lib
    return lib


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(_vp)


def np_dtype(dtype) -> np.dtype:
    """Map 'f32'/'f64'/numpy dtypes to a numpy dtype."""
    if isinstance(dtype, str):
        return np.dtype({"f32": np.float32, "f64": np.float64,
                         "float32": np.float32, "float64": np.float64}[dtype])
    return np.dtype(dtype)


def splitmix64(state0: int, i: int) -> int:
    return int(_load().spc3d_gen_splitmix64(state0, i))


def uniform(seed: int, stream: int, count: int, lo: float, hi: float, dtype="f64",
            first: int = 0) -> np.ndarray:
    """``count`` values U[lo,hi): element i is a function of (seed, stream, first+i)."""
    dt = np_dtype(dtype)
    out = np.empty(count, dtype=dt)
    rc = _load().spc3d_gen_uniform(seed, stream, first, count, lo, hi,
                                   1 if dt == np.float64 else 0, _ptr(out))
    if rc != 0:
        raise ValueError("spc3d_gen_uniform failed")
    return out


def dense_panel(rows: int, k: int, seed: int, dtype="f64") -> np.ndarray:
    """Row-major ``rows x k`` panel, U[-1,1) (``src/basic.hpp:30-36`` layout)."""
    return uniform(seed, 0, rows * k, -1.0, 1.0, dtype).reshape(rows, k)


def sparse_values(nnz: int, dtype="f64", seed: int = SEED_VALUES) -> np.ndarray:
    """U[0,1) values; entry e of the canonical (row-major sorted) order gets value e."""
    return uniform(seed, 0, nnz, 0.0, 1.0, dtype)


def hashed_permutation(seed: int, stream: int, n: int) -> np.ndarray:
    """Permutation of range(n): argsort of per-index hash keys (stable)."""
    keys = np.empty(n, dtype=np.uint64)
    _load().spc3d_gen_keys(seed, stream, n, _ptr(keys))
    return np.argsort(keys, kind="stable")


@dataclass
class Workload:
    name: str
    nrows: int            # A / Y panel height (S rows)
    ncols: int            # B / X panel height (S cols)
    k: int
    ii: np.ndarray        # uint32 [nnz]
    jj: np.ndarray        # uint32 [nnz]
    vv64: np.ndarray      # float64 [nnz]; cast for fp32 runs
    order: str = "sorted"  # 'sorted' (row-major) or 'shuffled'
    notes: dict = field(default_factory=dict)

    @property
    def nnz(self) -> int:
        return int(self.ii.shape[0])

    def values(self, dtype="f64") -> np.ndarray:
        return np.ascontiguousarray(self.vv64.astype(np_dtype(dtype), copy=False))

    def panel_A(self, dtype="f64") -> np.ndarray:
        return dense_panel(self.nrows, self.k, SEED_A, dtype)

    def panel_B(self, dtype="f64") -> np.ndarray:
        return dense_panel(self.ncols, self.k, SEED_B, dtype)

    def panel_Y0(self, dtype="f64") -> np.ndarray:
        return dense_panel(self.nrows, self.k, SEED_Y0, dtype)

    def touched(self):
        """(#rows with a nonzero, #cols with a nonzero)."""
        if "touched" not in self.notes:
            mt = int(np.count_nonzero(np.bincount(self.ii, minlength=self.nrows)))
            nt = int(np.count_nonzero(np.bincount(self.jj, minlength=self.ncols)))
            self.notes["touched"] = (mt, nt)
        return self.notes["touched"]

    def shuffled(self, seed: int = SEED_ORDER) -> "Workload":
        """Same matrix, entries presented in a seeded random order (the
        reference never sorts its COO stream: file / Alltoallv order)."""
        p = hashed_permutation(seed, 0, self.nnz)
        return Workload(self.name, self.nrows, self.ncols, self.k,
                        np.ascontiguousarray(self.ii[p]), np.ascontiguousarray(self.jj[p]),
                        np.ascontiguousarray(self.vv64[p]), "shuffled", dict(self.notes))

    def localized(self) -> "Workload":
        """Same entries with the local indices ``COOMatrix::localizeIndices`` gives them
        (src/SparseMatrix.hpp:69-99): every row (column) that holds an entry gets the next
        id the first time it appears in the entry stream, and the panels shrink to the
        touched rows and columns, which is the shape a rank of the reference runs its
        kernels on (miniapp/bench_both.cpp:158,189-190)."""
        def first_appearance(idx):
            u, first, inv = np.unique(idx, return_index=True, return_inverse=True)
            rank = np.empty(u.size, dtype=np.uint32)
            rank[np.argsort(first, kind="stable")] = np.arange(u.size, dtype=np.uint32)
            return np.ascontiguousarray(rank[inv]), int(u.size)
        li, m = first_appearance(self.ii)
        lj, n = first_appearance(self.jj)
        w = Workload(self.name + "_localized", m, n, self.k, li, lj, self.vv64, self.order,
                     dict(self.notes))
        w.notes["touched"] = (m, n)
        w.notes["global_shape"] = (self.nrows, self.ncols)
        return w

    def column_major(self) -> "Workload":
        """Same matrix, entries sorted by column and by row inside a column: the order
        of a MatrixMarket file, which the reference's converter and readers keep
        (tools/read_convert_mm.cpp:81-94, src/parallel_io.hpp:132-190)."""
        p = np.lexsort((self.ii, self.jj))
        return Workload(self.name, self.nrows, self.ncols, self.k,
                        np.ascontiguousarray(self.ii[p]), np.ascontiguousarray(self.jj[p]),
                        np.ascontiguousarray(self.vv64[p]), "column-major", dict(self.notes))


def _sort_unique(rows: np.ndarray, cols: np.ndarray):
    key = (rows.astype(np.uint64) << np.uint64(32)) | cols.astype(np.uint64)
    key = np.unique(key)
    return ((key >> np.uint64(32)).astype(np.uint32),
            (key & np.uint64(0xFFFFFFFF)).astype(np.uint32))


def erdos_renyi(n: int = 16384, deg: int = 16, k: int = 32, seed: int = SEED_PATTERN) -> Workload:
    """``n x n``, ``deg`` distinct uniform columns in every row, values U[0,1)."""
    rowptr = np.arange(n + 1, dtype=np.uint64) * np.uint64(deg)
    cols = np.empty(n * deg, dtype=np.uint32)
    if _load().spc3d_gen_distinct_cols(seed, n, n, _ptr(rowptr), _ptr(cols)) != 0:
        raise ValueError("distinct column generation failed")
    rows = np.repeat(np.arange(n, dtype=np.uint32), deg)
    return Workload(f"er{n}_d{deg}", n, n, k, rows, cols, sparse_values(n * deg))


def rmat(scale: int = 20, edge_factor: int = 16, k: int = 64, a=0.57, b=0.19, c=0.19,
         seed: int = SEED_PATTERN) -> Workload:
    """R-MAT, ``edge_factor * 2**scale`` draws, duplicates removed, no vertex
    scrambling; canonical order is row-major sorted; values by unique-edge rank."""
    n = 1 << scale
    ne = edge_factor * n
    rows = np.empty(ne, dtype=np.uint32)
    cols = np.empty(ne, dtype=np.uint32)
    if _load().spc3d_gen_rmat_edges(seed, scale, ne, a, b, c, _ptr(rows), _ptr(cols)) != 0:
        raise ValueError("rmat generation failed")
    ii, jj = _sort_unique(rows, cols)
    w = Workload(f"rmat{scale}_ef{edge_factor}", n, n, k, ii, jj, sparse_values(ii.shape[0]))
    w.notes["edge_draws"] = ne
    return w


def rmat_block(scale: int = 24, edge_factor: int = 16, k: int = 64, px: int = 4, py: int = 4,
               gx: int = 0, gy: int = 0, a=0.57, b=0.19, c=0.19,
               seed: int = SEED_PATTERN) -> Workload:
    """Block (gx, gy) of a ``px x py`` 2D partition of an R-MAT graph, made with
    the reference's random-permutation round-robin rule
    (``src/parallel_io.hpp:64-76``).  Local shape ``2**scale/px x 2**scale/py``
    (the slice shape; ``localizeIndices`` would shrink it to the touched rows)."""
    n = 1 << scale
    ne = edge_factor * n
    perm_r = hashed_permutation(SEED_PERM_R, 0, n)
    pos_r = np.empty(n, dtype=np.uint32)
    pos_r[perm_r] = np.arange(n, dtype=np.uint32)
    del perm_r
    perm_c = hashed_permutation(SEED_PERM_C, 0, n)
    pos_c = np.empty(n, dtype=np.uint32)
    pos_c[perm_c] = np.arange(n, dtype=np.uint32)
    del perm_c
    lib = _load()
    cnt = lib.spc3d_gen_rmat_block(seed, scale, ne, a, b, c, _ptr(pos_r), _ptr(pos_c),
                                   px, py, gx, gy, None, None, 0)
    if cnt < 0:
        raise ValueError("rmat block generation failed")
    rows = np.empty(cnt, dtype=np.uint32)
    cols = np.empty(cnt, dtype=np.uint32)
    got = lib.spc3d_gen_rmat_block(seed, scale, ne, a, b, c, _ptr(pos_r), _ptr(pos_c),
                                   px, py, gx, gy, _ptr(rows), _ptr(cols), cnt)
    if got != cnt:
        raise ValueError("rmat block generation failed")
    ii, jj = _sort_unique(rows, cols)
    w = Workload(f"rmat{scale}_blk{px}x{py}_{gx}{gy}", (n + px - 1) // px, (n + py - 1) // py,
                 k, ii, jj, sparse_values(ii.shape[0]))
    w.notes["kept_edge_draws"] = int(cnt)
    return w


def stencil5(nx: int = 4096, ny: int = 4096, k: int = 32) -> Workload:
    """5-point stencil on an ``nx x ny`` grid: row p = y*nx + x, diagonal 1.0,
    existing N/S/E/W neighbours -0.25.  Row-major sorted, columns ascending."""
    n = nx * ny
    p = np.arange(n, dtype=np.int64)
    x = p % nx
    y = p // nx
    cand = [(-nx, y > 0, -0.25), (-1, x > 0, -0.25), (0, np.ones(n, bool), 1.0),
            (1, x < nx - 1, -0.25), (nx, y < ny - 1, -0.25)]
    cnt = np.zeros(n, dtype=np.int64)
    for _, ok, _v in cand:
        cnt += ok
    rowptr = np.zeros(n + 1, dtype=np.int64)
    np.cumsum(cnt, out=rowptr[1:])
    nnz = int(rowptr[-1])
    ii = np.empty(nnz, dtype=np.uint32)
    jj = np.empty(nnz, dtype=np.uint32)
    vv = np.empty(nnz, dtype=np.float64)
    fill = rowptr[:-1].copy()
    for off, ok, v in cand:
        dst = fill[ok]
        ii[dst] = p[ok]
        jj[dst] = p[ok] + off
        vv[dst] = v
        fill[ok] += 1
    return Workload(f"stencil5_{nx}x{ny}", n, n, k, ii, jj, vv)


def hypergraph_zipf(nrows: int = 2_000_000, ncols: int = 500_000, k: int = 128, s: float = 1.2,
                    cap: int = 1024, seed: int = SEED_PATTERN) -> Workload:
    """Incidence matrix: pins per row = min(Zipf(s), cap) (the literal "capped"
    reading: the tail mass lands on ``cap``), distinct uniform columns per row in
    draw order, values U[0,1)."""
    lib = _load()
    deg = np.empty(nrows, dtype=np.uint32)
    if lib.spc3d_gen_zipf_capped(seed, 1, nrows, s, cap, _ptr(deg)) != 0:
        raise ValueError("zipf generation failed")
    rowptr = np.zeros(nrows + 1, dtype=np.uint64)
    np.cumsum(deg, out=rowptr[1:], dtype=np.uint64)
    nnz = int(rowptr[-1])
    cols = np.empty(nnz, dtype=np.uint32)
    if lib.spc3d_gen_distinct_cols(seed, nrows, ncols, _ptr(rowptr), _ptr(cols)) != 0:
        raise ValueError("distinct column generation failed")
    rows = np.repeat(np.arange(nrows, dtype=np.uint32), deg)
    w = Workload(f"hyper{nrows}x{ncols}_zipf{s}_cap{cap}", nrows, ncols, k, rows, cols,
                 sparse_values(nnz))
    w.notes["zipf_reading"] = "capped (min(Zipf, cap))"
    return w


# The five benchmark configurations, by the names bench.py and the tests use.
CONFIGS = {
    "er16k": lambda **kw: erdos_renyi(16384, 16, 32, **kw),
    "rmat20": lambda **kw: rmat(20, 16, 64, **kw),
    "rmat24_block": lambda **kw: rmat_block(24, 16, 64, 4, 4, 0, 0, **kw),
    "stencil4096": lambda **kw: stencil5(4096, 4096, 32),
    "hypergraph": lambda **kw: hypergraph_zipf(2_000_000, 500_000, 128, 1.2, 1024, **kw),
}


def make(name: str, **kw) -> Workload:
    return CONFIGS[name](**kw)
