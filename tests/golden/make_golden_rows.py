"""Writes tests/golden/rows_golden.npz: inputs and expected outputs of the
reference's own SparseComm::copy_to_sendbuff / copy_from_recvbuff /
SUM_from_recvbuff (src/comm.hpp:90-103,166-189).

Run in the build container only (needs oracle/_ref/libref_rows.so, which
`make -C oracle ref` compiles from the reference's comm.hpp):

    python tests/golden/make_golden_rows.py

The file holds data only (numpy arrays, loaded with allow_pickle=False).
"""
import ctypes
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
LIB = os.path.join(ROOT, "oracle", "_ref", "libref_rows.so")
OUT = os.path.join(HERE, "rows_golden.npz")


def ref_rows(lib, op, panel, rows, buf):
    panel, buf = panel.copy(), buf.copy()
    vp = lambda a: a.ctypes.data_as(ctypes.c_void_p)  # noqa: E731
    rc = lib.ref_rows_f64(op, panel.shape[0], panel.shape[1], vp(panel), rows.size, vp(rows),
                          vp(buf))
    assert rc == 0
    return panel, buf


def main():
    lib = ctypes.CDLL(LIB)
    lib.ref_rows_f64.restype = ctypes.c_int
    lib.ref_rows_f64.argtypes = [ctypes.c_int, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_void_p,
                                 ctypes.c_uint64, ctypes.c_void_p, ctypes.c_void_p]
    rng = np.random.default_rng(20240611)
    out = {}
    for name, m, k, n in (("k1", 30, 1, 80), ("k6", 40, 6, 100), ("k64", 25, 64, 60)):
        P = rng.uniform(-1, 1, (m, k))
        rows = rng.integers(0, m, n).astype(np.uint32)  # with repeats
        buf = rng.uniform(-1, 1, (n, k))
        out[f"{name}.P"], out[f"{name}.rows"], out[f"{name}.buf"] = P, rows, buf
        out[f"{name}.packed"] = ref_rows(lib, 0, P, rows, buf)[1]
        out[f"{name}.unpacked"] = ref_rows(lib, 1, P, rows, buf)[0]
        out[f"{name}.summed"] = ref_rows(lib, 2, P, rows, buf)[0]
    np.savez_compressed(OUT, **out)
    print("wrote", OUT, {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
