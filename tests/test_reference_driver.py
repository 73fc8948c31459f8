"""The reference's own sequential checker (miniapp/numCheckSeq.cpp: read a
MatrixMarket file, fill A and B with i/1000, run SpKernels::sddmm, print the sum
of C), built twice by `make -C oracle ref`: entirely from the reference's sources
(oracle/_ref/numCheckSeq_ref), and with the binding this library documents for a
maintainer of the reference (oracle/ref_binding/core_ops_hip.cpp) over the GPU library
in place of the reference's core_ops.cpp (oracle/_ref/numCheckSeq_hip).
Same program, same arguments: the printed numbers must be the same."""
import os
import re
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = os.path.join(ROOT, "oracle", "_ref", "numCheckSeq_ref")
HIP = os.path.join(ROOT, "oracle", "_ref", "numCheckSeq_hip")
IO = os.path.join(ROOT, "tests", "golden", "io")
needs_builds = pytest.mark.skipif(not (os.path.exists(REF) and os.path.exists(HIP)),
                                  reason="oracle/_ref is only built where the reference is mounted")


def run(binary, k, path):
    r = subprocess.run([binary, "-k", str(k), path], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    return r.stdout.strip()


def test_binding_file_is_the_one_documented():
    doc = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    snippet = re.search(r'```cpp\n(#include "SparseMatrix.hpp".*?)```', doc, re.S).group(1)
    src = open(os.path.join(ROOT, "oracle", "ref_binding", "core_ops_hip.cpp")).read()
    assert src.endswith(snippet)


@needs_builds
def test_reference_driver_prints_the_closed_form():
    # general.mtx: 9 entries (r, c, v), 1-based in the file; C_e = v * k * r * c / 10^6
    rows = [ln.split() for ln in open(os.path.join(IO, "general.mtx")) if ln[0] not in "%\n"][1:]
    want = sum(float(v) * 4 * (int(r) - 1) * (int(c) - 1) / 1e6 for r, c, v in rows)
    got = float(run(REF, 4, os.path.join(IO, "general.mtx")))
    assert abs(got - want) <= 1e-5 * abs(want)  # the driver prints 6 significant digits


@pytest.mark.gpu
@needs_builds
@pytest.mark.parametrize("name", ["general", "symmetric", "integer", "pattern_symmetric"])
@pytest.mark.parametrize("k", [4, 64])
def test_gpu_build_of_the_reference_driver_prints_the_same(name, k):
    path = os.path.join(IO, name + ".mtx")
    assert run(HIP, k, path) == run(REF, k, path)


@pytest.mark.gpu
@needs_builds
@pytest.mark.parametrize("k", [20, 64])
def test_gpu_build_of_the_reference_driver_on_a_generated_matrix(tmp_path, k):
    rng = np.random.default_rng(7)
    m, n, nnz = 20000, 15000, 200000
    ii = np.minimum(rng.pareto(0.8, nnz).astype(np.int64), m - 1) + 1  # skewed: hub rows
    jj = rng.integers(1, n + 1, nnz)
    vv = rng.uniform(0.5, 1.5, nnz)
    path = tmp_path / "generated.mtx"
    with open(path, "w") as f:
        f.write("%%MatrixMarket matrix coordinate real general\n")
        f.write(f"{m} {n} {nnz}\n")
        for r, c, v in zip(ii, jj, vv):
            f.write(f"{r} {c} {v:.17g}\n")
    assert run(HIP, k, str(path)) == run(REF, k, str(path))
