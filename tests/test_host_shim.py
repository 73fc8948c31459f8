"""Runs the C++ tests of the host shim (tests/cpp/test_shim.cpp): the reference's
call surface (denseMatrix, cooMat, SpKernels::sddmm / spmm, the dist_* wrappers)
over the GPU library, for real_t = double and float."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CPP = os.path.join(ROOT, "tests", "cpp")


def _binary(name):
    path = os.path.join(CPP, name)
    if not os.path.exists(path):
        subprocess.run(["make", "-C", os.path.join(ROOT, "spcomm3d_amd", "host")], check=True,
                       capture_output=True)
        subprocess.run(["make", "-C", CPP, name], check=True, capture_output=True)
    return path


def _run(name, *args):
    r = subprocess.run([_binary(name), *args], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "PASSED" in r.stdout, r.stdout[-3000:] + r.stderr[-3000:]


@pytest.mark.parametrize("name", ["test_shim_f64", "test_shim_f32"])
def test_host_types_index_transforms_and_errors(name):
    _run(name, "--host")


@pytest.mark.parametrize("name", ["test_io_f64", "test_io_f32"])
def test_matrixmarket_and_binary_io_against_reference_files(name):
    # tests/golden/io/*.bin were written by the reference's own converter
    _run(name, os.path.join(ROOT, "tests", "golden", "io"))


def test_binary_file_layout_with_numpy():
    # uint32 rows, uint32 cols, uint64 nnz, then nnz x {uint32, uint32, float64}
    # (tools/read_convert_mm.cpp:81-94): checked on the reference-written file
    import numpy as np

    raw = open(os.path.join(ROOT, "tests", "golden", "io", "general.bin"), "rb").read()
    rows, cols = np.frombuffer(raw, dtype="<u4", count=2)
    nnz = int(np.frombuffer(raw, dtype="<u8", count=1, offset=8)[0])
    assert (rows, cols, nnz) == (6, 5, 9) and len(raw) == 16 + 16 * nnz
    t = np.frombuffer(raw, dtype=np.dtype([("r", "<u4"), ("c", "<u4"), ("v", "<f8")]), offset=16)
    assert t["r"].tolist() == [0, 1, 1, 2, 3, 4, 5, 5, 2]
    assert t["c"].tolist() == [1, 0, 4, 2, 3, 1, 0, 4, 2]
    assert t["v"].tolist() == [1.5, -2.25, 3.0, 4.125, 5e-3, 6.0, 7.0, -8.5, 9.0]


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["test_shim_f64", "test_shim_f32"])
def test_shim_on_gpu(name):
    _run(name)


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["test_dist_resident_f64", "test_dist_resident_f32"])
def test_dist_wrappers_over_device_resident_operands(name):
    # the six wrappers over panels, plan, values and exchange buffers that stay on the device,
    # with self-addressed exchanges so that the pack / unpack / sum-unpack kernels run
    # (src/distributed_comp.cpp:17-76,141-236, src/comm.hpp:90-103,166-189): bit-equal to
    # the host-memory wrappers, both against the oracle
    _run(name)


def _mpi_env():
    """Environment in which a program linked with the image's MPI library starts: the
    system's libstdc++ ahead of the MPI library's own directory."""
    env = dict(os.environ)
    env["LD_LIBRARY_PATH"] = "/usr/lib/x86_64-linux-gnu:/opt/conda/lib:" + env.get("LD_LIBRARY_PATH", "")
    return env


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["test_dist_mpi_f64", "test_dist_mpi_f32"])
def test_dist_wrappers_under_the_reference_signatures(name):
    # void dist_*(..., MPI_Comm) on a 1 x 1 x 1 Cartesian communicator
    # (src/distributed_comp.hpp:11-64); built only where the image has an MPI
    path = os.path.join(CPP, name)
    if not os.path.exists(path):
        pytest.skip("no MPI installation where the tests were built")
    r = subprocess.run([path], capture_output=True, text=True, timeout=300, env=_mpi_env())
    if r.returncode == 127 or "error while loading shared libraries" in r.stderr:
        pytest.skip("the MPI library the test was linked with does not load here: " + r.stderr[-300:])
    assert r.returncode == 0 and "PASSED" in r.stdout, r.stdout[-3000:] + r.stderr[-3000:]


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["test_file_gpu_f64", "test_file_gpu_f32"])
@pytest.mark.parametrize("k", [4, 64])
def test_files_through_this_builds_readers_onto_the_gpu(name, k):
    # .mtx / .bin -> spc3d/io.hpp -> (2D block of a mesh) -> localizeIndices -> SDDMM + SpMM on
    # the GPU -> oracle; and, for the reference's real type, the printed SDDMM sum against
    # what the reference's own sequential checker prints for the same file
    io = os.path.join(ROOT, "tests", "golden", "io")
    r = subprocess.run([_binary(name), io, str(k)], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "PASSED" in r.stdout, r.stdout[-3000:] + r.stderr[-3000:]
    sums = {ln.split()[1]: ln.split()[2] for ln in r.stdout.splitlines() if ln.startswith("SUM ")}
    assert set(sums) == {"general", "symmetric", "integer", "pattern_symmetric", "complex"}
    ref = os.path.join(ROOT, "oracle", "_ref", "numCheckSeq_ref")
    if name.endswith("f64") and os.path.exists(ref):
        for stem, got in sums.items():
            want = subprocess.run([ref, "-k", str(k), os.path.join(io, stem + ".mtx")],
                                  capture_output=True, text=True, timeout=60)
            assert want.returncode == 0 and got == want.stdout.strip(), (stem, got, want.stdout)


@pytest.mark.gpu
@pytest.mark.parametrize("threads", [None, "8"])
def test_one_shot_host_calls_reuse_only_what_still_holds(threads):
    # spc3d_sddmm_host / spc3d_spmm_host called five times over one pattern as the reference's
    # drivers call the kernels (miniapp/bench_both.cpp:202-203), then with every operand
    # changed in the smallest way: plan and panels are reused by content, results against the oracle
    # once on the caller's thread alone (the default: one thread per rank, as the reference's
    # ranks run), once with eight host threads reading the operands and moving Y
    env = dict(os.environ)
    env.pop("SPC3D_HOST_THREADS", None)
    if threads:
        env["SPC3D_HOST_THREADS"] = threads
    r = subprocess.run([_binary("test_host_calls")], capture_output=True, text=True, timeout=600,
                       env=env)
    assert r.returncode == 0 and "PASSED" in r.stdout, r.stdout[-3000:] + r.stderr[-3000:]
    print("\n".join(ln for ln in r.stdout.splitlines() if ln.startswith("TIMING")))


def test_content_keys_of_the_one_shot_host_calls():
    # what decides whether a plan or a device panel is reused: every byte, the order of the
    # words and the length go into a key; any number of threads gives the same keys
    _run("test_keys")


@pytest.mark.gpu
def test_shim_without_the_cache_of_the_one_shot_calls():
    # SPC3D_HOST_CACHE=0: plan, upload, run, download, free on every call; same results
    env = dict(os.environ, SPC3D_HOST_CACHE="0")
    r = subprocess.run([_binary("test_shim_f64")], capture_output=True, text=True, timeout=300, env=env)
    assert r.returncode == 0 and "PASSED" in r.stdout, r.stdout[-3000:] + r.stderr[-3000:]
