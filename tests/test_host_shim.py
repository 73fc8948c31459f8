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


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["test_shim_f64", "test_shim_f32"])
def test_shim_on_gpu(name):
    _run(name)
