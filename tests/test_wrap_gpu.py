"""Panels and value vectors over the caller's own device memory (spc3d_panel_wrap,
spc3d_vals_wrap): the kernels must give what they give on panels the library
allocated, bit for bit, including on a block of rows inside a larger panel."""
import numpy as np
import pytest

from spcomm3d_amd import _capi as capi
from spcomm3d_amd import device
from spcomm3d_amd import workloads as W

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_block_of_rows_inside_a_larger_panel(ctx, dtype):
    w = W.rmat(13, 16, 64).shuffled()
    vv = w.values(dtype)
    A, B, Y0 = w.panel_A(dtype), w.panel_B(dtype), w.panel_Y0(dtype)
    S = ctx.plan(w.nrows, w.ncols, w.ii, w.jj, vv, seg_max=64)
    # reference run on the library's own panels
    dA, dB, dY = ctx.panel_from(A), ctx.panel_from(B), ctx.panel_from(Y0)
    dC = ctx.vals(w.nnz, dtype)
    ctx.sddmm(S, dA, dB, dC)
    ctx.spmm(S, dB, dY)
    C_want, Y_want = dC.download(), dY.download()
    # the same operands as blocks of rows of taller panels, and C inside a longer vector
    pad = 37
    item = np.dtype(dtype).itemsize
    bigA = ctx.panel_from(np.vstack([np.full((pad, w.k), np.nan, dtype), A]))
    bigB = ctx.panel_from(np.vstack([np.full((pad, w.k), np.nan, dtype), B,
                                     np.full((5, w.k), np.nan, dtype)]))
    bigY = ctx.panel_from(np.vstack([np.full((pad, w.k), 7.0, dtype), Y0]))
    bigC = ctx.vals(w.nnz + 64, dtype)
    bigC.fill(-1.0)
    off = pad * w.k * item
    vA = device.Panel(ctx, w.nrows, w.k, dtype, dev=bigA.device_ptr() + off)
    vB = device.Panel(ctx, w.ncols, w.k, dtype, dev=bigB.device_ptr() + off)
    vY = device.Panel(ctx, w.nrows, w.k, dtype, dev=bigY.device_ptr() + off)
    vC = device.Vals(ctx, w.nnz, dtype, dev=bigC.device_ptr() + 32 * item)
    ctx.sddmm(S, vA, vB, vC)
    ctx.spmm(S, vB, vY)
    assert np.array_equal(vC.download(), C_want)
    assert np.array_equal(vY.download(), Y_want)
    # nothing outside the views was written
    full = bigC.download()
    assert np.all(full[:32] == -1.0) and np.all(full[32 + w.nnz:] == -1.0)
    assert np.array_equal(full[32:32 + w.nnz], C_want)
    assert np.all(bigY.download()[:pad] == 7.0)
    # destroying a view leaves the memory to its owner
    for h in (vA, vB, vY, vC):
        h.close()
    assert np.array_equal(bigY.download()[pad:], Y_want)
    for h in (S, dA, dB, dY, dC, bigA, bigB, bigY, bigC):
        h.close()


def test_wrap_refuses_what_is_not_device_memory_of_this_gpu(ctx):
    host = np.zeros(1024, dtype=np.float32)
    with pytest.raises(capi.Spc3dError):
        device.Panel(ctx, 16, 64, np.float32, dev=host.ctypes.data)
    good = ctx.panel(16, 64, np.float32)
    with pytest.raises(capi.Spc3dError):
        device.Panel(ctx, 15, 64, np.float32, dev=good.device_ptr() + 4)  # not 16-byte aligned
    with pytest.raises(capi.Spc3dError):
        device.Vals(ctx, 10, np.float32, dev=0)
    empty = device.Vals(ctx, 0, np.float32, dev=0)  # nothing to point at
    empty.close()
    good.close()


def test_overlapping_row_blocks_are_refused_as_aliases(ctx):
    """X and Y as two row blocks of one tall panel that share rows: different base
    addresses, overlapping memory.  SpMM would read rows another lane group is writing."""
    w = W.rmat(10, 8, 16)
    vv = w.values(np.float64)
    S = ctx.plan(w.nrows, w.ncols, w.ii, w.jj, vv)
    tall = ctx.panel(2 * w.nrows, w.k, np.float64)
    tall.fill(1.0)
    row = w.k * 8
    X = device.Panel(ctx, w.ncols, w.k, np.float64, dev=tall.device_ptr())
    Y_over = device.Panel(ctx, w.nrows, w.k, np.float64, dev=tall.device_ptr() + row * (w.nrows - 1))
    Y_next = device.Panel(ctx, w.nrows, w.k, np.float64, dev=tall.device_ptr() + row * w.nrows)
    with pytest.raises(capi.Spc3dError) as e:
        ctx.spmm(S, X, Y_over)
    assert "overlap" in str(e.value)
    dC = ctx.vals(w.nnz, np.float64)
    with pytest.raises(capi.Spc3dError):
        ctx.sddmm_spmm(S, X, X, dC, Y_over)
    ctx.spmm(S, X, Y_next)  # adjacent, not overlapping: fine
    ctx.sync()
    for h in (X, Y_over, Y_next, dC, S, tall):
        h.close()
