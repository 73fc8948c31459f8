"""Thin object layer over the C ABI: device-resident panels, value vectors and
plans.  Every method is one C-ABI call; nothing is computed in Python."""
from __future__ import annotations

import ctypes

import numpy as np

from . import _capi as capi
from ._capi import PlanInfo, PlanOpts, check

_DT = {np.dtype(np.float32): capi.F32, np.dtype(np.float64): capi.F64}
_NP = {capi.F32: np.dtype(np.float32), capi.F64: np.dtype(np.float64)}


def dtype_code(dtype) -> int:
    if isinstance(dtype, str):
        dtype = {"f32": np.float32, "f64": np.float64}.get(dtype, dtype)
    if isinstance(dtype, int) and dtype in _NP:
        return dtype
    try:
        return _DT[np.dtype(dtype)]
    except (KeyError, TypeError):
        raise TypeError(f"unsupported real type {dtype!r}: float32 or float64") from None


def _vp(a: np.ndarray | None):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


_BUILDERS = {None: 0, "device": 2, "host": 1}


def make_opts(seg_max=None, k_hint=None, l2_hot_bytes=None, hub_min=None,
              xcd_slices=None, builder=None, col_blocks=None, staged_stores=None,
              sddmm_by_column=None, two_pass=None, two_pass_min=None,
              keep_entry_order=None, sweep=None, sweep_min_row=None,
              sweep_staged=None, slice_affinity=None) -> PlanOpts:
    """``spc3d_plan_opts``; ``None`` keeps the library default.  ``builder``:
    ``"device"`` or ``"host"`` (where ``spc3d_plan_create_ex`` builds the plan).
    ``staged_stores`` / ``sddmm_by_column`` / ``two_pass`` = False keep the plain stores
    of SDDMM results; ``keep_entry_order`` = True keeps the caller's order inside rows
    that arrive unsorted.  ``sweep``: ``None`` (the library decides), ``False`` (never) or
    ``True`` (row tiles x column blocks whenever ``k_hint`` has a width the kernels take);
    ``sweep_staged`` = True stages the tiles' SDDMM results whatever the entry order;
    ``slice_affinity`` = False deals the free segments of a sliced plan by rank alone."""
    o = PlanOpts()
    o.sweep = 0 if sweep is None else (2 if sweep else 1)
    o.sweep_min_row = int(sweep_min_row or 0)
    o.flags = ((capi.PLAN_NO_STAGED_STORES if staged_stores is False else 0) |
               (capi.PLAN_NO_SDDMM_BY_COLUMN if sddmm_by_column is False else 0) |
               (capi.PLAN_NO_TWO_PASS if two_pass is False else 0) |
               (capi.PLAN_KEEP_ENTRY_ORDER if keep_entry_order else 0) |
               (capi.PLAN_SWEEP_STAGED if sweep_staged else 0) |
               (capi.PLAN_NO_SLICE_AFFINITY if slice_affinity is False else 0))
    o.two_pass_min = int(two_pass_min or 0)
    o.builder = _BUILDERS[builder]
    o.seg_max = int(seg_max or 0)
    o.k_hint = int(k_hint or 0)
    o.l2_hot_bytes = int(l2_hot_bytes or 0)
    o.hub_min = int(hub_min or 0)
    o.xcd_slices = int(xcd_slices or 0)
    o.col_blocks = int(col_blocks or 0)
    return o


def _as_idx(a, name: str) -> np.ndarray:
    a = np.asarray(a)
    if a.dtype != np.uint32:
        if a.size and (a.min() < 0 or a.max() > 0xFFFFFFFF):
            raise capi.BadIndexError(capi.ERR_BAD_INDEX, f"{name} does not fit uint32", "as_idx")
        a = a.astype(np.uint32)
    return np.ascontiguousarray(a)


class Context:
    """One device and one stream (``spc3d_ctx``)."""

    def __init__(self, device: int = 0, host_threads: int | None = None,
                 aux_stream: bool | None = None, host_cache: bool | None = None):
        """No option given: ``spc3d_ctx_create`` (defaults, environment overrides); else
        ``spc3d_ctx_create_ex`` with ``spc3d_ctx_opts`` (``None`` fields keep the default)."""
        self._lib = capi.load()
        h = ctypes.c_void_p()
        if host_threads is None and aux_stream is None and host_cache is None:
            check(self._lib.spc3d_ctx_create(device, ctypes.byref(h)), "spc3d_ctx_create")
        else:
            o = capi.CtxOpts()
            o.host_threads = int(host_threads or 0)
            o.flags = ((capi.CTX_NO_AUX_STREAM if aux_stream is False else 0) |
                       (capi.CTX_NO_HOST_CACHE if host_cache is False else 0))
            check(self._lib.spc3d_ctx_create_ex(device, ctypes.byref(o), ctypes.byref(h)),
                  "spc3d_ctx_create_ex")
        self._h = h
        self.device = device

    def close(self):
        if getattr(self, "_h", None):
            self._lib.spc3d_ctx_destroy(self._h)
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def sync(self):
        check(self._lib.spc3d_ctx_sync(self._h), "spc3d_ctx_sync")

    def mark(self, slot: int):
        check(self._lib.spc3d_timer_mark(self._h, slot), "spc3d_timer_mark")

    def elapsed_ms(self, start: int, stop: int) -> float:
        ms = ctypes.c_float()
        check(self._lib.spc3d_timer_elapsed_ms(self._h, start, stop, ctypes.byref(ms)),
              "spc3d_timer_elapsed_ms")
        return float(ms.value)

    # -- factories ---------------------------------------------------------
    def panel(self, m: int, n: int, dtype) -> "Panel":
        return Panel(self, m, n, dtype)

    def panel_from(self, host: np.ndarray) -> "Panel":
        host = np.ascontiguousarray(host)
        if host.ndim != 2:
            raise ValueError("a panel is a 2-D row-major array")
        p = Panel(self, host.shape[0], host.shape[1], host.dtype)
        p.upload(host)
        return p

    def vals(self, n: int, dtype) -> "Vals":
        return Vals(self, n, dtype)

    def plan(self, nrows, ncols, ii, jj, vv=None, dtype=None, seg_max: int | None = None,
             **opts) -> "Plan":
        """``opts``: fields of :func:`make_opts`; none given = ``spc3d_plan_create`` defaults."""
        if seg_max is not None:
            opts["seg_max"] = seg_max
        return Plan(self, nrows, ncols, ii, jj, vv, dtype, opts or None)

    def sddmm_spmm(self, S: "Plan", A: "Panel", B: "Panel", C: "Vals", Y: "Panel",
                   chained: bool = False):
        """SDDMM and the SpMM of the same pattern over ``B`` in one pass
        (``spc3d_sddmm_spmm``): ``C`` as :meth:`sddmm`; ``Y += S B``, or ``Y += C B`` when
        ``chained``."""
        check(self._lib.spc3d_sddmm_spmm(self._h, S._h, A._h, B._h, C._h, Y._h, int(chained)),
              "spc3d_sddmm_spmm")

    def capture_begin(self):
        """Start recording kernel-launching calls instead of running them (``spc3d_capture_begin``)."""
        check(self._lib.spc3d_capture_begin(self._h), "spc3d_capture_begin")

    def capture_end(self) -> "Graph":
        h = ctypes.c_void_p()
        check(self._lib.spc3d_capture_end(self._h, ctypes.byref(h)), "spc3d_capture_end")
        return Graph(self, h)

    def probe_xcd(self, nblocks: int) -> np.ndarray:
        """XCD id each workgroup of an ``nblocks``-wide grid ran on (``spc3d_ctx_probe_xcd``)."""
        out = np.zeros(nblocks, dtype=np.uint32)
        check(self._lib.spc3d_ctx_probe_xcd(self._h, nblocks, _vp(out)), "spc3d_ctx_probe_xcd")
        return out

    # -- hot path ----------------------------------------------------------
    def sddmm(self, S: "Plan", A: "Panel", B: "Panel", C: "Vals"):
        """C.vv[e] = S.vv[e] * <A[ii[e]], B[jj[e]]>  (src/core_ops.cpp:5-22); asynchronous."""
        check(self._lib.spc3d_sddmm(self._h, S._h, A._h, B._h, C._h), "spc3d_sddmm")

    def spmm(self, A: "Plan", X: "Panel", Y: "Panel"):
        """Y[ii[e]] += A.vv[e] * X[jj[e]]  (src/core_ops.cpp:24-35); asynchronous."""
        check(self._lib.spc3d_spmm(self._h, A._h, X._h, Y._h), "spc3d_spmm")

    def spmm_noalloc(self, A: "Plan", X: "Panel", Y: "Panel"):
        """:meth:`spmm` without any allocation (``spc3d_spmm_noalloc``): the partial sums of
        cut rows live in an array that is part of the library's device code."""
        check(self._lib.spc3d_spmm_noalloc(self._h, A._h, X._h, Y._h), "spc3d_spmm_noalloc")

    def sddmm_host(self, A: np.ndarray, B: np.ndarray, ii, jj, svv: np.ndarray) -> np.ndarray:
        """One-shot SDDMM over host arrays (``spc3d_sddmm_host``); returns C.vv."""
        A, B, svv = (np.ascontiguousarray(x) for x in (A, B, svv))
        if A.ndim != 2 or B.ndim != 2 or A.dtype != B.dtype or A.dtype != svv.dtype:
            raise ValueError("A, B must be 2-D and share svv's dtype")
        if A.shape[1] != B.shape[1]:
            raise capi.Spc3dError(capi.ERR_SIZE_MISMATCH, "A.n != B.n", "sddmm_host")
        ii, jj = _as_idx(ii, "ii"), _as_idx(jj, "jj")
        out = np.empty(ii.size, dtype=A.dtype)
        check(self._lib.spc3d_sddmm_host(self._h, dtype_code(A.dtype), A.shape[0], B.shape[0],
                                         A.shape[1], _vp(A), _vp(B), ii.size, _vp(ii), _vp(jj),
                                         _vp(svv), _vp(out)), "spc3d_sddmm_host")
        return out

    def spmm_host(self, X: np.ndarray, ii, jj, avv: np.ndarray, Y: np.ndarray) -> None:
        """One-shot SpMM over host arrays (``spc3d_spmm_host``); adds into Y in place."""
        X, avv = np.ascontiguousarray(X), np.ascontiguousarray(avv)
        if not (Y.flags.c_contiguous and Y.flags.writeable):
            raise ValueError("Y must be a writable C-contiguous array")
        if X.ndim != 2 or Y.ndim != 2 or X.dtype != Y.dtype or X.dtype != avv.dtype:
            raise ValueError("X, Y must be 2-D and share avv's dtype")
        if X.shape[1] != Y.shape[1]:
            raise capi.Spc3dError(capi.ERR_SIZE_MISMATCH, "X.n != Y.n", "spmm_host")
        ii, jj = _as_idx(ii, "ii"), _as_idx(jj, "jj")
        check(self._lib.spc3d_spmm_host(self._h, dtype_code(X.dtype), X.shape[0], Y.shape[0],
                                        X.shape[1], _vp(X), ii.size, _vp(ii), _vp(jj), _vp(avv),
                                        _vp(Y)), "spc3d_spmm_host")

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Panel:
    """Device-resident ``denseMatrix::data`` (``src/basic.hpp:30-36``)."""

    def __init__(self, ctx: Context, m: int, n: int, dtype, dev: int | None = None):
        """``dev``: a device address to wrap (``spc3d_panel_wrap``) instead of allocating."""
        self.ctx, self.m, self.n = ctx, int(m), int(n)
        self.code = dtype_code(dtype)
        self.dtype = _NP[self.code]
        h = ctypes.c_void_p()
        if dev is None:
            check(ctx._lib.spc3d_panel_create(ctx._h, self.code, self.m, self.n, ctypes.byref(h)),
                  "spc3d_panel_create")
        else:
            check(ctx._lib.spc3d_panel_wrap(ctx._h, self.code, self.m, self.n,
                                            ctypes.c_void_p(dev), ctypes.byref(h)),
                  "spc3d_panel_wrap")
        self._h = h

    def upload(self, host: np.ndarray):
        host = np.ascontiguousarray(host)
        if host.dtype != self.dtype or host.size != self.m * self.n:
            raise ValueError("host array does not match the panel's dtype / size")
        check(self.ctx._lib.spc3d_panel_upload(self._h, _vp(host)), "spc3d_panel_upload")

    def download(self) -> np.ndarray:
        out = np.empty((self.m, self.n), dtype=self.dtype)
        check(self.ctx._lib.spc3d_panel_download(self._h, _vp(out)), "spc3d_panel_download")
        return out

    def fill(self, value: float):
        check(self.ctx._lib.spc3d_panel_fill(self._h, float(value)), "spc3d_panel_fill")

    def copy_from(self, src: "Panel"):
        """self = src on the device (``spc3d_panel_copy``); asynchronous."""
        check(self.ctx._lib.spc3d_panel_copy(self._h, src._h), "spc3d_panel_copy")

    def device_ptr(self) -> int:
        p = ctypes.c_void_p()
        check(self.ctx._lib.spc3d_panel_device_ptr(self._h, ctypes.byref(p)),
              "spc3d_panel_device_ptr")
        return p.value or 0

    def close(self):
        if getattr(self, "_h", None) and getattr(self.ctx, "_h", None):
            self.ctx._lib.spc3d_panel_destroy(self._h)
        self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Vals:
    """Device-resident ``cooMat::vv`` (``src/SparseMatrix.hpp:36``)."""

    def __init__(self, ctx: Context, n: int, dtype, dev: int | None = None):
        """``dev``: a device address to wrap (``spc3d_vals_wrap``) instead of allocating."""
        self.ctx, self.n = ctx, int(n)
        self.code = dtype_code(dtype)
        self.dtype = _NP[self.code]
        h = ctypes.c_void_p()
        if dev is None:
            check(ctx._lib.spc3d_vals_create(ctx._h, self.code, self.n, ctypes.byref(h)),
                  "spc3d_vals_create")
        else:
            check(ctx._lib.spc3d_vals_wrap(ctx._h, self.code, self.n, ctypes.c_void_p(dev),
                                           ctypes.byref(h)), "spc3d_vals_wrap")
        self._h = h

    def upload(self, host: np.ndarray):
        host = np.ascontiguousarray(host)
        if host.dtype != self.dtype or host.size != self.n:
            raise ValueError("host array does not match the vector's dtype / length")
        check(self.ctx._lib.spc3d_vals_upload(self._h, _vp(host)), "spc3d_vals_upload")

    def download(self) -> np.ndarray:
        out = np.empty(self.n, dtype=self.dtype)
        check(self.ctx._lib.spc3d_vals_download(self._h, _vp(out)), "spc3d_vals_download")
        return out

    def fill(self, value: float):
        check(self.ctx._lib.spc3d_vals_fill(self._h, float(value)), "spc3d_vals_fill")

    def device_ptr(self) -> int:
        p = ctypes.c_void_p()
        check(self.ctx._lib.spc3d_vals_device_ptr(self._h, ctypes.byref(p)),
              "spc3d_vals_device_ptr")
        return p.value or 0

    def close(self):
        if getattr(self, "_h", None) and getattr(self.ctx, "_h", None):
            self.ctx._lib.spc3d_vals_destroy(self._h)
        self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Plan:
    """Device-resident sparse operand: the pattern of a ``cooMat`` in kernel
    order plus its values (``spc3d_plan``)."""

    def __init__(self, ctx: Context, nrows, ncols, ii, jj, vv=None, dtype=None,
                 opts: dict | None = None):
        ii = _as_idx(ii, "ii")
        jj = _as_idx(jj, "jj")
        if ii.shape != jj.shape or ii.ndim != 1:
            raise ValueError("ii and jj must be 1-D arrays of the same length")
        if vv is not None:
            vv = np.ascontiguousarray(vv)
            if vv.shape != ii.shape:
                raise ValueError("vv must have one value per entry")
            dtype = vv.dtype if dtype is None else dtype
        if dtype is None:
            raise ValueError("dtype is required when vv is not given")
        self.ctx = ctx
        self.code = dtype_code(dtype)
        self.dtype = _NP[self.code]
        if vv is not None and vv.dtype != self.dtype:
            raise ValueError("vv dtype differs from the plan dtype")
        h = ctypes.c_void_p()
        lib = ctx._lib
        if opts is None:
            rc = lib.spc3d_plan_create(ctx._h, self.code, int(nrows), int(ncols), ii.size, _vp(ii),
                                       _vp(jj), _vp(vv), ctypes.byref(h))
        else:
            rc = lib.spc3d_plan_create_ex(ctx._h, self.code, int(nrows), int(ncols), ii.size,
                                          _vp(ii), _vp(jj), _vp(vv),
                                          ctypes.byref(make_opts(**opts)), ctypes.byref(h))
        check(rc, "spc3d_plan_create")
        self._h = h
        self.nnz = int(ii.size)

    @classmethod
    def from_device(cls, ctx: Context, nrows, ncols, ii: "Vals", jj: "Vals", nnz: int, dtype,
                    **opts) -> "Plan":
        """Plan of a pattern whose ``ii`` / ``jj`` already live on the device, as the
        first ``nnz`` 32-bit words of two value vectors (``spc3d_plan_create_from_device``)."""
        self = cls.__new__(cls)
        self.ctx = ctx
        self.code = dtype_code(dtype)
        self.dtype = _NP[self.code]
        h = ctypes.c_void_p()
        check(ctx._lib.spc3d_plan_create_from_device(
            ctx._h, self.code, int(nrows), int(ncols), int(nnz), ii.device_ptr(), jj.device_ptr(),
            ctypes.byref(make_opts(**opts)), ctypes.byref(h)), "spc3d_plan_create_from_device")
        self._h = h
        self.nnz = int(nnz)
        return self

    def download(self) -> dict:
        """The plan's arrays as they are on the device, in the layout of
        :func:`plan_build_host` (``spc3d_plan_download``)."""
        info = self.info
        col = np.empty(self.nnz, dtype=np.uint32)
        perm = np.empty(self.nnz, dtype=np.uint32)
        segs = np.empty((info.nsegments_padded, 4), dtype=np.uint32)
        splits = np.empty((info.nsplit_rows, 3), dtype=np.uint32)
        check(self.ctx._lib.spc3d_plan_download(self._h, _vp(col), _vp(perm), _vp(segs),
                                                info.nsegments_padded, _vp(splits),
                                                info.nsplit_rows), "spc3d_plan_download")
        return {"info": info, "col": col, "perm": perm, "segs": segs, "splits": splits}

    def set_values(self, vv: np.ndarray):
        vv = np.ascontiguousarray(vv)
        if vv.dtype != self.dtype or vv.size != self.nnz:
            raise ValueError("vv does not match the plan's dtype / nnz")
        check(self.ctx._lib.spc3d_plan_set_values(self._h, _vp(vv)), "spc3d_plan_set_values")

    def set_values_device(self, vv: Vals):
        check(self.ctx._lib.spc3d_plan_set_values_device(self._h, vv._h),
              "spc3d_plan_set_values_device")

    def probe_columns(self, mode: str, modulus: int = 0):
        """Measurement aid: rewrites the plan's columns in place so that every gather hits
        the L2 ("all_hit": c % modulus) or nearly none does ("all_miss"); the plan then
        computes another pattern and is good for timing only."""
        code = {"all_hit": 1, "all_miss": 2}[mode]
        check(self.ctx._lib.spc3d_plan_probe_columns(self._h, code, int(modulus)),
              "spc3d_plan_probe_columns")

    @property
    def info(self) -> PlanInfo:
        info = PlanInfo()
        check(self.ctx._lib.spc3d_plan_get_info(self._h, ctypes.byref(info)), "spc3d_plan_get_info")
        return info

    def close(self):
        if getattr(self, "_h", None) and getattr(self.ctx, "_h", None):
            self.ctx._lib.spc3d_plan_destroy(self._h)
        self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Graph:
    """A recorded sequence of calls, replayed with one launch (``spc3d_graph``)."""

    def __init__(self, ctx: Context, h):
        self.ctx, self._h = ctx, h

    def launch(self):
        check(self.ctx._lib.spc3d_graph_launch(self._h), "spc3d_graph_launch")

    def close(self):
        if getattr(self, "_h", None) and getattr(self.ctx, "_h", None):
            self.ctx._lib.spc3d_graph_destroy(self._h)
        self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class RowMap:
    """Buffer slot i <-> dense row ``rows[i]`` of a panel (``spc3d_rowmap``): the
    device form of ``SparseComm::sendptr`` / ``recvptr`` (``src/comm.hpp:41,49``)."""

    def __init__(self, ctx: Context, panel_rows: int, rows):
        rows = _as_idx(rows, "rows")
        self.ctx, self.n = ctx, int(rows.size)
        h = ctypes.c_void_p()
        check(ctx._lib.spc3d_rowmap_create(ctx._h, int(panel_rows), rows.size, _vp(rows),
                                           ctypes.byref(h)), "spc3d_rowmap_create")
        self._h = h

    def pack(self, panel: Panel, buf: Vals):
        """buf[i,:] = panel[rows[i],:]  (``copy_to_sendbuff``, ``src/comm.hpp:90-103``)."""
        check(self.ctx._lib.spc3d_rows_pack(self.ctx._h, panel._h, self._h, buf._h),
              "spc3d_rows_pack")

    def unpack(self, panel: Panel, buf: Vals):
        """panel[rows[i],:] = buf[i,:]  (``copy_from_recvbuff``, ``src/comm.hpp:166-177``)."""
        check(self.ctx._lib.spc3d_rows_unpack(self.ctx._h, panel._h, self._h, buf._h),
              "spc3d_rows_unpack")

    def unpack_sum(self, panel: Panel, buf: Vals):
        """panel[rows[i],:] += buf[i,:]  (``SUM_from_recvbuff``, ``src/comm.hpp:178-189``)."""
        check(self.ctx._lib.spc3d_rows_unpack_sum(self.ctx._h, panel._h, self._h, buf._h),
              "spc3d_rows_unpack_sum")

    def close(self):
        if getattr(self, "_h", None) and getattr(self.ctx, "_h", None):
            self.ctx._lib.spc3d_rowmap_destroy(self._h)
        self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def localize_device(ctx: Context, idx: Vals, n: int) -> tuple[int, Vals]:
    """``COOMatrix::localizeIndices`` (``src/SparseMatrix.hpp:69-99``) for one index
    array held as the first ``n`` 32-bit words of ``idx``: rewrites it to local ids
    in order of first appearance; returns their number and the local -> global map
    (a value vector of ``n`` words, the first ``nlocal`` of which are used)."""
    ltg = Vals(ctx, max(int(n), 1), np.float32)
    nlocal = ctypes.c_uint32()
    check(ctx._lib.spc3d_localize_device(ctx._h, int(n), idx.device_ptr(), ltg.device_ptr(),
                                         ctypes.byref(nlocal)), "spc3d_localize_device")
    return int(nlocal.value), ltg


def remap_device(ctx: Context, idx: Vals, n: int, mapping: Vals, map_len: int) -> None:
    """``COOMatrix::ReMapIndices`` (``src/SparseMatrix.hpp:100-106``):
    ``idx[e] = mapping[idx[e]]`` on the device."""
    check(ctx._lib.spc3d_remap_device(ctx._h, int(n), idx.device_ptr(), mapping.device_ptr(),
                                      int(map_len)), "spc3d_remap_device")


def coo_validate(nrows: int, ncols: int, ii, jj) -> None:
    """Host-only bounds check of a pattern; raises :class:`BadIndexError`."""
    ii = _as_idx(ii, "ii")
    jj = _as_idx(jj, "jj")
    check(capi.load().spc3d_coo_validate(int(nrows), int(ncols), ii.size, _vp(ii), _vp(jj)),
          "spc3d_coo_validate")


def plan_build_host(nrows: int, ncols: int, ii, jj, dtype="f32", **opts) -> dict:
    """Host-only view of the kernel-order form of a pattern
    (``spc3d_plan_build_host``): needs no GPU.  ``opts`` as :func:`make_opts`.
    Returns ``info``, ``col``, ``perm``, ``segs`` (``[nseg_padded, 4]``: row,
    start, len, slot) and ``splits`` (``[nsplit, 3]``: row,
    first_slot, nslots)."""
    lib = capi.load()
    ii = _as_idx(ii, "ii")
    jj = _as_idx(jj, "jj")
    code = dtype_code(dtype)
    o = make_opts(**opts)
    info = PlanInfo()
    check(lib.spc3d_plan_build_host(code, int(nrows), int(ncols), ii.size, _vp(ii), _vp(jj),
                                    ctypes.byref(o), ctypes.byref(info), None, None, None, 0,
                                    None, 0),
          "spc3d_plan_build_host")
    col = np.empty(ii.size, dtype=np.uint32)
    perm = np.empty(ii.size, dtype=np.uint32)
    segs = np.empty((info.nsegments_padded, 4), dtype=np.uint32)
    splits = np.empty((info.nsplit_rows, 3), dtype=np.uint32)
    check(lib.spc3d_plan_build_host(code, int(nrows), int(ncols), ii.size, _vp(ii), _vp(jj),
                                    ctypes.byref(o), ctypes.byref(info), _vp(col), _vp(perm),
                                    _vp(segs), info.nsegments_padded, _vp(splits),
                                    info.nsplit_rows),
          "spc3d_plan_build_host")
    return {"info": info, "col": col, "perm": perm, "segs": segs, "splits": splits}


def kernel_variant(dtype, k: int) -> str:
    """Which kernel variant dense rows of k reals of `dtype` run (spc3d_kernel_variant)."""
    r = capi.load().spc3d_kernel_variant(dtype_code(dtype), int(k))
    if r is None:
        raise ValueError("unknown dtype")
    return r.decode()

