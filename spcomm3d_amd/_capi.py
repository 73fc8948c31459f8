"""ctypes binding of the C ABI in ``include/spcomm3d_hip.h``.

Loads the in-tree ``spcomm3d_amd/lib/libspcomm3d_hip.so`` and nothing else:
there is no CPU fallback, and a missing library is an error.
"""
from __future__ import annotations

import ctypes
import os
import re

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libspcomm3d_hip.so")
HEADER_PATH = os.path.join(os.path.dirname(_HERE), "include", "spcomm3d_hip.h")

OK, ERR_INVALID_ARG, ERR_BAD_INDEX, ERR_SIZE_MISMATCH = 0, 1, 2, 3
ERR_TOO_LARGE, ERR_NO_DEVICE, ERR_HIP, ERR_ALLOC = 4, 5, 6, 7
F32, F64 = 0, 1

c_int, c_u32, c_u64 = ctypes.c_int, ctypes.c_uint32, ctypes.c_uint64
c_vp, c_double, c_float = ctypes.c_void_p, ctypes.c_double, ctypes.c_float
P = ctypes.POINTER


class PlanInfo(ctypes.Structure):
    _fields_ = [("nrows", c_u32), ("ncols", c_u32), ("nnz", c_u64),
                ("rows_touched", c_u32), ("cols_touched", c_u32),
                ("nsegments", c_u32), ("nsegments_padded", c_u32),
                ("nsplit_rows", c_u32), ("npartial_slots", c_u32),
                ("max_row_nnz", c_u32), ("seg_max", c_u32),
                ("order_is_identity", ctypes.c_int32), ("nqueues", c_u32),
                ("hot_cols", c_u32), ("hub_rows", c_u32), ("hot_entries", c_u64),
                ("nsegments_long", c_u32), ("ncol_blocks", c_u32),
                ("staged_entries", c_u64), ("positions_by_segment", c_u32),
                ("sddmm_by_column", c_u32), ("two_pass_results", c_u32),
                ("entries_by_column", c_u32), ("device_bytes", c_u64),
                ("sweep_entries", c_u64), ("sweep_tiles", c_u32), ("sweep_k", c_u32)]


class CtxOpts(ctypes.Structure):
    _fields_ = [("host_threads", c_u32), ("flags", c_u32), ("reserved", c_u32 * 6)]


CTX_NO_AUX_STREAM, CTX_NO_HOST_CACHE = 1, 2


class PlanOpts(ctypes.Structure):
    _fields_ = [("seg_max", c_u32), ("k_hint", c_u32), ("l2_hot_bytes", c_u32),
                ("hub_min", c_u32), ("xcd_slices", c_u32), ("builder", c_u32),
                ("col_blocks", c_u32), ("flags", c_u32), ("two_pass_min", c_u32),
                ("sweep", c_u32), ("sweep_min_row", c_u32), ("reserved", c_u32 * 1)]

PLAN_NO_STAGED_STORES, PLAN_NO_SDDMM_BY_COLUMN, PLAN_NO_TWO_PASS, PLAN_KEEP_ENTRY_ORDER = 1, 2, 4, 8
PLAN_SWEEP_STAGED, PLAN_NO_SLICE_AFFINITY = 16, 32


# name -> (restype, argtypes); one entry for every function the header declares.
SIGNATURES = {
    "spc3d_version": (ctypes.c_char_p, []),
    "spc3d_last_error": (ctypes.c_char_p, []),
    "spc3d_kernel_variant": (ctypes.c_char_p, [ctypes.c_int, ctypes.c_uint32]),
    "spc3d_status_name": (ctypes.c_char_p, [c_int]),
    "spc3d_device_count": (c_int, [P(c_int)]),
    "spc3d_ctx_create": (c_int, [c_int, P(c_vp)]),
    "spc3d_ctx_create_ex": (c_int, [c_int, P(CtxOpts), P(c_vp)]),
    "spc3d_ctx_destroy": (c_int, [c_vp]),
    "spc3d_ctx_sync": (c_int, [c_vp]),
    "spc3d_ctx_stream": (c_int, [c_vp, P(c_vp)]),
    "spc3d_ctx_probe_xcd": (c_int, [c_vp, c_u32, c_vp]),
    "spc3d_timer_mark": (c_int, [c_vp, c_int]),
    "spc3d_timer_elapsed_ms": (c_int, [c_vp, c_int, c_int, P(c_float)]),
    "spc3d_capture_begin": (c_int, [c_vp]),
    "spc3d_capture_end": (c_int, [c_vp, P(c_vp)]),
    "spc3d_graph_launch": (c_int, [c_vp]),
    "spc3d_graph_destroy": (c_int, [c_vp]),
    "spc3d_panel_create": (c_int, [c_vp, c_int, c_u32, c_u32, P(c_vp)]),
    "spc3d_panel_wrap": (c_int, [c_vp, c_int, c_u32, c_u32, c_vp, P(c_vp)]),
    "spc3d_panel_destroy": (c_int, [c_vp]),
    "spc3d_panel_upload": (c_int, [c_vp, c_vp]),
    "spc3d_panel_download": (c_int, [c_vp, c_vp]),
    "spc3d_panel_fill": (c_int, [c_vp, c_double]),
    "spc3d_panel_copy": (c_int, [c_vp, c_vp]),
    "spc3d_panel_device_ptr": (c_int, [c_vp, P(c_vp)]),
    "spc3d_panel_shape": (c_int, [c_vp, P(c_u32), P(c_u32), P(c_int)]),
    "spc3d_vals_create": (c_int, [c_vp, c_int, c_u64, P(c_vp)]),
    "spc3d_vals_wrap": (c_int, [c_vp, c_int, c_u64, c_vp, P(c_vp)]),
    "spc3d_vals_destroy": (c_int, [c_vp]),
    "spc3d_vals_upload": (c_int, [c_vp, c_vp]),
    "spc3d_vals_download": (c_int, [c_vp, c_vp]),
    "spc3d_vals_fill": (c_int, [c_vp, c_double]),
    "spc3d_vals_device_ptr": (c_int, [c_vp, P(c_vp)]),
    "spc3d_vals_copy": (c_int, [c_vp, c_u64, c_vp, c_u64, c_u64]),
    "spc3d_coo_validate": (c_int, [c_u32, c_u32, c_u64, c_vp, c_vp]),
    "spc3d_plan_create": (c_int, [c_vp, c_int, c_u32, c_u32, c_u64, c_vp, c_vp, c_vp, P(c_vp)]),
    "spc3d_plan_create_ex": (c_int, [c_vp, c_int, c_u32, c_u32, c_u64, c_vp, c_vp, c_vp,
                                     P(PlanOpts), P(c_vp)]),
    "spc3d_plan_build_host": (c_int, [c_int, c_u32, c_u32, c_u64, c_vp, c_vp, P(PlanOpts),
                                      P(PlanInfo), c_vp, c_vp, c_vp, c_u32, c_vp, c_u32]),
    "spc3d_plan_create_from_device": (c_int, [c_vp, c_int, c_u32, c_u32, c_u64, c_vp, c_vp,
                                              P(PlanOpts), P(c_vp)]),
    "spc3d_localize_device": (c_int, [c_vp, c_u64, c_vp, c_vp, P(c_u32)]),
    "spc3d_remap_device": (c_int, [c_vp, c_u64, c_vp, c_vp, c_u32]),
    "spc3d_plan_download": (c_int, [c_vp, c_vp, c_vp, c_vp, c_u32, c_vp, c_u32]),
    "spc3d_plan_destroy": (c_int, [c_vp]),
    "spc3d_plan_set_values": (c_int, [c_vp, c_vp]),
    "spc3d_plan_set_values_device": (c_int, [c_vp, c_vp]),
    "spc3d_plan_get_info": (c_int, [c_vp, P(PlanInfo)]),
    "spc3d_plan_probe_columns": (c_int, [c_vp, c_int, c_u32]),
    "spc3d_sddmm": (c_int, [c_vp, c_vp, c_vp, c_vp, c_vp]),
    "spc3d_spmm": (c_int, [c_vp, c_vp, c_vp, c_vp]),
    "spc3d_spmm_noalloc": (c_int, [c_vp, c_vp, c_vp, c_vp]),
    "spc3d_sddmm_spmm": (c_int, [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_int]),
    "spc3d_rowmap_create": (c_int, [c_vp, c_u32, c_u64, c_vp, P(c_vp)]),
    "spc3d_rowmap_destroy": (c_int, [c_vp]),
    "spc3d_rows_pack": (c_int, [c_vp, c_vp, c_vp, c_vp]),
    "spc3d_rows_unpack": (c_int, [c_vp, c_vp, c_vp, c_vp]),
    "spc3d_rows_unpack_sum": (c_int, [c_vp, c_vp, c_vp, c_vp]),
    "spc3d_sddmm_host": (c_int, [c_vp, c_int, c_u32, c_u32, c_u32, c_vp, c_vp, c_u64, c_vp, c_vp,
                                 c_vp, c_vp]),
    "spc3d_spmm_host": (c_int, [c_vp, c_int, c_u32, c_u32, c_u32, c_vp, c_u64, c_vp, c_vp, c_vp,
                                c_vp]),
    "spc3d_host_cache_clear": (c_int, [c_vp]),
    "spc3d_host_call_stats": (c_int, [c_vp, c_vp, c_vp, c_vp]),
}

_lib = None


def header_symbols() -> list[str]:
    """Names of all functions declared in the public header."""
    with open(HEADER_PATH) as f:
        text = f.read()
    return sorted(set(re.findall(r"SPC3D_API\s+[\w\s\*]+?\b(spc3d_\w+)\s*\(", text)))


def load() -> ctypes.CDLL:
    """The C-ABI library, with argument types declared.  Raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is not built (there is no CPU fallback); run "
            "`python -c 'import __graft_entry__ as g; g.build()'` or `make -C spcomm3d_amd/csrc`")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


class Spc3dError(RuntimeError):
    """A C-ABI call returned a non-zero status."""

    def __init__(self, status: int, message: str, call: str):
        self.status = status
        self.call = call
        name = load().spc3d_status_name(status).decode()
        super().__init__(f"{call}: {name} ({status}): {message}")


class BadIndexError(Spc3dError, IndexError):
    """ii/jj outside the pattern: the reference's std::out_of_range (core_ops.cpp:16,18,32)."""


def check(status: int, call: str) -> None:
    if status == OK:
        return
    msg = load().spc3d_last_error().decode(errors="replace")
    if status == ERR_BAD_INDEX:
        raise BadIndexError(status, msg, call)
    raise Spc3dError(status, msg, call)


def device_count() -> int:
    """Number of HIP devices, 0 if there is none (no exception)."""
    n = c_int(0)
    rc = load().spc3d_device_count(ctypes.byref(n))
    return n.value if rc == OK else 0
