#!/usr/bin/env python3
"""Benchmark of the local SDDMM + SpMM step on one MI355X.

A step is one pass of the hot path over one resident workload: SDDMM
(C = S .* (A B^T)) followed by SpMM (Y += S X), both through the C ABI, with
every operand already in HBM when the timed region starts.  Default workload:
R-MAT scale 20, edge factor 16, K = 64 (the configuration the metric is quoted
on), in the reference's real type (fp64); the other real type is measured in
the same run and reported under "also".

Prints one JSON line.  `value` is (flops of both kernels) / (wall time per
step).  `roofline` is the slower of the two kernels: strict-model bytes per
launch over its mean launch time, measured with HIP events on the library's
stream inside the timed region, against 8 TB/s.  `cpu_baseline` is the
reference's own kernels (where their build is present, fp64) or else the CPU
oracle (a serial restatement of the reference's loops), timed on one host core
on the same workload.  `fused_step` is the same step through the one-pass entry
point spc3d_sddmm_spmm (an extension without counterpart in the reference); it is
reported beside `value`, which always comes from the two separate calls.
`roofline.device_copy_gbs` is a plain device copy of one panel timed in the same run
(read + write), with the kernel's strict-model rate and its measured traffic as fractions
of it.  `row_copies` times the pack and sum-unpack copies of a sparse exchange over the
touched rows of Y (algorithmic bytes: rows read + buffer written; buffer read +
rows read and written).  `also` holds the other real type, the same workload
handed over in shuffled COO order (the reference never sorts its entries) and in
column-major order (the order of the MatrixMarket files it reads) in both types,
and `configs`: one compact row per other benchmark configuration (time per kernel,
strict-model fraction of the HBM peak).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "SDDMM & SpMM GFLOP/s + % HBM roofline on 1 MI355X, RMAT-20 K=64"

# Bytes that cross between the eight L2s and the fabric (Infinity Cache / HBM) per call,
# measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE and calibrated on a plain copy.
# They cannot be collected from inside this process, so they are read from the profile
# summary they were recorded in, for the workload and plan options it was taken on, and
# are null for any other.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "sddmm_spmm_rmat20_k64_hbm_traffic.md")
TRAFFIC_LEVEL = "l2_fabric (FETCH_SIZE x 2 + WRITE_SIZE: fills and write-backs of the L2s; " \
                "hits in the Infinity Cache are included, no HBM-side counter is exposed)"
TRAFFIC_WORKLOAD = ("rmat20_ef16", 64, "sorted")


def traffic_is_current(path=TRAFFIC_PROFILE):
    """True when the traffic profile was recorded on the device code that is in the tree
    now (the digest in its header against the sources')."""
    from spcomm3d_amd import provenance

    return provenance.recorded_hash(path) == provenance.source_hash()


def measured_traffic(path=TRAFFIC_PROFILE):
    """{(dtype, call): bytes} from the 'Per call' table of the traffic profile."""
    import re

    out = {}
    try:
        text = open(path).read()
    except OSError:
        return out
    row = re.compile(r"^\|\s*(f32|f64)\s*\|\s*(sddmm_spmm|sddmm|spmm)[^|]*\|\s*([\d,]+\.?\d*)\s*\|",
                     re.M)
    for dtype, call, mb in row.findall(text.split("Per call", 1)[-1]):
        out[(dtype, call)] = float(mb.replace(",", "")) * 1e6
    return out


def log(*a):
    print(*a, file=sys.stderr, flush=True)


# Plan options of the main workload's plans beside k_hint (--col-blocks, --sweep): for the
# comparisons the profile summaries hold; the default run passes none.
PLAN_OPTS: dict = {}


def plan_opts(w):
    """k_hint when the workload's K is not the library's default of 64 (the plan sizes its
    L2-resident set, and chooses column blocks / row tiles, for the width it is told), an
    explicit one whenever other options are given."""
    hint = {} if w.k == 64 and not PLAN_OPTS else {"k_hint": w.k}
    return dict(hint, **PLAN_OPTS)


def ensure_built():
    need = ["spcomm3d_amd/lib/libspcomm3d_hip.so", "spcomm3d_amd/gen/libspc3d_gen.so"]
    if not all(os.path.exists(os.path.join(ROOT, p)) for p in need):
        import __graft_entry__

        __graft_entry__.build()


def run_gpu(w, dtype, steps, warmup, seg_max=None, max_timed=1300, copies=0):
    """Times `steps` SDDMM+SpMM passes on resident operands; returns a dict."""
    from spcomm3d_amd import device, roofline
    from spcomm3d_amd import workloads as W

    wbytes = np.dtype(W.np_dtype(dtype)).itemsize
    A, B, Y0, vv = w.panel_A(dtype), w.panel_B(dtype), w.panel_Y0(dtype), w.values(dtype)
    with device.Context(0) as ctx:
        t0 = time.perf_counter()
        S = ctx.plan(w.nrows, w.ncols, w.ii, w.jj, vv, seg_max=seg_max, **plan_opts(w))
        ctx.sync()
        plan_s = time.perf_counter() - t0
        info = S.info
        t0 = time.perf_counter()
        dA, dB, dY = ctx.panel_from(A), ctx.panel_from(B), ctx.panel_from(Y0)
        dC = ctx.vals(w.nnz, dtype)
        ctx.sync()
        upload_s = time.perf_counter() - t0
        del A, B, Y0

        if copies:
            # Plain device copies of known size, so that a counter run of this same
            # command has a dispatch (copy_kernel) to calibrate FETCH_SIZE/WRITE_SIZE on.
            dT = ctx.panel(w.nrows, w.k, dtype)
            for _ in range(copies):
                dT.copy_from(dA)
            ctx.sync()
            dT.close()
            log(f"calibration: {copies} x copy_kernel, {w.nrows * w.k * wbytes} bytes read and "
                f"as many written per launch")
        for _ in range(warmup):
            ctx.sddmm(S, dA, dB, dC)
            ctx.spmm(S, dB, dY)
        ctx.sync()
        ntimed = min(steps, max_timed)
        t0 = time.perf_counter()
        for i in range(steps):
            if i < ntimed:
                ctx.mark(3 * i)
                ctx.sddmm(S, dA, dB, dC)
                ctx.mark(3 * i + 1)
                ctx.spmm(S, dB, dY)
                ctx.mark(3 * i + 2)
            else:
                ctx.sddmm(S, dA, dB, dC)
                ctx.spmm(S, dB, dY)
        ctx.sync()
        wall = time.perf_counter() - t0
        sd = np.array([ctx.elapsed_ms(3 * i, 3 * i + 1) for i in range(ntimed)])
        sp = np.array([ctx.elapsed_ms(3 * i + 1, 3 * i + 2) for i in range(ntimed)])
        # The same step through the fused entry point (both results from one pass over
        # the gathered rows); reported beside the headline, never as it.
        for _ in range(warmup):
            ctx.sddmm_spmm(S, dA, dB, dC, dY)
        ctx.sync()
        t0 = time.perf_counter()
        for _ in range(steps):
            ctx.sddmm_spmm(S, dA, dB, dC, dY)
        ctx.sync()
        fused_wall = time.perf_counter() - t0
        # The copies either side of a sparse exchange on the same panel: every touched
        # row of Y packed into a buffer, and the buffer summed back (src/comm.hpp:90-103,
        # 178-189), `steps` times each.
        touched = np.flatnonzero(np.bincount(w.ii, minlength=w.nrows)).astype(np.uint32)
        rmap = device.RowMap(ctx, w.nrows, touched)
        dbuf = ctx.vals(touched.size * w.k, dtype)
        for _ in range(warmup):
            rmap.pack(dY, dbuf)
            rmap.unpack_sum(dY, dbuf)
        ctx.sync()
        ctx.mark(4000)
        for _ in range(steps):
            rmap.pack(dY, dbuf)
        ctx.mark(4001)
        for _ in range(steps):
            rmap.unpack_sum(dY, dbuf)
        ctx.mark(4002)
        pack_ms = ctx.elapsed_ms(4000, 4001) / steps
        sum_ms = ctx.elapsed_ms(4001, 4002) / steps
        nrow_bytes = touched.size * w.k * wbytes
        rows = {"rows": int(touched.size),
                "pack": {"ms": pack_ms, "bytes": int(2 * nrow_bytes + 4 * touched.size)},
                "unpack_sum": {"ms": sum_ms, "bytes": int(3 * nrow_bytes + 4 * touched.size)}}
        for v in (rows["pack"], rows["unpack_sum"]):
            v["gbs"] = v["bytes"] / v["ms"] / 1e6
            v["frac"] = v["gbs"] / roofline.HBM_PEAK_GBS
        rmap.close()
        dbuf.close()
        # A plain device copy of one panel (read + write), the rate this machine moves bytes
        # at when nothing is gathered: the second yardstick beside the 8 TB/s peak.
        dT = ctx.panel(w.nrows, w.k, dtype)
        for _ in range(warmup):
            dT.copy_from(dA)
        ctx.mark(4003)
        for _ in range(steps):
            dT.copy_from(dA)
        ctx.mark(4004)
        copy_gbs = 2 * w.nrows * w.k * wbytes / (ctx.elapsed_ms(4003, 4004) / steps) / 1e6
        dT.close()
        for h in (S, dA, dB, dY, dC):
            h.close()

    m_t, n_t = info.rows_touched, info.cols_touched
    with_perm = not info.order_is_identity
    fl = roofline.flops(w.nnz, w.k)
    out = {"dtype": dtype, "ms_per_step": wall / steps * 1e3, "plan_build_s": plan_s,
           "plan_device_bytes": int(info.device_bytes), "col_blocks": int(info.ncol_blocks),
           "sweep_entries": int(info.sweep_entries), "sweep_tiles": int(info.sweep_tiles),
           "staged_entries": int(info.staged_entries),
           "upload_s": upload_s, "nsegments": info.nsegments, "nsplit_rows": info.nsplit_rows,
           "seg_max": info.seg_max, "rows_touched": m_t, "cols_touched": n_t,
           "gflops": 2 * fl / (wall / steps) / 1e9, "kernels": {}}
    fb = roofline.fused_bytes(w.nrows, w.nnz, w.k, wbytes, m_t, n_t, with_perm)
    out["fused_step"] = {"entry": "spc3d_sddmm_spmm", "ms_per_step": fused_wall / steps * 1e3,
                         "gflops": 2 * fl / (fused_wall / steps) / 1e9, "strict_bytes": int(fb),
                         "strict_frac": fb / (fused_wall / steps) / 1e9 / roofline.HBM_PEAK_GBS}
    out["row_copies"] = rows
    out["device_copy_gbs"] = copy_gbs
    for name, ms, strict, gather in (
            ("sddmm", sd,
             roofline.sddmm_bytes(w.nrows, w.nnz, w.k, wbytes, m_t, n_t, with_perm),
             roofline.sddmm_bytes(w.nrows, w.nnz, w.k, wbytes, m_t, n_t, with_perm, gather=True)),
            ("spmm", sp,
             roofline.spmm_bytes(w.nrows, w.nnz, w.k, wbytes, m_t, n_t),
             roofline.spmm_bytes(w.nrows, w.nnz, w.k, wbytes, m_t, n_t, gather=True))):
        avg = float(ms.mean())
        out["kernels"][name] = {
            "ms_avg": avg, "ms_min": float(ms.min()), "ms_median": float(np.median(ms)),
            "gflops": fl / avg / 1e6, "strict_bytes": int(strict), "gather_bytes": int(gather),
            "strict_gbs": strict / avg / 1e6, "gather_gbs": gather / avg / 1e6,
            "strict_frac": strict / avg / 1e6 / roofline.HBM_PEAK_GBS,
            "gather_frac": gather / avg / 1e6 / roofline.HBM_PEAK_GBS}
    return out


def run_floors(w, dtype, steps, warmup, seg_max=None):
    """The two floors of the same launches: the plan of `w` as the timed runs build it, with
    its columns rewritten on the device (spc3d_plan_probe_columns) so that every gathered
    dense row is found in the L2 (a table of 1 MiB per L2), then so that nearly none is
    (uniform random columns).  Segments, queues, streams and instruction stream are those
    of the real plan; only the gather addresses differ."""
    from spcomm3d_amd import device
    from spcomm3d_amd import workloads as W

    wbytes = np.dtype(W.np_dtype(dtype)).itemsize
    modulus = max(64, (1 << 20) // (w.k * wbytes))
    out = {"dtype": dtype, "all_hit_table_rows": modulus, "steps": steps}
    with device.Context(0) as ctx:
        S = ctx.plan(w.nrows, w.ncols, w.ii, w.jj, w.values(dtype), seg_max=seg_max,
                     **plan_opts(w))
        dA, dB = ctx.panel_from(w.panel_A(dtype)), ctx.panel_from(w.panel_B(dtype))
        dY = ctx.panel_from(w.panel_Y0(dtype))
        dC = ctx.vals(w.nnz, dtype)
        for mode in ("all_hit", "all_miss"):
            S.probe_columns(mode, modulus)
            for _ in range(warmup):
                ctx.sddmm(S, dA, dB, dC)
                ctx.spmm(S, dB, dY)
            ctx.sync()
            ctx.mark(0)
            for _ in range(steps):
                ctx.sddmm(S, dA, dB, dC)
            ctx.mark(1)
            for _ in range(steps):
                ctx.spmm(S, dB, dY)
            ctx.mark(2)
            out[mode] = {"sddmm_ms": ctx.elapsed_ms(0, 1) / steps,
                         "spmm_ms": ctx.elapsed_ms(1, 2) / steps}
        for h in (S, dA, dB, dY, dC):
            h.close()
    return out


def run_dist_step(w, dtype, reps):
    """One step of the reference's distributed wrappers over device-resident operands
    (dist_sddmm_spcomm, dist_spmm_spcomm; src/distributed_comp.cpp:141-193,17-76): the
    host C++ program spcomm3d_amd/lib/dist_step_<real> reads the workload from a .bin file
    (the reference's format, tools/read_convert_mm.cpp:81-94) written here, and reports the
    wall-clock time per wrapper call beside the device time of the kernel inside it.  None
    when the program is not built."""
    import subprocess
    import tempfile

    exe = os.path.join(ROOT, "spcomm3d_amd", "lib", f"dist_step_{dtype}")
    if not os.path.exists(exe):
        return None
    rec = np.empty(w.nnz, dtype=np.dtype([("r", "<u4"), ("c", "<u4"), ("v", "<f8")]))
    rec["r"], rec["c"], rec["v"] = w.ii, w.jj, w.values("f64")
    with tempfile.TemporaryDirectory(dir="/dev/shm" if os.path.isdir("/dev/shm") else None) as d:
        path = os.path.join(d, "workload.bin")
        with open(path, "wb") as f:
            f.write(np.array([w.nrows, w.ncols], dtype="<u4").tobytes())
            f.write(np.array([w.nnz], dtype="<u8").tobytes())
            rec.tofile(f)
        del rec
        r = subprocess.run([exe, path, str(w.k), str(reps)], capture_output=True, text=True,
                           timeout=600)
    if r.returncode != 0:
        log(f"dist_step failed: {r.stderr[-500:]}")
        return None
    return json.loads(r.stdout.strip().splitlines()[-1])


def run_compact(w, dtype, steps, warmup):
    """One compact row for a workload: mean time per kernel over `steps` passes on
    resident operands, strict-model fraction of the HBM peak, the rows and columns that
    hold entries, and the device memory the plan takes."""
    from spcomm3d_amd import device, roofline
    from spcomm3d_amd import workloads as W

    wbytes = np.dtype(W.np_dtype(dtype)).itemsize
    vv = w.values(dtype)
    with device.Context(0) as ctx:
        hint = {} if w.k == 64 else {"k_hint": w.k}
        t0 = time.perf_counter()
        S = ctx.plan(w.nrows, w.ncols, w.ii, w.jj, vv, **hint)
        ctx.sync()
        plan_s = time.perf_counter() - t0
        del vv
        info = S.info
        dA, dB = ctx.panel_from(w.panel_A(dtype)), ctx.panel_from(w.panel_B(dtype))
        dY = ctx.panel_from(w.panel_Y0(dtype))
        dC = ctx.vals(w.nnz, dtype)
        for _ in range(warmup):
            ctx.sddmm(S, dA, dB, dC)
            ctx.spmm(S, dB, dY)
        ctx.sync()
        ctx.mark(0)
        for _ in range(steps):
            ctx.sddmm(S, dA, dB, dC)
        ctx.mark(1)
        for _ in range(steps):
            ctx.spmm(S, dB, dY)
        ctx.mark(2)
        sd_ms = ctx.elapsed_ms(0, 1) / steps
        sp_ms = ctx.elapsed_ms(1, 2) / steps
        for h in (S, dA, dB, dY, dC):
            h.close()
    m_t, n_t = info.rows_touched, info.cols_touched
    with_perm = not info.order_is_identity
    fl = roofline.flops(w.nnz, w.k)
    sd_b = roofline.sddmm_bytes(w.nrows, w.nnz, w.k, wbytes, m_t, n_t, with_perm)
    sp_b = roofline.spmm_bytes(w.nrows, w.nnz, w.k, wbytes, m_t, n_t)
    return {"workload": f"{w.name} K={w.k} ({w.order} COO)", "dtype": dtype, "nnz": w.nnz,
            "nrows": w.nrows, "ncols": w.ncols, "k": w.k, "steps": steps,
            "sddmm_ms": sd_ms, "spmm_ms": sp_ms,
            "sddmm_frac": sd_b / sd_ms / 1e6 / roofline.HBM_PEAK_GBS,
            "spmm_frac": sp_b / sp_ms / 1e6 / roofline.HBM_PEAK_GBS,
            "sddmm_strict_bytes": int(sd_b), "spmm_strict_bytes": int(sp_b),
            "rows_touched": m_t, "cols_touched": n_t,
            "plan_device_bytes": int(info.device_bytes), "col_blocks": int(info.ncol_blocks),
            "sweep_entries": int(info.sweep_entries),
            "gflops": 2 * fl / (sd_ms + sp_ms) / 1e6, "plan_build_s": plan_s}


# The other benchmark configurations as (name, real types, timed passes): the reference's own
# CPU-runnable case in its real type, the three larger ones in fp32 as they are specified,
# the stencil also in the reference's real type.
OTHER_CONFIGS = (("er16k", ("f64",), 50), ("rmat24_block", ("f32",), 10),
                 ("stencil4096", ("f32", "f64"), 10), ("hypergraph", ("f32",), 3))


def run_reference_baseline(w):
    """The reference's own core_ops.cpp (compiled into oracle/_ref where the
    reference tree was available; fp64 only, its real_t is a fixed macro) over
    the same workload: one SDDMM + SpMM pass on one core, timed inside the shim
    as the reference times its kernels.  None if that build is not there."""
    import ctypes

    from tests import _oracle as oracle

    if not oracle.have_ref():
        return None
    try:
        lib = ctypes.CDLL(oracle.REF_LIB)
        fn = lib.ref_time_f64
    except (OSError, AttributeError):
        return None
    fn.restype = ctypes.c_int
    fn.argtypes = ([ctypes.c_uint32] * 3 + [ctypes.c_void_p] * 3 + [ctypes.c_uint64] +
                   [ctypes.c_void_p] * 3 + [ctypes.POINTER(ctypes.c_double)] * 3)
    A, B, Y0, vv = w.panel_A("f64"), w.panel_B("f64"), w.panel_Y0("f64"), w.values("f64")
    vp = lambda a: a.ctypes.data_as(ctypes.c_void_p)  # noqa: E731
    ts, tp, cs = ctypes.c_double(), ctypes.c_double(), ctypes.c_double()
    if fn(w.nrows, w.ncols, w.k, vp(A), vp(B), vp(Y0), w.nnz, vp(w.ii), vp(w.jj), vp(vv),
          ctypes.byref(ts), ctypes.byref(tp), ctypes.byref(cs)) != 0:
        return None
    fl = 2 * w.nnz * w.k
    return {"value": 2 * fl / (ts.value + tp.value) / 1e9, "unit": "GFLOP/s", "cores": 1,
            "kind": "reference",
            "sample": f"one full SDDMM+SpMM pass of the reference's core_ops.cpp over {w.name} "
                      f"K={w.k} f64 ({w.order} COO, nnz={w.nnz})",
            "sddmm_s": ts.value, "spmm_s": tp.value,
            "sddmm_gflops": fl / ts.value / 1e9, "spmm_gflops": fl / tp.value / 1e9,
            "host_cores": os.cpu_count(), "flags": "g++ -O3 -ffp-contract=off"}


def run_cpu_baseline(w, dtype):
    """The CPU oracle (serial, one core, as the reference's per-rank path is:
    no threads anywhere in it) on the same workload, one SDDMM + SpMM pass."""
    import subprocess

    from tests import _oracle as oracle

    native = os.path.join(oracle.ORACLE_DIR, "liboracle_native.so")
    try:
        subprocess.run(["make", "-C", oracle.ORACLE_DIR, "liboracle_native.so"], check=True,
                       capture_output=True)
        lib = oracle.load(native)
        flags = "-O3 -march=native -ffp-contract=off"
    except Exception:  # noqa: BLE001 - any build problem: time the portable build instead
        lib = oracle.load()
        flags = "-O3 -ffp-contract=off"
    try:
        os.sched_setaffinity(0, {sorted(os.sched_getaffinity(0))[0]})
        pinned = True
    except OSError:
        pinned = False
    A, B, Y0, vv = w.panel_A(dtype), w.panel_B(dtype), w.panel_Y0(dtype), w.values(dtype)
    t0 = time.perf_counter()
    oracle.sddmm(A, B, w.ii, w.jj, vv, lib=lib)
    t1 = time.perf_counter()
    oracle.spmm(B, w.ii, w.jj, vv, Y0, lib=lib)
    t2 = time.perf_counter()
    fl = 2 * w.nnz * w.k
    return {"value": 2 * fl / (t2 - t0) / 1e9, "unit": "GFLOP/s", "cores": 1, "kind": "port",
            "sample": f"one full SDDMM+SpMM pass over {w.name} K={w.k} {dtype} "
                      f"({w.order} COO, nnz={w.nnz})",
            "sddmm_s": t1 - t0, "spmm_s": t2 - t1,
            "sddmm_gflops": fl / (t1 - t0) / 1e9, "spmm_gflops": fl / (t2 - t1) / 1e9,
            "host_cores": os.cpu_count(), "pinned": pinned, "flags": flags,
            "note": "spmm time includes one copy of Y (the oracle leaves its input intact)"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", default="rmat20", help="workload name (spcomm3d_amd.workloads)")
    ap.add_argument("--dtype", default="f64", choices=["f32", "f64"],
                    help="real type of the headline value (the reference's is f64)")
    ap.add_argument("--order", default="sorted", choices=["sorted", "shuffled", "column-major"],
                    help="order in which the COO entries are handed to the library")
    ap.add_argument("--seg-max", type=int, default=None)
    ap.add_argument("--localized", action="store_true",
                    help="the workload at the shape a rank of the reference runs it on: local "
                         "indices in first-appearance order, panels of the touched rows / "
                         "columns only")
    ap.add_argument("--col-blocks", type=int, default=None,
                    help="spc3d_plan_opts.col_blocks of the main workload's plan")
    ap.add_argument("--sweep", default=None, choices=["off", "on"],
                    help="spc3d_plan_opts.sweep of the main workload's plan (row tiles)")
    ap.add_argument("--calibration-copies", type=int, default=0,
                    help="also launch this many plain device copies of an m x K panel "
                         "(a known-size dispatch for counter calibration)")
    ap.add_argument("--floors", action="store_true",
                    help="only the all-hit / all-miss floors of the workload's launches "
                         "(they are part of the default run as well)")
    ap.add_argument("--no-floors", action="store_true", help="skip the floors")
    ap.add_argument("--no-dist", action="store_true",
                    help="skip the step through the device-resident dist_* wrappers")
    ap.add_argument("--only", action="store_true", help="skip the other real type")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-configs", action="store_true",
                    help="skip the shuffled-order runs and the rows of the other configurations")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path; run with --gpus 1")

    ensure_built()
    from spcomm3d_amd import workloads as W

    t0 = time.perf_counter()
    w = W.make(args.config)
    if args.order == "shuffled":
        w = w.shuffled()
    elif args.order == "column-major":
        w = w.column_major()
    if args.localized:
        w = w.localized()
    if args.col_blocks is not None:
        PLAN_OPTS["col_blocks"] = args.col_blocks
    if args.sweep is not None:
        PLAN_OPTS["sweep"] = args.sweep == "on"
    log(f"workload {w.name}: {w.nrows}x{w.ncols} nnz={w.nnz} K={w.k} order={w.order} "
        f"(generated in {time.perf_counter() - t0:.1f}s)")

    if args.floors:
        fl = {dt: run_floors(w, dt, max(5, args.steps // 2), args.warmup, args.seg_max)
              for dt in (("f64", "f32") if not args.only else (args.dtype,))}
        print(json.dumps({"workload": f"{w.name} K={w.k} ({w.order} COO)", "floors": fl}),
              flush=True)
        return

    main_r = run_gpu(w, args.dtype, args.steps, args.warmup, args.seg_max,
                     copies=args.calibration_copies)
    log(json.dumps(main_r))
    also = {}
    if not args.only:
        other = "f32" if args.dtype == "f64" else "f64"
        also[other] = run_gpu(w, other, args.steps, args.warmup, args.seg_max)
        log(json.dumps(also[other]))
    floors = None
    if not args.no_floors:
        floors = {dt: run_floors(w, dt, max(5, args.steps // 2), args.warmup, args.seg_max)
                  for dt in ((args.dtype,) if args.only else ("f64", "f32"))}
        log(json.dumps(floors))
    dist_step = None
    if not args.no_dist:
        dist_step = run_dist_step(w, args.dtype, max(5, args.steps // 2))
        log(json.dumps(dist_step))
    if not (args.only or args.no_configs):
        ws = w.shuffled() if w.order == "sorted" else None
        if ws is not None:
            also["shuffled"] = {dt: run_compact(ws, dt, max(5, args.steps // 2), args.warmup)
                                for dt in ("f64", "f32")}
            # unsorted COO is what the reference's kernels are handed (src/core_ops.cpp:7-10):
            # the same roofline object as the headline's, for that order
            r = also["shuffled"][args.dtype]
            sdom = "sddmm" if r["sddmm_ms"] >= r["spmm_ms"] else "spmm"
            also["shuffled"]["roofline"] = {
                "bound": "hbm", "kernel": sdom, "dtype": args.dtype,
                "achieved": r[sdom + "_strict_bytes"] / r[sdom + "_ms"] / 1e6,
                "peak": 8000.0, "unit": "GB/s", "frac": r[sdom + "_frac"],
                "bytes_per_launch": r[sdom + "_strict_bytes"], "ms_per_launch": r[sdom + "_ms"],
                "model": "strict (each operand once)"}
            log(json.dumps(also["shuffled"]))
            del ws
            wc = w.column_major()
            also["column_major"] = {dt: run_compact(wc, dt, max(5, args.steps // 2), args.warmup)
                                    for dt in ("f64", "f32")}
            log(json.dumps(also["column_major"]))
            del wc
        rows = []
        for name, dtypes, steps in OTHER_CONFIGS:
            if name == args.config:
                continue
            t0 = time.perf_counter()
            wo = W.make(name)
            for dt in dtypes:
                row = run_compact(wo, dt, steps, 2)
                row["wall_s"] = time.perf_counter() - t0
                rows.append(row)
                log(json.dumps(row))
                t0 = time.perf_counter()
            if name == "rmat24_block":
                # the same block at the shape a rank of the reference runs it on: local
                # indices in first-appearance order, panels of the touched rows / columns only
                # (src/SparseMatrix.hpp:69-99, miniapp/bench_both.cpp:158,189-190)
                wl = wo.localized()
                for dt in dtypes:
                    row = run_compact(wl, dt, steps, 2)
                    row["wall_s"] = time.perf_counter() - t0
                    rows.append(row)
                    log(json.dumps(row))
                    t0 = time.perf_counter()
                del wl
            del wo
        also["configs"] = rows
    cpu = None
    if not args.no_cpu:
        port = run_cpu_baseline(w, args.dtype)
        ref = run_reference_baseline(w) if args.dtype == "f64" else None
        cpu = dict(ref, port=port) if ref else port

    dom = max(main_r["kernels"], key=lambda k: main_r["kernels"][k]["ms_avg"])
    kd = main_r["kernels"][dom]
    from spcomm3d_amd import roofline

    traffic = None
    traffic_stale = False
    if (args.seg_max is None and not PLAN_OPTS
            and not any(k.startswith("SPC3D_") for k in os.environ)
            and (w.name, w.k, w.order) == TRAFFIC_WORKLOAD):
        if traffic_is_current():
            traffic = measured_traffic().get((args.dtype, dom))
        else:  # recorded on other device code than this: not this code's traffic
            traffic_stale = True

    line = {
        "metric": METRIC, "value": main_r["gflops"], "unit": "GFLOP/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": main_r["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": args.dtype,
        "data": "synthetic",
        "config": {"workload": f"{w.name} K={w.k} ({w.order} COO)", "nrows": w.nrows,
                   "ncols": w.ncols, "nnz": w.nnz, "k": w.k, "step": "SDDMM then SpMM",
                   "rows_touched": main_r["rows_touched"], "cols_touched": main_r["cols_touched"]},
        "roofline": {"bound": "hbm", "kernel": dom, "achieved": kd["strict_gbs"],
                     "peak": roofline.HBM_PEAK_GBS, "unit": "GB/s", "frac": kd["strict_frac"],
                     "traffic": traffic, "traffic_stale": traffic_stale,
                     "traffic_level": TRAFFIC_LEVEL,
                     "traffic_source": os.path.relpath(TRAFFIC_PROFILE, ROOT),
                     "traffic_gbs": None if traffic is None else traffic / kd["ms_avg"] / 1e6,
                     "device_copy_gbs": main_r["device_copy_gbs"],
                     "frac_of_device_copy": kd["strict_gbs"] / main_r["device_copy_gbs"],
                     "traffic_frac_of_device_copy": None if traffic is None else
                     traffic / kd["ms_avg"] / 1e6 / main_r["device_copy_gbs"],
                     "floor_all_hit_ms": None if floors is None else
                     floors[args.dtype]["all_hit"][dom + "_ms"],
                     "floor_all_miss_ms": None if floors is None else
                     floors[args.dtype]["all_miss"][dom + "_ms"],
                     "floors": floors,
                     "bytes_per_launch": kd["strict_bytes"],
                     "ms_per_launch": kd["ms_avg"], "model": "strict (each operand once)"},
        "cpu_baseline": cpu,
        "kernels": main_r["kernels"],
        "fused_step": main_r["fused_step"],
        "dist_step": dist_step,
        "row_copies": main_r["row_copies"],
        "plan": {k: main_r[k] for k in ("plan_build_s", "upload_s", "nsegments", "nsplit_rows",
                                        "seg_max", "plan_device_bytes", "col_blocks",
                                        "sweep_entries", "sweep_tiles", "staged_entries")},
        "also": also,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
