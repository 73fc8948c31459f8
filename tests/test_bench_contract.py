"""The contract of bench.py and __graft_entry__ that can be checked without a GPU."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_bench_refuses_more_than_one_gpu():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_entry_points_exist():
    sys.path.insert(0, ROOT)
    import __graft_entry__ as g

    assert callable(g.build) and callable(g.smoke)


def test_byte_models_of_the_roofline():
    from spcomm3d_amd import roofline

    # R-MAT 20, K = 64, fp64, with the output permutation read: the figures the bench line
    # and the profiles quote
    nnz, m, mt, nt = 16086740, 1048576, 547169, 547037
    sd = roofline.sddmm_bytes(m, nnz, 64, 8, mt, nt, True)
    sp = roofline.spmm_bytes(m, nnz, 64, 8, mt, nt)
    fz = roofline.fused_bytes(m, nnz, 64, 8, mt, nt, True)
    index = 4 * (m + 1) + 4 * nnz
    assert sd == index + 4 * nnz + 2 * 8 * nnz + 8 * 64 * (mt + nt) == 950509540
    assert sp == index + 8 * nnz + 8 * 64 * nt + 2 * 8 * 64 * mt == 1037619188
    assert fz == sd + 2 * 8 * 64 * mt
    assert roofline.flops(nnz, 64) == 2 * nnz * 64


def test_traffic_in_the_bench_line_is_what_the_profile_summary_holds():
    """bench.py quotes the measured L2 <-> fabric traffic from the committed profile
    summary: the 'Per call' table must parse, add up from the per-launch table of the same
    file, and lie between the strict and the gather model."""
    import re

    sys.path.insert(0, ROOT)
    import bench
    from spcomm3d_amd import roofline

    got = bench.measured_traffic()
    assert set(got) == {(d, c) for d in ("f32", "f64") for c in ("sddmm", "spmm", "sddmm_spmm")}
    text = open(bench.TRAFFIC_PROFILE).read()
    per_launch = text.split("Per call", 1)[0]
    rows = re.findall(r"^\|\s*(f32|f64)\s*\|\s*`(\w+)<([^`]*)>`\s*\|[^|]*\|[^|]*\|[^|]*\|[^|]*\|"
                      r"\s*([\d,\.]+)\s*\|", per_launch, re.M)
    assert len(rows) >= 16
    total = {}
    for dtype, kernel, targs, mb in rows:
        mb = float(mb.replace(",", ""))
        fused = kernel.startswith("sddmm") and targs.strip().endswith("1")
        call = "sddmm_spmm" if fused else ("sddmm" if kernel.startswith("sddmm") else "spmm")
        if kernel == "unstage_pairs_kernel":  # ends the SDDMM and the one-pass call alike
            call = "sddmm"
            total[(dtype, "sddmm_spmm")] = total.get((dtype, "sddmm_spmm"), 0.0) + mb * 1e6
        total[(dtype, call)] = total.get((dtype, call), 0.0) + mb * 1e6
        if kernel == "spmm_fixup_kernel":  # the one-pass call ends with the same fix-up
            total[(dtype, "sddmm_spmm")] = total.get((dtype, "sddmm_spmm"), 0.0) + mb * 1e6
    nnz, m, mt, nt = 16086740, 1048576, 547169, 547037
    for (dtype, call), traffic in got.items():
        assert abs(total[(dtype, call)] - traffic) <= 0.002 * traffic, (dtype, call)
        w = 8 if dtype == "f64" else 4
        strict = {"sddmm": roofline.sddmm_bytes(m, nnz, 64, w, mt, nt, True),
                  "spmm": roofline.spmm_bytes(m, nnz, 64, w, mt, nt),
                  "sddmm_spmm": roofline.fused_bytes(m, nnz, 64, w, mt, nt, True)}[call]
        gather = roofline.fused_bytes(m, nnz, 64, w, mt, nt, True, gather=True)
        assert strict < traffic < gather, (dtype, call)
    assert "l2_fabric" in bench.TRAFFIC_LEVEL


def test_profiles_were_recorded_on_the_device_code_in_the_tree():
    """Every summary under profiles/ names the digest of the device sources it was recorded
    on; a change to those sources makes the summaries stale, this test fail and bench.py
    report `traffic: null, traffic_stale: true` until they are recorded again."""
    sys.path.insert(0, ROOT)
    import bench
    from spcomm3d_amd import provenance

    now = provenance.source_hash()
    names = sorted(n for n in os.listdir(os.path.join(ROOT, "profiles")) if n.endswith(".md"))
    assert names
    stale = [n for n in names
             if provenance.recorded_hash(os.path.join(ROOT, "profiles", n)) != now]
    assert not stale, f"recorded on other sources than {now}: {stale}"
    assert bench.traffic_is_current()


def test_a_stale_profile_is_not_quoted(tmp_path):
    sys.path.insert(0, ROOT)
    import bench

    text = open(bench.TRAFFIC_PROFILE).read()
    old = tmp_path / "traffic.md"
    old.write_text(text.replace("Source hash: `", "Source hash: `0"))
    assert bench.measured_traffic(str(old))  # the table still parses
    assert not bench.traffic_is_current(str(old))
    none = tmp_path / "none.md"
    none.write_text("# no digest in here\n")
    assert not bench.traffic_is_current(str(none))


@pytest.mark.gpu
def test_bench_line_has_the_contract_fields():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--config", "er16k",
                        "--steps", "5", "--warmup", "1", "--no-configs"], capture_output=True,
                       text=True,
                       timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [ln for ln in r.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step",
              "higher_is_better", "scaling", "vs_baseline", "dtype", "data", "config", "roofline",
              "cpu_baseline"):
        assert k in d, k
    assert d["n_gpus"] == 1 and d["steps"] == 5 and d["vs_baseline"] is None
    assert d["dtype"] == "f64" and "workload" in d["config"]
    assert set(("bound", "achieved", "peak", "unit", "frac", "traffic", "traffic_stale",
                "traffic_level")) <= set(d["roofline"])
    assert d["roofline"]["bound"] == "hbm" and d["roofline"]["peak"] == 8000.0
    assert abs(d["roofline"]["frac"] - d["roofline"]["achieved"] / 8000.0) < 1e-12
    assert set(("value", "unit", "cores", "kind", "sample")) <= set(d["cpu_baseline"])
    assert d["cpu_baseline"]["kind"] in ("reference", "port")
