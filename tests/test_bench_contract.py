"""The benchmark's command-line contract: what can be checked without a GPU, and the JSON
line itself on a GPU (a short run on the smallest workload)."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_traffic_figure_comes_from_the_tracked_profile_and_is_tied_to_the_kernel_sources(tmp_path):
    sys.path.insert(0, ROOT)
    import bench
    rows = bench.read_traffic_profile()
    assert "c2_interleaved" in rows
    text = open(bench.TRAFFIC_PROFILE).read()
    for name, rec in rows.items():
        line = next(ln for ln in text.splitlines() if ln.startswith("| " + name + " "))
        cells = [c.strip() for c in line.strip("|").split("|")]
        assert rec["bytes"] == int((float(cells[1]) * float(cells[2]) + float(cells[3]) * float(cells[4])) * 1024)
        assert rec["kernel_source_hash"] == cells[5]
        # compulsory bytes of c2: Q, K, V, O of [2, 32, 4096, 128] 16-bit: the counters cannot show less
        if name == "c2_interleaved":
            assert rec["bytes"] >= 4 * 2 * 32 * 4096 * 128 * 2
    value, prov = bench.traffic_for("c2_interleaved")
    assert prov["kernel_source_hash"] == bench.kernel_source_hash()
    if prov["measured_at_head"]:
        assert value == rows["c2_interleaved"]["bytes"]
    else:
        assert value is None and prov["stale_bytes"] == rows["c2_interleaved"]["bytes"]
    assert bench.traffic_for("no_such_workload")[0] is None
    # a row with another hash is never reported
    p = tmp_path / "t.md"
    p.write_text("| c2_interleaved | 10 | 2.0 | 5 | 1.0 | 0123456789abcdef |\n")
    assert bench.read_traffic_profile(str(p))["c2_interleaved"]["bytes"] == 25 * 1024


@pytest.mark.gpu
def test_json_line_has_the_contract_fields(gpu_device):
    r = subprocess.run([sys.executable, BENCH, "--workload", "c1_causal", "--steps", "5", "--warmup", "2",
                        "--cpu-budget-s", "1"], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [ln for ln in r.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better",
                "scaling", "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 5 and d["warmup"] == 2 and d["vs_baseline"] is None
    assert d["clock_settle"]["launches"] > 0 and d["clock_settle"]["ms"] >= 250.0
    assert d["unit"] == "TFLOP/s" and d["dtype"] in ("bf16", "f16") and d["data"] == "synthetic"
    assert "workload" in d["config"] and "model" not in d["config"]
    rf = d["roofline"]
    assert rf["bound"] == "mfma" and rf["unit"] == "TFLOP/s" and rf["peak"] == 2500.0
    assert abs(rf["frac"] - rf["achieved"] / rf["peak"]) < 1e-12 and "traffic" in rf
    assert 500.0 < rf["measured_mfma_peak"] < 2600.0 and "measured_at_head" in rf["traffic_provenance"]
    cb = d["cpu_baseline"]
    assert cb["kind"] == "port" and cb["cores"] >= 1 and cb["value"] > 0 and cb["sample"]
    assert d["from_idle"]["steps"] == 5 and d["from_idle"]["warmup"] == 2 and d["from_idle"]["value"] > 0
    for name in ("c1_causal", "c2_interleaved"):
        op = d["operator"][name]
        assert op["operator_ms_per_call"] >= op["kernel_ms"] * 0.9 and op["capi_ms_per_call"] > 0


def test_reference_flop_count_reproduces_the_reference_printed_figures():
    """The dense-equivalent flop count of bench.py --reference-grid against figures the reference
    printed with its own (omni_attention_report.pdf, appendix: seq 2048, B=1 H=8 D=64: swizzle
    0.31 ms = 28.10 TFLOPS, shared_kv 0.48 ms = 18.39, simple 66.68 ms = 0.13; ms.md:19-24: seq 1024,
    shared_kv 0.25 ms = 8.73).  The times are printed to two digits, hence the intervals."""
    import bench
    f2048 = bench.reference_dense_flops(1, 8, 2048, 64)
    f1024 = bench.reference_dense_flops(1, 8, 1024, 64)
    assert f2048 / 0.315e-3 / 1e12 <= 28.10 <= f2048 / 0.305e-3 / 1e12
    assert f2048 / 0.485e-3 / 1e12 <= 18.39 <= f2048 / 0.475e-3 / 1e12
    assert abs(f2048 / 66.68e-3 / 1e12 - 0.13) < 0.005
    assert f1024 / 0.255e-3 / 1e12 <= 8.73 <= f1024 / 0.245e-3 / 1e12
    assert set(bench.REFERENCE_GRID_PUBLISHED) == {"causal", "interleaved"}


@pytest.mark.gpu
def test_reference_grid_mode_covers_the_published_table(gpu_device):
    r = subprocess.run([sys.executable, BENCH, "--reference-grid"], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    d = json.loads(r.stdout.strip().splitlines()[-1])
    assert len(d["rows"]) == 12
    assert {(x["mask"], x["seq_len"], x["block"]) for x in d["rows"]} == {
        (m, s, b) for m in ("causal", "interleaved") for s in (512, 1024, 2048) for b in (64, 128)}
    for x in d["rows"]:
        assert x["listed_blocks"] > 0 and 0 < x["kernel_ms_median"] <= x["wall_ms_one_call"]
        assert x["effective_tflops_kernel"] <= x["dense_equivalent_tflops_kernel"] * 1.01

