"""bench.py's command line and its one JSON line: the keys a driver reads, the two extra objects,
and the refusal of more than one GPU."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused_with_a_message():
    p = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, cwd=ROOT)
    assert p.returncode != 0
    assert "one GPU" in p.stderr and "--gpus 2" in p.stderr
    assert p.stdout.strip() == ""  # no JSON line that a driver could take for a measurement


def test_without_a_gpu_the_bench_fails_instead_of_measuring_the_cpu():
    import torch
    if torch.cuda.is_available():
        pytest.skip("needs a machine without a GPU")
    p = subprocess.run([sys.executable, BENCH, "--steps", "2", "--warmup", "1"], capture_output=True, text=True,
                       cwd=ROOT)
    assert p.returncode != 0
    assert p.stdout.strip() == ""


@pytest.mark.gpu
def test_json_line_has_the_contract_keys(gpu_device):
    p = subprocess.run([sys.executable, BENCH, "--steps", "20", "--warmup", "4", "--cpu-seconds", "1"],
                       capture_output=True, text=True, cwd=ROOT, timeout=170)
    assert p.returncode == 0, p.stderr[-2000:]
    lines = [ln for ln in p.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1, lines
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline", "two_launches", "cold",
                "workloads", "workloads_geomean", "moe_layer"):
        assert key in d, key
    # the form that runs around a real expert, the cold-cache protocol of the reference's harness, every
    # named workload and the expert layer are part of the one line
    assert d["two_launches"]["dispatch_combine_us"] >= d["dispatch_combine_us"] - 0.5
    assert 0 < d["cold"]["pct_of_hbm_peak"] < 100 and d["cold"]["steps"] <= 30
    assert set(d["workloads"]) == {"tiny", "dsv3_rank", "skew_world", "fp8_dispatch", "prefill_graph"}
    for name, w in d["workloads"].items():
        assert 0 < w["pct_of_hbm_peak"] < 100 and 0 < w["roofline_frac"] < 1 and w["launches_per_step"] >= 1, name
        assert w["ms_per_step"] * 1e3 >= w["dispatch_combine_us"] - 0.01, name
        if name != "dsv3_rank":
            assert w["gpu_output_bit_identical"] is True, name
    assert d["workloads"]["dsv3_rank"]["dispatch_combine_us"] == d["dispatch_combine_us"]
    m = d["moe_layer"]
    assert m["combine_bit_identical_to_oracle_on_gpu_expert_rows"] is True
    assert m["expert_rows_worst_error_of_tolerance"] <= 1.0 and m["experts_checked"] >= 1
    # two measurements of the same steps (whole steps on the wall clock, kernels by their own events):
    # they agree to within the clocks' drift
    assert m["wall_us_per_step"] >= 0.95 * m["expert_gemm"]["us"]
    assert d["n_gpus"] == 1 and d["steps"] == 20 and d["warmup"] == 4
    assert d["unit"] == "GB/s" and d["higher_is_better"] is True and d["vs_baseline"] is None
    assert d["data"] == "synthetic" and d["dtype"] == "bf16"
    assert d["config"]["workload"] == "dsv3_rank" and "model" not in d["config"]
    r = d["roofline"]
    assert r["bound"] == "hbm" and r["peak"] == 8000.0 and r["unit"] == "GB/s"
    assert abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-3
    assert r["traffic"] is None or r["traffic"] > 0
    assert isinstance(r["traffic_source"], str) and r["traffic_source"]
    # the headline times what custom_kernel runs, and says how many launches that is
    assert d["config"]["fused_stub"] is True and d["config"]["launches_per_step"] >= 1
    # the figure cannot beat the memory system; a step's wall time holds its kernels and their launch
    # overhead, so the period-based figure cannot beat the kernels' own durations either
    assert 0 < d["value"] < 8000.0
    assert d["ms_per_step"] * 1e3 >= d["dispatch_combine_us"] - 0.01
    assert d["dispatch_combine_us"] >= d["kernel_only"]["dispatch_combine_us"] - 0.01
    assert abs(r["avg_us"] - (r["kernel_only_us"] + d["launch_overhead_us_per_launch"])) < 0.01
    c = d["cpu_baseline"]
    assert c["kind"] in ("port", "reference") and c["cores"] >= 1 and c["value"] > 0 and c["sample"]
    assert c["gpu_output_bit_identical"] is True


def test_traffic_record_counts_only_for_the_sources_it_was_measured_on(tmp_path):
    """roofline.traffic comes from profiles/traffic.json and is null, with the reason, unless the
    record names this workload and kernel and was taken on the present kernel sources."""
    sys.path.insert(0, ROOT)
    import bench

    now = bench.kernel_source_hash()
    rec = dict(factor=dict(FETCH_SIZE=2.0, WRITE_SIZE=1.0),
               entries=[dict(workload="dsv3_rank", kernel="forward_token", symbol="forward_token_kernel<...>",
                             fetch_kib=100.0, write_kib=200.0, bytes=409600, source_hash=now, commit="abc"),
                        dict(workload="skew_world", kernel="combine_rows", fetch_kib=1.0, write_kib=1.0, bytes=3072,
                             source_hash="0000000000000000", commit="abc")])
    path = tmp_path / "traffic.json"
    path.write_text(json.dumps(rec))
    got, why = bench.measured_traffic("dsv3_rank", "forward_token", str(path))
    assert got == 409600 and "profiles/traffic.json" in why and now in why
    got, why = bench.measured_traffic("skew_world", "combine_rows", str(path))
    assert got is None and "other kernel sources" in why  # stale: measured on different code
    got, why = bench.measured_traffic("dsv3_rank", "route_dispatch", str(path))
    assert got is None and "no record" in why
    got, why = bench.measured_traffic("dsv3_rank", "forward_token", str(tmp_path / "missing.json"))
    assert got is None and "missing" in why
    # the committed record, if there is one, parses and names its sources
    if os.path.exists(bench.TRAFFIC_FILE):
        for e in json.load(open(bench.TRAFFIC_FILE))["entries"]:
            assert {"workload", "kernel", "bytes", "source_hash", "commit", "fetch_kib", "write_kib"} <= set(e)


@pytest.mark.gpu
def test_gemm_rs_leg_prints_one_line_per_shape_with_its_roofline(gpu_device):
    p = subprocess.run([sys.executable, BENCH, "--gemm-rs", "512,4096,12288,bias", "--steps", "5", "--warmup", "1",
                        "--cpu-seconds", "1"], capture_output=True, text=True, cwd=ROOT, timeout=110)
    assert p.returncode == 0, p.stderr[-2000:]
    lines = [ln for ln in p.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1, lines
    d = json.loads(lines[0])
    assert d["unit"] == "TFLOP/s" and d["n_gpus"] == 1 and d["dtype"] == "bf16" and d["data"] == "synthetic"
    c = d["config"]
    assert c["workload"] == "gemm_rs" and (c["m"], c["n"], c["k"]) == (512, 4096, 12288) and c["emulated_ranks"] == 8
    assert c["has_bias"] is True and "model" not in c
    r = d["roofline"]
    assert r["bound"] in ("mfma", "hbm") and 0 < r["frac"] < 1 and abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-3
    assert 0 < d["value"] < 2500.0  # below the dense bf16 peak
    assert abs(d["value"] - 2.0 * 512 * 4096 * 12288 / d["kernel_us"] / 1e6) < 0.5
    assert d["reference_speed_of_light_us_per_gpu_of_8"] == 8.19
    cb = d["cpu_baseline"]
    assert cb["kind"] == "port" and cb["cores"] >= 1 and cb["value"] > 0 and cb["sample"]
