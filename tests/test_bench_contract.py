"""bench.py's command line and the one JSON line it prints."""
import json
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0
    assert "one GPU" in r.stderr
    assert r.stdout.strip() == ""


def test_committed_profile_summaries_give_the_traffic_figures():
    sys.path.insert(0, str(ROOT))
    import bench

    for name in ("flash_attention_B8_H32_N4096_d128_bf16.md", "row_softmax_16384x4096_f32.md",
                 "gemm_nt_4096x4096x4096_bf16.md", "flash_attention_B1_H16_N32768_d64_bf16.md",
                 "flash_attention_B2_H32_N4096_d128_f32.md"):
        traffic = bench.measured_traffic(name)
        assert isinstance(traffic, int) and traffic > 0, name
    assert bench.measured_traffic("no_such_summary.md") is None


@pytest.mark.gpu
def test_one_json_line_with_roofline_and_cpu_baseline():
    r = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--steps", "2", "--warmup", "1"],
                       capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [ln for ln in r.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1
    rec = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in rec, key
    assert rec["n_gpus"] == 1 and rec["steps"] == 2 and rec["warmup"] == 1
    assert rec["unit"] == "TFLOP/s" and rec["dtype"] == "bf16" and rec["vs_baseline"] is None
    assert "workload" in rec["config"] and "model" not in rec["config"]
    roof = rec["roofline"]
    assert roof["bound"] == "mfma" and roof["unit"] == "TFLOP/s" and roof["peak"] == 2500.0
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-9
    cpu = rec["cpu_baseline"]
    assert cpu["kind"] == "port" and cpu["form"].startswith("emitted-c") and cpu["cores"] == 1 and cpu["value"] > 0 and cpu["sample"] and cpu["host_cpu"]
    assert rec["pre_warmup_launches"] == 41 and rec["rel_err"] <= 2e-2
    assert rec["roofline"]["kernel"] == "attn_fwd_bf16_d128_bn64_direct_w8"
    # the clock the kernel counted for itself, and the committed profile's cycles at that clock against the measured time
    assert 1.0 < roof["shader_clock_ghz"] < 2.6
    assert abs(roof["frac_at_measured_clock"] - roof["frac"] * 2.4 / roof["shader_clock_ghz"]) < 1e-9
    assert 0.85 < roof["kernel_ms_measured_over_predicted"] < 1.2
    assert rec["library_gemm_probe"] is None  # (timed from 20 steps on)
    second = rec["secondary"]
    assert len(second) == 8
    host = second[6]  # (the host entry point: PCIe-inclusive, never the headline)
    assert "i_exec_into" in host["workload"] and host["pcie_GBps"] > 0 and host["rel_err_against_f64"] <= 1e-4
    one_head = second[7]  # (one head on its own: its keys in parts over workgroups, beside the same call unsplit)
    assert "(keys in " in one_head["launches"] and one_head["ms_per_call_unsplit"] > 0 and one_head["rel_err_against_unsplit"] <= 2e-3
    for entry, bar in zip(second, (1e-4, 1e-4, 2e-2, 2e-2, 1e-4, 1e-4)):
        assert entry["cpu_baseline"]["value"] > 0 and entry["rel_err"] <= bar, entry["workload"]
    c5 = second[3]
    assert c5["second_bound"]["binds"] in ("mfma", "valu") and 0.5 < c5["second_bound"]["frac_of_sum_of_bounds_at_measured_clock"] < 1.3
    f32_line = second[5]
    assert f32_line["dtype"] == "f32" and f32_line["roofline"]["peak"] == 157.3
    assert f32_line["roofline"]["kernel"] == "attn_fwd_f32_d128_bn32_direct"
    # the value is work over wall time of exactly `steps` calls
    flop = 4.0 * 8 * 32 * 4096 * 4096 * 128
    assert abs(rec["value"] - flop / (rec["ms_per_step"] * 1e-3) / 1e12) / rec["value"] < 1e-6
