"""The line bench.py prints: one JSON object with the fields the driver reads, on a small workload."""

from __future__ import annotations

import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench(*flags, timeout=300):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *flags], cwd=ROOT, capture_output=True, text=True,
                          timeout=timeout)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = _bench("--gpus", "2")
    assert r.returncode != 0 and not r.stdout.strip()
    assert "one GPU" in r.stderr


@pytest.mark.gpu
def test_bench_line_has_the_contract_fields(gpu_device):
    r = _bench("--workload", "moe_experts_row_parallel_w2", "--steps", "3", "--warmup", "1", "--cpu-seconds", "1")
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1, "exactly one line on stdout"
    d = json.loads(lines[0])
    assert d["n_gpus"] == 1 and d["steps"] == 3 and d["warmup"] == 1
    assert d["higher_is_better"] is True and d["scaling"] == "weak" and d["vs_baseline"] is None and d["data"] == "synthetic"
    assert d["unit"] == "GB/s" and d["value"] > 0 and d["ms_per_step"] > 0
    assert d["config"]["workload"] == "moe_experts_row_parallel_w2" and "model" not in d["config"]
    assert abs(d["value"] - d["config"]["payload_bytes"] / (d["ms_per_step"] * 1e-3) / 1e9) < 0.01 * d["value"]
    assert d["device_ms_per_step"] <= d["ms_per_step"] * 1.01
    roof = d["roofline"]
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0 and roof["unit"] == "GB/s"
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3 and 0 < roof["frac"] < 1
    assert roof["traffic"] is None or roof["traffic"] > 0
    cpu = d["cpu_baseline"]
    assert cpu["kind"] == "port" and cpu["unit"] == "GB/s" and cpu["cores"] >= 1 and cpu["value"] > 0 and cpu["sample"]
    assert "extra_legs_error" not in d


@pytest.mark.gpu
def test_default_line_carries_every_configuration(gpu_device):
    """The default run (the one the driver makes): the headline on config 2 plus one entry per other configuration,
    the copy ceiling, the counter-derived HBM rate and the two legs that run in worker processes."""
    r = _bench("--steps", "20", "--warmup", "3", "--cpu-seconds", "2", timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    assert d["config"]["workload"] == "llama3_8b_fsdp8_to_tp2" and d["steps"] == 20 and d["warmup"] == 3
    assert "extra_legs_error" not in d
    wl = d["workloads"]
    assert set(wl) == {"single_fp32_shard0_to_shard1", "many_small_2d_to_replicate", "partial4_to_shard2",
                       "moe_experts_and_uneven_vocab", "llama3_8b_fsdp8_to_tp2_fp32_to_bf16", "transposed_parents",
                       "partial4_transposed_to_shard2"}
    for name, w in wl.items():
        assert "error" not in w, (name, w)
        assert w["steps"] >= 20 and w["warmup"] >= 3
        for key in ("device_ms_per_step", "algorithmic_bytes_per_step", "pct_of_hbm_peak", "effective_GB/s", "launches_per_step"):
            assert w[key] > 0, (name, key)
        assert abs(w["pct_of_hbm_peak"] - 100 * w["algorithmic_bytes_per_step"] / (w["device_ms_per_step"] * 1e-3) / 8e12) < 0.05
        assert w["pct_of_hbm_peak"] < 100
    assert wl["partial4_to_shard2"]["algorithmic_bytes_per_step"] == 7 * (1 << 30)  # 4 reads + 1 write, then unpack 1 + 1
    for leg in ("bf16_to_bf16", "fp32_to_bf16"):
        c = d["copy_ceiling"][leg]
        assert 0 < c["pct_of_hbm_peak"] < 100 and c["bytes_read"] == 4 << 30
    roof = d["roofline"]
    detail = roof["traffic_detail"]
    if detail is not None:
        assert isinstance(detail["stale"], bool) and detail["running_library_digest"]
        assert abs(roof["hbm_GB/s"] - (detail["fetch_bytes_per_step"] + detail["write_bytes_per_step"]) / (d["device_ms_per_step"] * 1e-3) / 1e9) < 1
    for leg in ("two_process_wire", "bus_end_to_end"):
        assert "error" not in d[leg], d[leg]
        assert d[leg]["ms_per_transfer"] > 0 and d[leg]["effective_GB/s"] > 0
    assert d["two_process_wire"]["pool"] == "ring" and d["two_process_wire"]["bit_equal_target_tensors"] == 290
    assert d["two_process_wire"]["pool_reserved_bytes"] < d["config"]["payload_bytes"] // 4
