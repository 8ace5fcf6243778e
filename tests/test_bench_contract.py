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
