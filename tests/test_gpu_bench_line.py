"""The driver's bench command, at a few steps: one JSON line that carries BASELINE's headline configuration and,
under "configs", the long-context, fp8 and growth-and-swap configurations, the last one with its swap events
inside the run and a bit-exact check of every swapped byte (BASELINE.json configs[2..4])."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_bench_line_carries_every_configuration():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "1", "--steps", "3", "--warmup", "1",
                        "--repeats", "1", "--other-repeats", "1", "--cpu-seconds", "1"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    line = json.loads(r.stdout.strip().splitlines()[-1])
    assert line["n_gpus"] == 1 and line["unit"] == "GB/s" and line["vs_baseline"] is None
    assert line["config"]["workload"].startswith("llama3-8b-decode-bf16 B=64")
    roof = line["roofline"]
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0 and 0.3 < roof["frac"] < 1.0
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3 and roof["traffic_replayed_from_profile"] is True
    assert line["algorithmic_bytes_per_step"] > 5e8
    assert line["cpu_baseline"]["kind"] in ("reference", "port") and line["cpu_baseline"]["cores"] >= 1
    others = line["configs"]
    assert sorted(others) == ["c3", "c4", "c5"]
    for name in ("c3", "c4"):
        assert others[name]["value"] > 1000 and 0.3 < others[name]["roofline"]["frac"] < 1.0
    c5 = others["c5"]
    assert c5["steps"] == 64 and len(c5["blocks_gbps"]) == 4 and c5["value"] > 1000
    assert [e["after_step"] for e in c5["swap_events"]] == [16, 32, 48, 64]
    assert all(e["sequences"] == 64 and e["bytes_per_direction"] > 2e8 and e["out_gbps"] > 5 and e["in_gbps"] > 5
               for e in c5["swap_events"])
    assert c5["bit_exact"] is True and c5["swapped_bytes_checked"] > 1e9 and c5["appended_rows_checked"] == 256 * 64 * 2
    assert c5["chunks_mapped_while_growing"] > 0


def test_bench_line_of_the_float32_configuration():
    # BASELINE.json configs[0] (fp32, 8 sequences of 128..1024 rows) through the float32 kernels
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "1", "--config", "c1", "--steps", "3",
                        "--warmup", "1"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    line = json.loads(r.stdout.strip().splitlines()[-1])
    assert line["dtype"] == "f32" and line["unit"] == "GB/s" and line["n_gpus"] == 1 and line["value"] > 10
    assert line["config"]["workload"].startswith("fp32 B=8") and line["roofline"]["bound"] == "hbm"
    assert 2e7 < line["algorithmic_bytes_per_step"] < 5e7
