"""bench.py's output contract, on the GPU: one JSON line whose headline comes from exactly the
warm-up and step counts asked for, with the settled sweep, the sustained prefill figures and the
roofline beside it; and the ceiling probes' JSON."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args, timeout=300):
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], cwd=ROOT, capture_output=True,
                         text=True, timeout=timeout)
    assert res.returncode == 0, res.stderr[-2000:]
    lines = [l for l in res.stdout.splitlines() if l.strip()]
    assert len(lines) == 1, res.stdout[-2000:]
    return json.loads(lines[0])


def test_bench_line_follows_the_flags_it_was_given():
    d = _run("--no-cpu", "--no-decoder", "--warmup", "2", "--steps", "3")
    assert d["n_gpus"] == 1 and d["steps"] == 3 and d["warmup"] == 2
    assert d["unit"] == "GB/s" and d["higher_is_better"] is True and d["vs_baseline"] is None
    assert d["config"]["workload"].startswith("decode GEMV sweep")
    # value and ms_per_step describe the same run
    step_bytes = d["config"]["bytes_per_step"]
    assert abs(step_bytes / (d["ms_per_step"] * 1e-3) / 1e9 - d["value"]) <= 0.01 * d["value"]
    assert 0.0 < d["value"] < 8000.0
    r = d["roofline"]
    assert r["bound"] == "hbm" and r["peak"] == 8000.0 and r["unit"] == "GB/s"
    assert abs(r["achieved"] / r["peak"] - r["frac"]) < 1e-3
    assert abs(r["bytes_per_launch"] / (r["avg_launch_us"] * 1e-6) / 1e9 - r["achieved"]) <= 0.01 * r["achieved"]
    # the clock-settled sweep is reported under its own key, with what ran before it
    s = d["settled"]
    assert s["untimed_steps"] == 50 and s["steps"] == 3 and s["value"] > 0
    assert d["other_qweight_rows"]["rows"] == "contiguous"
    assert len(d["decode_points"]) == 16 and "launch" in d["decode_points_note"]
    pf = d["prefill"]
    assert len(pf["points"]) == 12
    for p in pf["points"]:
        assert p["TFLOPs"] > 0 and p["TFLOPs_burst"] > 0
        assert p["form"] == ("fused" if p["M"] < 2048 else "dequantise once + dense")
    assert 0.0 < pf["aggregate"] < 2500.0 and 0.0 < pf["aggregate_burst"] < 2500.0
    assert [p["T"] for p in d["moe"]["points"]] == [1, 16, 128, 512]


def test_mfma_probe_prints_both_instruction_shapes():
    d = _run("--probe", "mfma")
    shapes = [p["instruction"] for p in d["points"]]
    assert shapes == ["v_mfma_f32_32x32x16_f16", "v_mfma_f32_16x16x32_f16"]
    for p in d["points"]:
        assert 500.0 < p["TFLOPs_sustained"] < 2500.0
