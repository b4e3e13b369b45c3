"""Result block: the reader against blocks recorded by the harness (tests/golden/results/*.txt
are the "Serving Benchmark Result" blocks of three of its result files, values below read off
them by eye), and writer -> reader round trip."""
import pathlib
from importlib import import_module

import pytest

GOLD = pathlib.Path(__file__).parent / "golden" / "results"

RECORDED = {
    "pro6000_x_1_QuantTrio_Qwen3-Coder-30B-A3B-Instruct-AWQ":
        (8424.65, dict(request_throughput=4.22, output_throughput=4218.26, mean_ttft_ms=5903.25, mean_tpot_ms=86.95)),
    "l40s_x_2_ibnzterrell_Meta-Llama-3.3-70B-Instruct-AWQ-INT4":
        (495.11, dict(request_throughput=0.25, output_throughput=247.90, mean_ttft_ms=513735.38, mean_tpot_ms=88.11)),
    "rtx5090_x_4_QuantTrio_Qwen3-Coder-30B-A3B-Instruct-AWQ":
        (12743.99, dict(request_throughput=6.38, output_throughput=6380.98, mean_ttft_ms=12972.56, mean_tpot_ms=44.64)),
}


@pytest.fixture(scope="module")
def report(sba):
    return import_module(sba.__name__ + ".report")


@pytest.mark.parametrize("name", sorted(RECORDED))
def test_reader_on_recorded_blocks(report, name):
    total, metrics = report.parse_serving_result((GOLD / f"{name}.txt").read_text())
    want_total, want = RECORDED[name]
    assert total == want_total
    assert metrics == want


REFERENCE_RESULTS = pathlib.Path("/root/reference/results")


@pytest.mark.skipif(not REFERENCE_RESULTS.is_dir(), reason="the harness's recorded results are not on this machine")
def test_reader_on_every_recorded_result_file(report):
    """Every benchmark log the harness recorded: what the reader returns must agree with the
    block's own totals (tokens and requests over the duration, read here line by line, not
    through the reader's patterns) and with the latency lines."""
    files = sorted(REFERENCE_RESULTS.glob("*/*_vllm_benchmark.txt"))
    assert len(files) >= 20
    checked = 0
    for f in files:
        text = f.read_text(errors="replace")
        if "Serving Benchmark Result" not in text:
            continue          # a run that failed before the result block
        field = {}
        for line in text.splitlines():
            if ":" in line:
                k, _, v = line.rpartition(":")
                try:
                    field[k.strip()] = float(v)
                except ValueError:
                    pass
        total, m = report.parse_serving_result(text)
        dur = field["Benchmark duration (s)"]
        assert total == field["Total Token throughput (tok/s)"], f.name
        assert total == pytest.approx((field["Total input tokens"] + field["Total generated tokens"]) / dur, rel=2e-3), f.name
        assert m["output_throughput"] == pytest.approx(field["Total generated tokens"] / dur, rel=2e-3), f.name
        assert m["request_throughput"] == pytest.approx(field["Successful requests"] / dur, abs=0.006), f.name
        assert m["mean_ttft_ms"] == field["Mean TTFT (ms)"] and m["mean_tpot_ms"] == field["Mean TPOT (ms)"], f.name
        checked += 1
    assert checked >= 20


def test_reader_without_total(report):
    assert report.parse_serving_result("Request throughput (req/s):   4.2\n") == (None, {})
    total, metrics = report.parse_serving_result("Total Token throughput (tok/s):   10.5\n")
    assert total == 10.5 and metrics == {}


def test_writer_reader_round_trip(report):
    res = dict(batch=64, prompt_len=1024, new_tokens=256, prefill_s=1.5, decode_s=3.5, ms_per_decode_step=13.73)
    block = report.format_serving_result(res)
    lines = block.splitlines()
    assert lines[0].strip("=").strip() == "Serving Benchmark Result" and set(lines[-1]) == {"="}
    total, m = report.parse_serving_result(block)
    assert total == pytest.approx(64 * 1280 / 5.0, abs=0.01)
    assert m["output_throughput"] == pytest.approx(64 * 256 / 5.0, abs=0.01)
    assert m["request_throughput"] == pytest.approx(12.8, abs=0.01)
    assert m["mean_ttft_ms"] == 1500.0 and m["mean_tpot_ms"] == 13.73
