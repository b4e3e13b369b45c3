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
