"""Serving-result block: writer and reader.

The harness keeps what `vllm bench serve` prints between the "Serving Benchmark Result"
banner and the closing rule (reference benchmarks/3_vllm_benchmark.sh:177) and later scrapes
five figures from it (reference generate_benchmark_report.py:47-87: total token throughput —
without which a result counts as missing — request throughput, output token throughput, mean
TTFT, mean TPOT).  `format_serving_result` prints the decoder driver's measurements in that
layout, so its output can be dropped into the harness's result folder; `parse_serving_result`
reads the same five figures back (from this writer's blocks and from recorded ones).
"""
from __future__ import annotations

import re
from typing import Optional

_WIDTH = 50
_FIELDS = (
    ("request_throughput", "Request throughput (req/s):"),
    ("output_throughput", "Output token throughput (tok/s):"),
    ("mean_ttft_ms", "Mean TTFT (ms):"),
    ("mean_tpot_ms", "Mean TPOT (ms):"),
)
_TOTAL = "Total Token throughput (tok/s):"


def _number_after(label: str, text: str) -> Optional[float]:
    m = re.search(re.escape(label) + r"\s+([0-9][0-9.]*)", text)
    return float(m.group(1)) if m else None


def parse_serving_result(text: str):
    """(total token throughput, {request_throughput, output_throughput, mean_ttft_ms,
    mean_tpot_ms}) — (None, {}) when the total is absent; metrics that are absent are left out."""
    total = _number_after(_TOTAL, text)
    if total is None:
        return None, {}
    metrics = {}
    for key, label in _FIELDS:
        v = _number_after(label, text)
        if v is not None:
            metrics[key] = v
    return total, metrics


def _line(label: str, value) -> str:
    v = f"{value:.2f}" if isinstance(value, float) else str(value)
    return f"{label:<41}{v:<10}"


def format_serving_result(res: dict) -> str:
    """res: the dict of decoder.run_serving_load.  One batch of `batch` requests runs in
    lock-step, so TTFT is the prefill time and TPOT the decode step time."""
    batch, n_in, n_out = res["batch"], res["prompt_len"], res["new_tokens"]
    dur = res["prefill_s"] + res["decode_s"]
    rows = [
        " Serving Benchmark Result ".center(_WIDTH, "="),
        _line("Successful requests:", batch),
        _line("Maximum request concurrency:", batch),
        _line("Benchmark duration (s):", float(dur)),
        _line("Total input tokens:", batch * n_in),
        _line("Total generated tokens:", batch * n_out),
        _line("Request throughput (req/s):", batch / dur),
        _line("Output token throughput (tok/s):", batch * n_out / dur),
        _line(_TOTAL, batch * (n_in + n_out) / dur),
        "Time to First Token".center(_WIDTH, "-"),
        _line("Mean TTFT (ms):", res["prefill_s"] * 1e3),
        "Time per Output Token (excl. 1st token)".center(_WIDTH, "-"),
        _line("Mean TPOT (ms):", float(res["ms_per_decode_step"])),
        "=" * _WIDTH,
    ]
    return "\n".join(rows) + "\n"
