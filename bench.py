#!/usr/bin/env python3
"""Benchmark of the AWQ W4A16 linear path on one MI355X.

A "step" is one pass of the decode sweep the metric is quoted on: the four Qwen2.5-72B AWQ
linears (qkv_proj, o_proj, gate_up_proj, down_proj; group 128) at M in {1, 4, 8, 16} fp16
tokens, 16 launches of awq_gemm through the C ABI.  Inputs are resident in HBM before the
timed region.  Every layer keeps four distinct weight copies and the M-th launch of a layer
uses copy M, so between two uses of the same buffer ~1.8 GB of other weights stream through
and the 256 MB Infinity Cache cannot serve them: the reported figure is HBM bandwidth.

`value` = algorithmic bytes of a step (packed weights + scales + packed zeros + activations
in + out) / time per step, timed over exactly --steps steps after exactly --warmup untimed ones.
The chip's clocks take about 20 ms of load to settle, so the same sweep timed after at least 50
untimed steps is reported beside it under "settled".  The dense layers' qweight is held as this
package's layer method holds it after loading (--rows method, the path a served model takes);
the contiguous layout's sweep is reported under "other_qweight_rows".

The prefill sweep (M in {512, 2048, 8192}, fp16 MFMA TFLOP/s) is measured after the timed region
and reported under "prefill": per point the sustained rate (at least 100 ms of back-to-back calls
timed after at least 50 ms untimed; the chip holds a lower clock under lasting matrix load) with
the burst rate of a few launches beside it.  The CPU baseline leg times the PyTorch
dequantize-then-matmul oracle on the host cores over a bounded sample.

--probe measures a ceiling instead (what HBM delivers for the decode kernel's access pattern,
what the matrix pipe sustains under the power limit, where a decode launch's time goes);
--pmc-target runs a fixed set of launches for rocprofv3 counter collection.

Prints ONE JSON line on stdout; progress goes to stderr.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X published HBM3E bandwidth
MFMA_FP16_PEAK_TFLOPS = 2500.0  # MI355X published dense fp16 MFMA rate
TRAFFIC_PROFILE = os.path.join("profiles", "awq_gemv_kernel_decode_sweep_pmc_hbm_traffic.md")


def decode_sweep_traffic(lib, layers, G):
    """HBM bytes per awq_gemv launch averaged over the decode sweep, as two rocprofv3 --pmc runs
    (FETCH_SIZE, WRITE_SIZE; counters cannot be read while timing) of `bench.py --pmc-target
    decode` measured them.  The tracked summary of those runs carries the figure together with
    the library version and the split-K factors it was measured with; it is only reported when
    both still describe the library that is running, otherwise None."""
    import re
    try:
        text = open(os.path.join(ROOT, TRAFFIC_PROFILE)).read()
    except OSError:
        return None
    m_bytes = re.search(r"^traffic_bytes_per_launch:\s*(\d+)", text, re.M)
    m_ver = re.search(r"^library_version:\s*(\d+)", text, re.M)
    m_split = re.search(r"^split_k:\s*(.+)$", text, re.M)
    if not (m_bytes and m_ver and m_split):
        return None
    if int(m_ver.group(1)) != lib.awqmi_version():
        return None
    want = dict(kv.split("=") for kv in m_split.group(1).split())
    for name, K, N in layers:
        if str(lib.awqmi_gemm_auto_split_k(16, K, N, G)) != want.get(name):
            return None
    return int(m_bytes.group(1))


CLOCK_SETTLE_STEPS = 50     # untimed steps every timed sweep is preceded by at least (20 ms)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def make_weights(K, N, G, device, gen):
    import torch
    lo, hi = -(2 ** 31), 2 ** 31
    qw = torch.randint(lo, hi, (K, N // 8), dtype=torch.int32, device=device, generator=gen)
    qz = torch.randint(lo, hi, (K // G, N // 8), dtype=torch.int32, device=device, generator=gen)
    sc = (torch.rand((K // G, N), device=device, generator=gen) * 0.019 + 0.001).to(torch.float16)
    return qw, sc, qz


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # 50 untimed steps are 20 ms: with 5 (2 ms) the timed steps still ran 4 - 5 % slower than any later
    # sweep of the same process (0.41 against 0.39 ms per step)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--launch", choices=("graph", "direct"), default="graph",
                    help="replay the step as a HIP graph (how a serving engine decodes) or launch directly")
    ap.add_argument("--split-k", type=int, default=0, help="0 = library heuristic")
    ap.add_argument("--variant", type=int, default=-1,
                    help="development: run the decode sweep through awqmi_dev_gemm_f16 with this launch-rule variant")
    ap.add_argument("--rows", choices=("contiguous", "method"), default="method",
                    help="layout of the dense layers' qweight: as this package's "
                         "AWQLinearMethod.process_weights_after_loading holds it, i.e. what the layer method's apply -- the "
                         "path a served model takes -- multiplies by (rows of N >= 8192 that are a multiple of 512 bytes "
                         "get one 128-byte line of pitch more; same values, same algorithmic bytes), or contiguous as in "
                         "the checkpoint (what the bare ops awq_gemm / awq_dequantize are handed when only they are "
                         "rebound under vLLM's own method); the other layout's sweep is timed beside it")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--decoder", action="store_true", help=argparse.SUPPRESS)   # kept for old command lines
    ap.add_argument("--no-decoder", action="store_true",
                    help="skip the 48-layer synthetic MoE decoder load (batch 64, 1024 in / 256 out)")
    ap.add_argument("--detail", action="store_true", help="per-point timings on stderr")
    ap.add_argument("--sweep-only", action="store_true",
                    help="only the timed decode sweep (no per-point, prefill, dequantize, MoE or CPU legs)")
    ap.add_argument("--pmc-target", choices=("decode", "prefill", "moe"), default=None,
                    help="counter-collection mode for rocprofv3 --pmc, no timing.  decode: the 16-launch "
                         "decode sweep twice (direct launches) plus four 256 MiB device copies "
                         "(calibration of FETCH_SIZE / WRITE_SIZE).  prefill: awq_gemm at o_proj, "
                         "M=8192, twelve times in its default form (panel pass + dense kernel) and twelve times as "
                         "the per-tile kernel.  moe: the Qwen3-30B-A3B MoE block at T=512, five times, then its w13 GEMM "
                         "alone with 16-row and with 32-row sorted-token blocks, five times each")
    ap.add_argument("--probe", choices=("hbm-stream", "mfma", "decode-timeline"), default=None,
                    help="measure a ceiling instead of the benchmark and print it as JSON.  hbm-stream: the skinny "
                         "kernel's weight access pattern with the arithmetic removed over the four 72B qweight "
                         "matrices (four rotating copies each, so every launch reads HBM), plus a plain linear read of "
                         "1 GiB.  mfma: a bare loop of fp16 MFMAs on random operands, 60 launches of about 25 ms per "
                         "instruction shape (what the matrix pipe sustains under the power limit).  decode-timeline: "
                         "per-workgroup time stamps at the phase boundaries of the skinny kernel for every layer of the "
                         "sweep at M = 1 and 16 (where a launch's time goes)")
    ap.add_argument("--pmc-data", choices=("random", "const"), default="random",
                    help="with --pmc-target prefill: random operands (the benchmark's data) or the same value in "
                         "every weight, zero point, scale and activation (no operand bit toggles in the matrix pipe)")
    args = ap.parse_args()

    if args.variant >= 0:
        args.rows = "contiguous"      # the development entry point takes contiguous rows only
    if args.gpus != 1:
        log("bench.py: this build measures one GPU only: column-parallel layers shard the weight "
            "triple on N with no exchange, row-parallel layers shard K and add one all-reduce, "
            "and the kernels take a shard's shape as it is.  Run with --gpus 1.")
        sys.exit(2)

    import torch
    sba = __import__("server_benchmark_amd")
    from server_benchmark_amd import _lib, workloads

    if not torch.cuda.is_available():
        log("bench.py: no GPU visible; the HIP path has no CPU fallback")
        sys.exit(1)
    lib = _lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    st = lib.awqmi_init()        # the library's one-time set-up, as a binding does after loading it
    if st != 0:
        log(f"bench.py: awqmi_init failed: {lib.awqmi_status_string(st).decode()}")
        sys.exit(1)
    gen = torch.Generator(device=dev).manual_seed(0)
    G = 128
    layers = workloads.QWEN25_72B_LAYERS
    Ms = workloads.DECODE_M
    NCOPY = len(Ms)

    t0 = time.time()
    W = {}
    X = {}
    Y = {}
    from server_benchmark_amd import ops

    def held(triple):
        qw, sc, qz = triple
        return (ops.pad_qweight_rows(qw) if args.rows == "method" else qw), sc, qz

    for name, K, N in layers:
        W[name] = [held(make_weights(K, N, G, dev, gen)) for _ in range(NCOPY)]
        X[name] = {M: torch.randn((M, K), device=dev, generator=gen).to(torch.float16) for M in Ms}
        Y[name] = {M: torch.empty((M, N), dtype=torch.float16, device=dev) for M in Ms}
    ws_bytes = max(lib.awqmi_gemm_workspace_bytes(M, K, N, args.split_k) for _, K, N in layers
                   for M in tuple(Ms) + tuple(workloads.PREFILL_M))
    ws = torch.zeros(ws_bytes, dtype=torch.uint8, device=dev)
    torch.cuda.synchronize()
    log(f"[bench] inputs resident after {time.time() - t0:.1f}s, "
        f"{torch.cuda.memory_allocated() / 2**30:.2f} GiB allocated")

    def launch(name, K, N, M, copy, stream_ptr, weights=None):
        qw, sc, qz = (weights or W)[name][copy]
        a = (X[name][M].data_ptr(), qw.data_ptr(), sc.data_ptr(), qz.data_ptr(), Y[name][M].data_ptr(),
             ws.data_ptr(), ws.numel(), M, K, N, G, args.split_k, stream_ptr)
        if args.variant < 0:
            st = lib.awqmi_gemm_ld_f16(a[0], a[1], qw.stride(0), *a[2:])
        else:
            st = lib.awqmi_dev_gemm_f16(*a, args.variant)
        if st != 0:
            raise RuntimeError(f"awq_gemm failed: {lib.awqmi_status_string(st).decode()}")

    def step(stream_ptr, weights=None):
        for ci, M in enumerate(Ms):
            for name, K, N in layers:
                launch(name, K, N, M, ci, stream_ptr, weights)

    step_bytes = sum(workloads.linear_bytes(M, K, N, G) for _, K, N in layers for M in Ms)
    n_launch = len(layers) * len(Ms)

    if args.probe == "hbm-stream":
        sp = torch.cuda.current_stream().cuda_stream
        res = {"probe": "hbm-stream", "peak_GBps": HBM_PEAK_GBS, "points": []}
        sink = torch.empty(1 << 20, dtype=torch.int32, device=dev)
        def flush_cache(name, r):
            # the other layers' copies between two timed launches, as in the sweep
            for oname, oK, oN in layers:
                if oname != name:
                    lib.awqmi_dev_stream_probe(W[oname][r % NCOPY][0].data_ptr(), sink.data_ptr(), 1, 0, 0, 1,
                                               oK * oN // 2 // 1024 * 1024, sp)

        for name, K, N in layers:
            parts = lib.awqmi_gemm_auto_split_k(1, K, N, G)
            nbytes = K * N // 2
            contiguous = [W[name][c][0].contiguous() for c in range(NCOPY)]
            padded = [ops.pad_qweight_rows(t) for t in contiguous]
            forms = [("skinny kernel's reads, contiguous rows", 0, contiguous, None)]
            if padded[0].stride(0) != contiguous[0].stride(0):
                forms.append(("skinny kernel's reads, rows one 128-byte line further apart", 0, padded, None))
            forms.append(("one contiguous run per wave", 1, contiguous, nbytes // 1024 * 1024))
            for label, pattern, copies, linear_bytes in forms:
                evs = []
                for r in range(40):
                    flush_cache(name, r)
                    t = copies[r % NCOPY]
                    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    a.record()
                    st = lib.awqmi_dev_stream_probe(t.data_ptr(), sink.data_ptr(), pattern, K, N, parts,
                                                    t.stride(0) if linear_bytes is None else linear_bytes, sp)
                    b.record()
                    if st != 0:
                        raise RuntimeError(lib.awqmi_status_string(st).decode())
                    evs.append((a, b))
                torch.cuda.synchronize()
                ts = sorted(a.elapsed_time(b) * 1e3 for a, b in evs[8:])
                med = ts[len(ts) // 2]
                res["points"].append({"pattern": label, "layer": name, "K": K, "N": N, "parts": parts,
                                      "workgroups": (N // 256) * parts if pattern == 0 else 256, "bytes": nbytes,
                                      "us": round(med, 2), "GBps": round(nbytes / med / 1e3, 1),
                                      "frac_hbm": round(nbytes / med / 1e3 / HBM_PEAK_GBS, 4)})
                log(f"   stream probe {name:13s} {med:8.2f} us  {nbytes / med / 1e3:8.1f} GB/s  ({label})")
            del contiguous, padded
        big = [torch.empty(1 << 30, dtype=torch.uint8, device=dev).random_(0, 255) for _ in range(2)]
        evs = []
        for r in range(20):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            st = lib.awqmi_dev_stream_probe(big[r % 2].data_ptr(), sink.data_ptr(), 1, 0, 0, 1, 1 << 30, sp)
            b.record()
            assert st == 0
            evs.append((a, b))
        torch.cuda.synchronize()
        ts = sorted(a.elapsed_time(b) * 1e3 for a, b in evs[4:])
        med = ts[len(ts) // 2]
        res["points"].append({"pattern": "one contiguous run per wave", "layer": "1 GiB buffer", "workgroups": 256,
                              "bytes": 1 << 30, "us": round(med, 2),
                              "GBps": round((1 << 30) / med / 1e3, 1), "frac_hbm": round((1 << 30) / med / 1e3 / HBM_PEAK_GBS, 4)})
        log(f"   stream probe linear 1 GiB  {med:8.2f} us  {(1 << 30) / med / 1e3:8.1f} GB/s")
        print(json.dumps(res))
        return
    if args.probe == "decode-timeline":
        sp = torch.cuda.current_stream().cuda_stream
        phases = ["workgroup starts", "main loop left", "cross-wave LDS sum done", "partial stores acknowledged",
                  "arrival counted", "last arriver: partials summed", "output stored, workgroup ends"]
        res = {"probe": "decode-timeline", "unit": "us after the first workgroup's start; min / median / max over the "
               "workgroups that reach the phase", "points": []}
        for name, K, N in layers:
            for M in (1, 16):
                split = lib.awqmi_gemm_auto_split_k(M, K, N, G)
                wgs = ((N // 8 + 31) // 32) * split
                stamps = torch.zeros(wgs * 8, dtype=torch.int64, device=dev)
                rows = None
                for r in range(12):
                    # the other layers in between, as in the sweep: every launch reads its weights from HBM
                    for oname, oK, oN in layers:
                        if oname != name:
                            launch(oname, oK, oN, 16, r % NCOPY, sp)
                    qw, sc, qz = W[name][r % NCOPY]
                    stamps.zero_()
                    st = lib.awqmi_dev_gemm_timeline_f16(X[name][M].data_ptr(), qw.data_ptr(), sc.data_ptr(), qz.data_ptr(),
                                                         Y[name][M].data_ptr(), ws.data_ptr(), ws.numel(), M, K, N, G, 0, sp,
                                                         stamps.data_ptr(), stamps.numel() * 8)
                    if st != 0:
                        raise RuntimeError(lib.awqmi_status_string(st).decode())
                    torch.cuda.synchronize()
                    t = stamps.view(wgs, 8).cpu().double() / 100.0          # 100 MHz counter -> us
                    t0 = float(t[:, 0].min())
                    cur = []
                    for k in range(7):
                        v = t[:, k][t[:, k] > 0] - t0
                        cur.append(None if v.numel() == 0 else
                                   [round(float(v.min()), 2), round(float(v.median()), 2), round(float(v.max()), 2), int(v.numel())])
                    if r >= 4:        # the first launches warm code and clocks
                        rows = cur if rows is None else [a if b is None else [round((a[i] * (r - 4) + b[i]) / (r - 3), 2) for i in range(3)] + [b[3]]
                                                         for a, b in zip(rows, cur)]
                pt = {"layer": name, "M": M, "K": K, "N": N, "split_k": split, "workgroups": wgs,
                      "phases": {phases[k]: rows[k] for k in range(7) if rows[k] is not None}}
                res["points"].append(pt)
                log(f"   timeline {name:13s} M={M:2d} split {split} ({wgs} workgroups): " +
                    "; ".join(f"{phases[k]} {rows[k][0]:.2f}/{rows[k][1]:.2f}/{rows[k][2]:.2f}" for k in range(7) if rows[k] is not None))
        print(json.dumps(res))
        return
    if args.probe == "mfma":
        sp = torch.cuda.current_stream().cuda_stream
        src = torch.randn(8 << 20, device=dev, generator=gen).to(torch.float16)      # 16 MiB of N(0, 1) fp16 values
        sink = torch.empty(65536, dtype=torch.float32, device=dev)
        res = {"probe": "mfma", "peak_TFLOPs": MFMA_FP16_PEAK_TFLOPS, "points": []}
        for shape, iname in ((0, "v_mfma_f32_32x32x16_f16"), (1, "v_mfma_f32_16x16x32_f16")):
            iters = 20000
            fl = 256 * 4 * iters * 2097152.0
            evs = [torch.cuda.Event(enable_timing=True) for _ in range(61)]
            evs[0].record()
            for i in range(60):
                st = lib.awqmi_dev_mfma_probe(src.data_ptr(), sink.data_ptr(), shape, iters, sp)
                assert st == 0
                evs[i + 1].record()
            torch.cuda.synchronize()
            tf = [fl / (evs[i].elapsed_time(evs[i + 1]) * 1e-3) / 1e12 for i in range(60)]
            settled = sorted(tf[20:])[20]
            res["points"].append({"instruction": iname, "operands": "random N(0,1) fp16 in registers, two alternating sets",
                                  "TFLOPs_first_launch": round(tf[0], 1), "TFLOPs_sustained": round(settled, 1),
                                  "frac_mfma": round(settled / MFMA_FP16_PEAK_TFLOPS, 4), "launch_ms": round(fl / settled / 1e9, 2)})
            log(f"   mfma probe {iname}: first launch {tf[0]:.0f}, sustained {settled:.0f} TFLOP/s")
        print(json.dumps(res))
        return
    if args.pmc_target == "prefill":
        name, K, N = layers[1]
        qw, sc, qz = W[name][0]
        xp = torch.randn((8192, K), device=dev, generator=gen).to(torch.float16)
        if args.pmc_data == "const":
            qw, sc, qz = torch.full_like(qw, 0x77777777), torch.full_like(sc, 0.01), torch.full_like(qz, 0x33333333)
            xp.fill_(1.0)
        yp = torch.empty((8192, N), dtype=torch.float16, device=dev)
        # twelve calls of the default rule (dequantise once + dense kernel at this row count), then
        # twelve of the per-tile kernel through the development entry point, for a side-by-side record
        for variant in (-1, 1 << 25):
            for _ in range(12):
                st = lib.awqmi_dev_gemm_f16(xp.data_ptr(), qw.data_ptr(), sc.data_ptr(), qz.data_ptr(), yp.data_ptr(),
                                            ws.data_ptr(), ws.numel(), 8192, K, N, G, 0,
                                            torch.cuda.current_stream().cuda_stream, variant)
                assert st == 0
        torch.cuda.synchronize()
        log(f"[bench] pmc target: awq_gemm {name} M=8192 K={K} N={N} ({workloads.linear_flops(8192, K, N)} flops each), "
            f"{args.pmc_data} operands: 12 calls as awq_dequant_panel_kernel + awq_gemm_dense_kernel, then 12 calls as "
            f"awq_gemm_mfma_kernel")
        return
    if args.pmc_target == "moe":
        mq = workloads.QWEN3_MOE
        H, E, topk, I = mq["hidden"], mq["experts"], mq["topk"], mq["inter"]
        w13 = tuple(torch.stack(t) for t in zip(*[make_weights(H, 2 * I, G, dev, gen) for _ in range(E)]))
        w2 = tuple(torch.stack(t) for t in zip(*[make_weights(I, H, G, dev, gen) for _ in range(E)]))
        xm = torch.randn((512, H), device=dev, generator=gen).to(torch.float16)
        lg = torch.randn((512, E), device=dev, generator=gen)
        for _ in range(5):
            sba.fused_moe_awq(xm, w13, w2, lg, topk, True)
        torch.cuda.synchronize()
        # the w13 expert GEMM alone, step by step: 16-row sorted-token blocks (what the block above uses
        # at this size), then 32-row blocks with one packed word per lane -- for a side-by-side record of
        # what the wider blocks do to the L2 request count
        wts, ids = ops.topk_softmax(lg, topk, True)
        for bs in (16, 32):
            sorted_ids, expert_ids, npp = ops.moe_align_block_size(ids, bs, E)
            for _ in range(5):
                ops.moe_awq_gemm(xm, *w13, sorted_ids, expert_ids, npp, 512 * topk, topk, block_size=bs)
        torch.cuda.synchronize()
        log(f"[bench] pmc target: 5 x MoE block, T=512, {E} experts, top-{topk}, hidden {H}, inter {I}; then the w13 "
            f"GEMM alone 5 x with 16-row and 5 x with 32-row blocks")
        return
    if args.pmc_target == "decode":
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        sp = torch.cuda.current_stream().cuda_stream
        step(sp)
        step(sp)
        for _ in range(4):
            dst.copy_(src)
        torch.cuda.synchronize()
        log(f"[bench] pmc target: 2 decode sweeps = {2 * n_launch} awq_gemm launches, "
            f"{step_bytes / n_launch:.0f} algorithmic bytes per launch on average; "
            f"4 device copies of {src.numel()} bytes")
        return

    def time_sweep(weights, untimed):
        """`untimed` untimed steps, then exactly K timed ones; returns (wall seconds, event milliseconds)."""
        graph = None
        if args.launch == "graph":
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                step(side.cuda_stream, weights)          # warm the code objects outside capture
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                step(torch.cuda.current_stream().cuda_stream, weights)

        def run_step():
            if graph is not None:
                graph.replay()
            else:
                step(torch.cuda.current_stream().cuda_stream, weights)

        for _ in range(untimed):
            run_step()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t_start = time.perf_counter()
        e0.record()
        for _ in range(args.steps):
            run_step()
        e1.record()
        torch.cuda.synchronize()
        return time.perf_counter() - t_start, e0.elapsed_time(e1)

    # headline: exactly --warmup untimed steps, then --steps timed ones
    wall, ev_ms = time_sweep(None, args.warmup)
    ms_per_step = wall * 1e3 / args.steps
    value = step_bytes / (wall / args.steps) / 1e9
    kern_avg_us = ev_ms * 1e3 / (args.steps * n_launch)
    achieved = step_bytes / n_launch / (kern_avg_us * 1e-6) / 1e9
    log(f"[bench] decode sweep: {ms_per_step:.3f} ms/step wall, {ev_ms / args.steps:.3f} ms/step events, "
        f"{value:.0f} GB/s ({value / HBM_PEAK_GBS:.1%} of {HBM_PEAK_GBS:.0f})")

    # the same sweep once the clocks have settled: a handful of warm-up steps is 2 ms, and the timed
    # steps behind them still run 4 - 5 % slower than any later sweep of the same process
    settled = None
    if not args.sweep_only:
        wall_s, ev_s = time_sweep(None, max(args.warmup, CLOCK_SETTLE_STEPS))
        settled = {"value": round(step_bytes / (wall_s / args.steps) / 1e9, 1), "unit": "GB/s",
                   "ms_per_step": round(wall_s * 1e3 / args.steps, 4),
                   "untimed_steps": max(args.warmup, CLOCK_SETTLE_STEPS), "steps": args.steps,
                   "frac_hbm": round(step_bytes / (wall_s / args.steps) / 1e9 / HBM_PEAK_GBS, 4),
                   "avg_launch_us": round(ev_s * 1e3 / (args.steps * n_launch), 2)}
        log(f"[bench] decode sweep after {settled['untimed_steps']} untimed steps: {settled['ms_per_step']:.3f} ms/step, "
            f"{settled['value']:.0f} GB/s ({settled['frac_hbm']:.1%})")

    # the same sweep on the other qweight layout (only the layers whose rows the method pads differ)
    other_rows = None
    if args.variant < 0 and not args.sweep_only:
        if args.rows == "method":
            W_other = {n: [(qw.contiguous(), sc, qz) for qw, sc, qz in W[n]] for n in W}
        else:
            W_other = {n: [(ops.pad_qweight_rows(qw), sc, qz) for qw, sc, qz in W[n]] for n in W}
        wall_o, ev_o = time_sweep(W_other, max(args.warmup, CLOCK_SETTLE_STEPS))
        wall_again, _ = time_sweep(None, max(args.warmup, CLOCK_SETTLE_STEPS))   # the headline layout once more, right behind it (clock drift)
        other_rows = {"rows": ("contiguous" if args.rows == "method" else
                               "as AWQLinearMethod.process_weights_after_loading holds them (qkv / o / down rows "
                               "one 128-byte line further apart)"),
                      "value": round(step_bytes / (wall_o / args.steps) / 1e9, 1), "unit": "GB/s",
                      "ms_per_step": round(wall_o * 1e3 / args.steps, 4),
                      "frac_hbm": round(step_bytes / (wall_o / args.steps) / 1e9 / HBM_PEAK_GBS, 4),
                      "headline_layout_retimed_GBps": round(step_bytes / (wall_again / args.steps) / 1e9, 1)}
        log(f"[bench] the same sweep with the other qweight row layout ({'contiguous' if args.rows == 'method' else 'method'}): "
            f"{other_rows['ms_per_step']:.3f} ms/step, {other_rows['value']:.0f} GB/s; headline layout again: "
            f"{other_rows['headline_layout_retimed_GBps']:.0f} GB/s")
        del W_other

    if args.sweep_only:
        args.no_prefill = args.no_cpu = True
    # per-point detail (direct launches, event pair per point, same rotation)
    points = []
    stream_ptr = torch.cuda.current_stream().cuda_stream
    reps = 50          # per point: 50 timed launches (the sweep before this was the warm-up), median + p10 / p90
    for name, K, N in ([] if args.sweep_only else layers):
        for ci, M in enumerate(Ms):
            # flush the last-level cache with the other layers' copies between points
            evs = []
            for r in range(reps):
                for oname, oK, oN in layers:
                    if oname != name:
                        launch(oname, oK, oN, 16, (ci + r) % NCOPY, stream_ptr)
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                launch(name, K, N, M, (ci + r) % NCOPY, stream_ptr)
                b.record()
                evs.append((a, b))
            torch.cuda.synchronize()
            ts = sorted(a.elapsed_time(b) * 1e3 for a, b in evs)
            med = ts[len(ts) // 2]
            nbytes = workloads.linear_bytes(M, K, N, G)
            points.append({"layer": name, "M": M, "K": K, "N": N, "us": round(med, 2),
                           "us_p10": round(ts[len(ts) // 10], 2), "us_p90": round(ts[(9 * len(ts)) // 10], 2),
                           "GBps": round(nbytes / med / 1e3, 1),
                           "frac_hbm": round(nbytes / med / 1e3 / HBM_PEAK_GBS, 4),
                           "split_k": lib.awqmi_gemm_auto_split_k(M, K, N, G) if args.split_k == 0 else args.split_k})
            if args.detail:
                log(f"   {name:13s} M={M:2d}  {med:8.2f} us  {nbytes / med / 1e3:8.1f} GB/s")

    out = {
        "metric": "AWQ W4A16 GEMM HBM GB/s (decode) & TFLOP/s (prefill), 72B shapes, 1 GPU",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16 (int4 weights dequantised to f16, f32 accumulate)",
        "data": "synthetic: on-device seeded uniform int4 weights/zeros in AWQ packing, "
                "U[0.001,0.02] fp16 scales, N(0,1) fp16 activations",
        "config": {"workload": "decode GEMV sweep, Qwen2.5-72B AWQ layer shapes (qkv 8192x10240, o 8192x8192, "
                               "gate_up 8192x59136, down 29568x8192), group 128, M in {1,4,8,16}; "
                               "16 awq_gemm launches per step, 4 rotating weight copies per layer",
                   "launch": args.launch, "split_k": args.split_k, "bytes_per_step": step_bytes,
                   "qweight_rows": ("as AWQLinearMethod.process_weights_after_loading holds them: int32 [K, N/8] "
                                    "with the rows of qkv / o / down (multiples of 512 bytes, 32 lines or more) one 128-byte "
                                    "line further apart, values and shapes unchanged, pad never read"
                                    if args.rows == "method" else "contiguous, as in the checkpoint")},
        "settled": settled,
        "other_qweight_rows": other_rows,
        "peaks": {"hbm_GBps": HBM_PEAK_GBS, "hbm_source": "MI355X published HBM3E bandwidth, 8 TB/s",
                  "mfma_fp16_TFLOPs": MFMA_FP16_PEAK_TFLOPS,
                  "mfma_source": "256 CUs x 4096 fp16 flop/clk/CU (dense MFMA) x 2.4 GHz = 2516.6 TFLOP/s, "
                                 "quoted as 2.5 PFLOP/s",
                  "device": torch.cuda.get_device_name(dev),
                  "compute_units": torch.cuda.get_device_properties(dev).multi_processor_count},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": decode_sweep_traffic(lib, layers, G) if args.split_k == 0 and args.variant < 0 else None,
                     "traffic_source": TRAFFIC_PROFILE,
                     "kernel": "awq_gemv_kernel", "avg_launch_us": round(kern_avg_us, 2),
                     "bytes_per_launch": step_bytes // n_launch},
        "decode_points_note": "one event pair around one direct launch per sample (includes the launch "
                              "overhead of about 2 - 3 us that the kernel trace does not show); median of 50",
        "decode_points": points,
    }

    # ------------------------------------------------------------------ prefill sweep
    if not args.no_prefill:
        pts = []
        tot_f, tot_t, tot_tb = 0.0, 0.0, 0.0
        for name, K, N in layers:
            qw, sc, qz = W[name][0]
            for M in workloads.PREFILL_M:
                x = torch.randn((M, K), device=dev, generator=gen).to(torch.float16)
                y = torch.empty((M, N), dtype=torch.float16, device=dev)

                def call():
                    st = lib.awqmi_gemm_ld_f16(x.data_ptr(), qw.data_ptr(), qw.stride(0), sc.data_ptr(), qz.data_ptr(),
                                               y.data_ptr(), ws.data_ptr(), ws.numel(), M, K, N, G, 0, stream_ptr)
                    if st != 0:
                        raise RuntimeError(lib.awqmi_status_string(st).decode())

                def timed(n_it):
                    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    a.record()
                    for _ in range(n_it):
                        call()
                    b.record()
                    torch.cuda.synchronize()
                    return a.elapsed_time(b) / n_it

                fl = workloads.linear_flops(M, K, N)
                # burst: two warm-up launches, then 3 - 6 timed ones (a few milliseconds of load)
                call()
                call()
                torch.cuda.synchronize()
                ms_burst = timed(3 if M >= 8192 else 6)
                # sustained: at least 50 ms of the same launches untimed, then at least 100 ms timed
                n50 = max(2, int(50.0 / ms_burst) + 1)
                for _ in range(n50):
                    call()
                ms = timed(2 * n50)
                tf, tf_burst = fl / ms / 1e9, fl / ms_burst / 1e9
                tot_f += fl
                tot_t += ms
                tot_tb += ms_burst
                pts.append({"layer": name, "M": M, "ms": round(ms, 4), "TFLOPs": round(tf, 1),
                            "frac_mfma": round(tf / MFMA_FP16_PEAK_TFLOPS, 4),
                            "ms_burst": round(ms_burst, 4), "TFLOPs_burst": round(tf_burst, 1),
                            "form": {2: "fused", 3: "dequantise once + dense"}.get(lib.awqmi_dev_last_gemm_form(), "other")})
                if args.detail:
                    log(f"   prefill {name:13s} M={M:5d} {ms:9.3f} ms {tf:8.1f} TFLOP/s sustained, {tf_burst:8.1f} burst")
                del x, y
        agg, agg_burst = tot_f / tot_t / 1e9, tot_f / tot_tb / 1e9
        out["prefill"] = {"unit": "TFLOP/s", "aggregate": round(agg, 1), "peak": MFMA_FP16_PEAK_TFLOPS,
                          "frac": round(agg / MFMA_FP16_PEAK_TFLOPS, 4),
                          "aggregate_burst": round(agg_burst, 1), "frac_burst": round(agg_burst / MFMA_FP16_PEAK_TFLOPS, 4),
                          "timing": "per point: TFLOPs = at least 100 ms of back-to-back launches timed after at least "
                                    "50 ms of the same launches untimed (sustained: the chip holds a lower clock under "
                                    "this load than in its first milliseconds); TFLOPs_burst = 3 - 6 launches after two "
                                    "warm-up launches; aggregate = total flops / total time over the 12 points",
                          "kernels": "awq_gemm_mfma_kernel (fused) below 2048 rows; awq_dequant_panel_kernel + "
                                     "awq_gemm_dense_kernel from 2048 rows on these layers (the panel pass is inside the timed call)",
                          "points": pts}
        log(f"[bench] prefill sweep aggregate {agg:.1f} TFLOP/s sustained ({agg / MFMA_FP16_PEAK_TFLOPS:.1%} of fp16 MFMA "
            f"peak), {agg_burst:.1f} burst")

    # ------------------------------------------------------------------ awq_dequantize (write-bound)
    if not args.no_prefill:
        dq = []
        for name, K, N in layers:
            qw, sc, qz = W[name][0]
            o = torch.empty((K, N), dtype=torch.float16, device=dev)

            def call():
                st = lib.awqmi_dequantize_ld_f16(qw.data_ptr(), qw.stride(0), sc.data_ptr(), qz.data_ptr(), o.data_ptr(),
                                                 K, N, G, stream_ptr)
                if st != 0:
                    raise RuntimeError(lib.awqmi_status_string(st).decode())

            call()
            torch.cuda.synchronize()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(5):
                call()
            b.record()
            torch.cuda.synchronize()
            us = a.elapsed_time(b) * 1e3 / 5
            nbytes = workloads.linear_bytes(0, K, N, G) + 2 * K * N     # packed in + fp16 out
            dq.append({"layer": name, "K": K, "N": N, "us": round(us, 1), "GBps": round(nbytes / us / 1e3, 1),
                       "frac_hbm": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)})
            del o
        out["dequantize"] = {"unit": "GB/s", "kernel": "awq_dequant_kernel", "bound": "hbm (write)", "points": dq}

    # ------------------------------------------------------------------ fused MoE block (Qwen3-30B-A3B shapes)
    if not args.no_prefill:
        mq = workloads.QWEN3_MOE
        H, E, topk, I = mq["hidden"], mq["experts"], mq["topk"], mq["inter"]
        # Sixteen weight sets (the experts of sixteen layers, 5 GB), one per call of a 16-call graph:
        # between two uses of a set the other fifteen stream through, so even at T = 1 (8 experts,
        # 20 MB per call) the weights come from HBM and not from the 256 MB Infinity Cache, as they
        # do in a decoder whose every layer has experts of its own.  The cache-warm figure (one set,
        # every call on the same experts) is reported beside it.
        NSETS = 16

        def expert_set():
            lo, hi = -(2 ** 31), 2 ** 31
            def triple(K, N):
                return (torch.randint(lo, hi, (E, K, N // 8), dtype=torch.int32, device=dev, generator=gen),
                        (torch.rand((E, K // G, N), device=dev, generator=gen) * 0.019 + 0.001).to(torch.float16),
                        torch.randint(lo, hi, (E, K // G, N // 8), dtype=torch.int32, device=dev, generator=gen))
            return triple(H, 2 * I), triple(I, H)

        sets = [expert_set() for _ in range(NSETS)]
        mo = []

        def graph_us(calls, n_it=20):
            """calls: list of (x, w13, w2, logits); one graph holding them all, replayed; us per call."""
            gs = torch.cuda.Stream()
            gs.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(gs):
                ys = [sba.fused_moe_awq(x_, a_, b_, l_, topk, True).clone() for x_, a_, b_, l_ in calls]   # sizes the workspace
                torch.cuda.synchronize()
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph, stream=gs):
                    yg = [sba.fused_moe_awq(x_, a_, b_, l_, topk, True) for x_, a_, b_, l_ in calls]
                for _ in range(3):
                    graph.replay()
                torch.cuda.synchronize()
                ea, eb = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                ea.record()
                for _ in range(n_it):
                    graph.replay()
                eb.record()
                torch.cuda.synchronize()
            torch.cuda.current_stream().wait_stream(gs)
            for i, (y1, y2) in enumerate(zip(ys, yg)):
                if not torch.equal(y1, y2):
                    raise RuntimeError(f"MoE block: call {i} of the replayed graph differs from the eager call")
            return ea.elapsed_time(eb) * 1e3 / (n_it * len(calls))

        for T in workloads.MOE_T:
            xm = torch.randn((T, H), device=dev, generator=gen).to(torch.float16)
            lgs = [torch.randn((T, E), device=dev, generator=gen) for _ in range(NSETS)]
            distinct = sum(int(torch.unique(sba.topk_softmax(l_, topk, True)[1]).numel()) for l_ in lgs) / NSETS
            w13_0, w2_0 = sets[0]
            for _ in range(3):
                sba.fused_moe_awq(xm, w13_0, w2_0, lgs[0], topk, True)
            torch.cuda.synchronize()
            n_it = 20
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(n_it):
                sba.fused_moe_awq(xm, w13_0, w2_0, lgs[0], topk, True)
            b.record()
            torch.cuda.synchronize()
            us_eager = a.elapsed_time(b) * 1e3 / n_it
            # replayed from a HIP graph (how a serving engine runs decode steps; a graph holds many
            # layers, so the launch gap between two replays is not part of a block's time)
            us = graph_us([(xm, sets[i][0], sets[i][1], lgs[i]) for i in range(NSETS)])
            us_warm = graph_us([(xm, w13_0, w2_0, lgs[0])] * 8)
            nbytes = workloads.moe_bytes(1, T, H, I, G) * 0 + distinct * workloads.moe_bytes(1, 0, H, I, G) + 2 * (T * H * 2)
            fl = workloads.moe_flops(T, topk, H, I)
            mo.append({"T": T, "distinct_experts": round(distinct, 1), "us": round(us, 1),
                       "us_cache_warm": round(us_warm, 1), "us_eager_call": round(us_eager, 1),
                       "GBps": round(nbytes / us / 1e3, 1), "frac_hbm": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4),
                       "TFLOPs": round(fl / us / 1e6, 2), "frac_mfma": round(fl / us / 1e6 / MFMA_FP16_PEAK_TFLOPS, 5)})
            if args.detail:
                log(f"   moe T={T:4d} experts hit {distinct:5.1f}  {us:9.1f} us from HBM ({us_warm:6.1f} cache-warm, eager "
                    f"call {us_eager:6.1f})  {nbytes / us / 1e3:8.1f} GB/s")
        out["moe"] = {"workload": "Qwen3-30B-A3B MoE block: route + align + grouped w13 GEMM + SiLU*up + grouped w2 "
                                  "GEMM + slot sum, 128 experts, top-8, hidden 2048, inter 768; whole block per call, "
                                  "16 calls per HIP graph on 16 different expert sets and routings (weights from HBM), "
                                  "graph replayed; us_cache_warm: 8 calls per graph on one set",
                      "points": mo}
        del sets

    # ------------------------------------------------------------------ serving-shaped decoder load (opt-in)
    if not args.no_decoder and not args.sweep_only and args.pmc_target is None:
        from importlib import import_module
        # a failure in this leg fails the run: it is the only leg that drives the layer methods
        # (AWQLinearMethod / AWQMoEMethod .apply) at the serving shapes
        dec = import_module(sba.__name__ + ".decoder")
        torch.cuda.empty_cache()     # the decoder needs about 25 GB
        res = dec.run_serving_load(dec.QWEN3_30B_A3B, batch=64, prompt_len=1024, new_tokens=256, device=dev)
        res["workload"] = ("48-layer Qwen3-30B-A3B-shaped synthetic AWQ decoder, batch 64, random prompts of "
                           "1024 ids, 256 output tokens, greedy, own minimal driver (no vLLM in this image); "
                           "attention, norms, embedding and lm_head are stock PyTorch; after the timed load every "
                           "AWQ call of the first and last layer (one decode step, one prefill) is compared with "
                           "the dequantize kernel + library matmul on the same input")
        out["decoder"] = res
        log(f"[bench] decoder: prefill {res['prefill_s']} s, {res['ms_per_decode_step']} ms/decode step, "
            f"{res['output_tokens_per_s']} output tok/s; AWQ ops vs dequantize+matmul: "
            f"{res['awq_ops_rel_frobenius_max']} over {res['awq_ops_checked']} calls")
        log(import_module(sba.__name__ + ".report").format_serving_result(res))
        if not res["awq_ops_checked"] or max(res["awq_ops_rel_frobenius_max"].values()) > 2e-3:
            log("[bench] ERROR: an AWQ op of the decoder differs from dequantize + matmul beyond 2e-3")
            print(json.dumps(out))
            sys.exit(1)

    # ------------------------------------------------------------------ CPU baseline leg
    if not args.no_cpu:
        from oracle import awq_ref   # the checker: timed here as the reference CPU path
        ncores = os.cpu_count() or 1
        nthreads = min(ncores, int(os.environ.get("OMP_NUM_THREADS", ncores)))
        torch.set_num_threads(nthreads)

        def rel(a, b):
            a, b = a.float(), b.float()
            return float((a - b).norm() / b.norm())

        # bounded sample: two passes over the 16 calls of one step (about 3.7 GB of operands);
        # pass 1 times dequantize + matmul as one call (the baseline figure), pass 2 times the two
        # halves separately
        calls = [(n, K, N, M) for (n, K, N) in layers for M in Ms]
        worst = 0.0
        n0, K0, N0 = layers[1]
        awq_ref.cpu_linear_torch(X[n0][1].cpu(), *(t.cpu() for t in W[n0][0]), G)      # warm-up
        sample_bytes, t_both, t_deq, t_mm = 0, 0.0, 0.0, 0.0
        cpu_points = []
        for name, K, N, M in calls:
            qw, sc, qz = (t.cpu() for t in W[name][0])
            xc = X[name][M].cpu()
            t1 = time.perf_counter()
            yc = awq_ref.cpu_linear_torch(xc, qw, sc, qz, G)
            t2 = time.perf_counter()
            Wc = awq_ref.cpu_dequantize_torch(qw, sc, qz, G)
            t3 = time.perf_counter()
            yc2 = awq_ref.cpu_matmul_torch(xc, Wc)
            t4 = time.perf_counter()
            t_both += t2 - t1
            t_deq += t3 - t2
            t_mm += t4 - t3
            nb = workloads.linear_bytes(M, K, N, G)
            sample_bytes += nb
            cpu_points.append({"layer": name, "M": M, "cpu_ms": round((t2 - t1) * 1e3, 1),
                               "cpu_dequant_ms": round((t3 - t2) * 1e3, 1), "cpu_matmul_ms": round((t4 - t3) * 1e3, 1),
                               "cpu_GBps": round(nb / (t2 - t1) / 1e9, 3)})
            # the same call on the GPU must agree with the CPU path (checker)
            yg = sba.awq_gemm(X[name][M], *W[name][0], 0).cpu()
            worst = max(worst, rel(yg, yc), rel(yg, yc2))
            del qw, sc, qz, yc, yc2, Wc
        # the CPU-runnable configuration (M=16, K=N=4096, seed 0, drawn on the CPU generator)
        c0 = workloads.config0()
        g0 = c0.to(dev)
        for _ in range(10):
            y0 = sba.awq_gemm(g0.x, g0.qweight, g0.scales, g0.qzeros, 0)
        torch.cuda.synchronize()
        evs = []
        for _ in range(50):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            y0 = sba.awq_gemm(g0.x, g0.qweight, g0.scales, g0.qzeros, 0)
            b.record()
            evs.append((a, b))
        torch.cuda.synchronize()
        t0s = sorted(a.elapsed_time(b) * 1e3 for a, b in evs)
        cpu_ts, deq_ts, mm_ts = [], [], []
        for _ in range(7):
            t1 = time.perf_counter()
            yc0 = awq_ref.cpu_linear_torch(c0.x, c0.qweight, c0.scales, c0.qzeros, 128)
            t2 = time.perf_counter()
            Wc0 = awq_ref.cpu_dequantize_torch(c0.qweight, c0.scales, c0.qzeros, 128)
            t3 = time.perf_counter()
            awq_ref.cpu_matmul_torch(c0.x, Wc0)
            t4 = time.perf_counter()
            cpu_ts.append(t2 - t1); deq_ts.append(t3 - t2); mm_ts.append(t4 - t3)
        med = lambda ts: sorted(ts[2:])[len(ts[2:]) // 2]      # two warm-ups, five timed, median
        err0 = rel(y0.cpu(), yc0)
        out["config0"] = {"workload": "M=16, K=N=4096, group 128, seed 0 (cache-warm: 8.9 MB of weights)",
                          "gpu_us_median": round(t0s[len(t0s) // 2], 2), "gpu_us_p10": round(t0s[5], 2),
                          "gpu_us_p90": round(t0s[45], 2),
                          "cpu_ms_median": round(med(cpu_ts) * 1e3, 2),
                          "cpu_dequant_ms_median": round(med(deq_ts) * 1e3, 2),
                          "cpu_matmul_ms_median": round(med(mm_ts) * 1e3, 2), "cpu_threads": nthreads,
                          "gpu_vs_cpu_rel_frobenius": round(err0, 6)}
        worst = max(worst, err0)
        # one prefill point on the CPU path (o_proj, M = 512: 69 GFLOP; larger ones take minutes)
        xp = torch.randn((512, K0), generator=torch.Generator().manual_seed(512), dtype=torch.float32).half()
        qw, sc, qz = (t.cpu() for t in W[n0][0])
        t1 = time.perf_counter()
        Wc = awq_ref.cpu_dequantize_torch(qw, sc, qz, G)
        t2 = time.perf_counter()
        ycp = awq_ref.cpu_matmul_torch(xp, Wc)
        t3 = time.perf_counter()
        ygp = sba.awq_gemm(xp.to(dev), *W[n0][0], 0).cpu()
        errp = rel(ygp, ycp)
        worst = max(worst, errp)
        cpu_prefill = {"layer": n0, "M": 512, "cpu_ms": round((t3 - t1) * 1e3, 1),
                       "cpu_dequant_ms": round((t2 - t1) * 1e3, 1), "cpu_matmul_ms": round((t3 - t2) * 1e3, 1),
                       "cpu_TFLOPs": round(2.0 * 512 * K0 * N0 / (t3 - t1) / 1e12, 4),
                       "gpu_vs_cpu_rel_frobenius": round(errp, 6)}
        del qw, sc, qz, ycp, ygp, Wc
        # the MoE block at T = 1 and 16 on the CPU path (the experts that are hit are dequantised
        # and applied to their tokens), against the library's one-call block
        mq = workloads.QWEN3_MOE
        H, E, topk, I = mq["hidden"], mq["experts"], mq["topk"], mq["inter"]
        gm = torch.Generator(device=dev).manual_seed(3)
        w13 = tuple(torch.stack(t) for t in zip(*[make_weights(H, 2 * I, G, dev, gm) for _ in range(E)]))
        w2 = tuple(torch.stack(t) for t in zip(*[make_weights(I, H, G, dev, gm) for _ in range(E)]))
        w13c, w2c = tuple(t.cpu() for t in w13), tuple(t.cpu() for t in w2)
        cpu_moe = []
        for T in (1, 16):
            xm = torch.randn((T, H), device=dev, generator=gm).half()
            lg = torch.randn((T, E), device=dev, generator=gm)
            tw, ids = sba.topk_softmax(lg, topk, True)
            ym = sba.fused_moe_awq(xm, w13, w2, lg, topk, True).cpu()
            xc, idc, twc = xm.cpu(), ids.cpu().long(), tw.cpu()
            ts = []
            for _ in range(4):
                t1 = time.perf_counter()
                yc = awq_ref.cpu_moe_torch(xc, w13c, w2c, idc, twc, G)
                ts.append(time.perf_counter() - t1)
            tm = sorted(ts[1:])[1]
            distinct = int(torch.unique(idc).numel())
            errm = rel(ym, yc)
            worst = max(worst, errm)
            cpu_moe.append({"T": T, "distinct_experts": distinct, "cpu_ms": round(tm * 1e3, 1),
                            "cpu_GBps": round(workloads.moe_bytes(distinct, T, H, I, G) / tm / 1e9, 3),
                            "gpu_vs_cpu_rel_frobenius": round(errm, 6)})
        del w13, w2, w13c, w2c
        cpu_model = ""
        try:
            with open("/proc/cpuinfo") as f:
                for line in f:
                    if line.startswith("model name"):
                        cpu_model = line.split(":", 1)[1].strip()
                        break
        except OSError:
            pass
        out["cpu_baseline"] = {"value": round(sample_bytes / t_both / 1e9, 3), "unit": "GB/s",
                               "cores": nthreads, "kind": "port",
                               "sample": f"the 16 calls of one step, one PyTorch dequantize+matmul call each "
                                         f"({t_both:.1f} s), then dequantize and matmul of the same calls timed "
                                         f"separately ({t_deq:.1f} s + {t_mm:.1f} s)",
                               "cpu": cpu_model, "dequant_s": round(t_deq, 2), "matmul_s": round(t_mm, 2),
                               "together_s": round(t_both, 2), "points": cpu_points,
                               "prefill_point": cpu_prefill, "moe_points": cpu_moe,
                               "gpu_vs_cpu_rel_frobenius_max": round(worst, 6)}
        log(f"[bench] cpu baseline {out['cpu_baseline']['value']} GB/s on {nthreads} threads "
            f"(dequantize {t_deq:.1f} s + matmul {t_mm:.1f} s apart, {t_both:.1f} s as one call); "
            f"GPU vs CPU rel. Frobenius max {worst:.2e}")
        if worst > 2e-3:
            log("[bench] ERROR: GPU result differs from the CPU path beyond 2e-3")
            print(json.dumps(out))
            sys.exit(1)

    print(json.dumps(out))


if __name__ == "__main__":
    main()
