"""Benchmark-size checks (Qwen2.5-72B layer shapes), where the CPU oracle would take minutes:
the GEMM kernels against the bit-exact dequantize kernel followed by a library matmul, plus
properties that need no reference (rows independent of M, split-K invariance)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

TOL = 2e-3
LAYERS = [("qkv_proj", 8192, 10240), ("o_proj", 8192, 8192), ("gate_up_proj", 8192, 59136),
          ("down_proj", 29568, 8192)]


def _weights(K, N, gpu, seed):
    g = torch.Generator(device=gpu).manual_seed(seed)
    qw = torch.randint(-2 ** 31, 2 ** 31, (K, N // 8), dtype=torch.int32, device=gpu, generator=g)
    qz = torch.randint(-2 ** 31, 2 ** 31, (K // 128, N // 8), dtype=torch.int32, device=gpu, generator=g)
    sc = (torch.rand((K // 128, N), device=gpu, generator=g) * 0.019 + 0.001).half()
    return qw, sc, qz, g


def _rel(a, b):
    a, b = a.float(), b.float()
    return float((a - b).norm() / b.norm())


@pytest.mark.parametrize("name,K,N", LAYERS)
def test_decode_sizes_against_dequant_matmul(sba, gpu, name, K, N):
    qw, sc, qz, g = _weights(K, N, gpu, 1)
    W = sba.awq_dequantize(qw, sc, qz).float()
    x16 = torch.randn((16, K), device=gpu, generator=g).half()
    ref = x16.float() @ W
    y16 = sba.awq_gemm(x16, qw, sc, qz, 0)
    err = _rel(y16, ref)
    print(f"[full {name} M=16] rel_fro={err:.2e}", flush=True)
    assert err <= TOL
    # fewer rows: same rows of the result, to rounding of the split-K sum order at most
    for M in (1, 4, 8):
        yM = sba.awq_gemm(x16[:M].contiguous(), qw, sc, qz, 0)
        assert _rel(yM, ref[:M]) <= TOL
        same = bool(torch.equal(yM, y16[:M]))
        print(f"[full {name}] rows of M={M} equal rows of M=16 bit for bit: {same}", flush=True)
    # split-K invariance
    for split in (1, 3, 16):
        ys = sba.awq_gemm(x16, qw, sc, qz, force_split_k=split)
        assert _rel(ys, ref) <= TOL
        assert _rel(ys, y16) <= 2e-3


@pytest.mark.parametrize("name,K,N,M", [("qkv_proj", 8192, 10240, 512), ("o_proj", 8192, 8192, 2048),
                                        ("down_proj", 29568, 8192, 512), ("gate_up_proj", 8192, 59136, 2048),
                                        ("o_proj", 8192, 8192, 8192), ("qkv_proj", 8192, 10240, 100),
                                        ("down_proj", 29568, 8192, 160)])
def test_prefill_sizes_against_dequant_matmul(sba, gpu, name, K, N, M):
    qw, sc, qz, g = _weights(K, N, gpu, 2)
    W = sba.awq_dequantize(qw, sc, qz)
    x = torch.randn((M, K), device=gpu, generator=g).half()
    y = sba.awq_gemm(x, qw, sc, qz, 0)
    # library fp16 GEMM (fp32 accumulate) on the bit-exact dequantised weights, in slabs of rows
    worst = 0.0
    for r0 in range(0, M, 2048):
        ref = (x[r0:r0 + 2048].float() @ W.float()) if M <= 2048 else (x[r0:r0 + 2048] @ W).float()
        worst = max(worst, _rel(y[r0:r0 + 2048], ref))
    print(f"[full {name} M={M}] rel_fro={worst:.2e}", flush=True)
    assert worst <= TOL
    y2 = sba.awq_gemm(x, qw, sc, qz, 0)
    assert torch.equal(y, y2)          # deterministic


def test_activations_beyond_4gib_run_as_row_slabs(sba, gpu):
    """X larger than the 32-bit buffer range of the MFMA kernel: the call is cut into row slabs;
    checked on the rows around the cut and at both ends."""
    K, N = 29568, 256
    M = 72448 + 300                      # 72448 = largest multiple of 256 rows below 4 GiB / (2 K)
    qw, sc, qz, g = _weights(K, N, gpu, 3)
    W = sba.awq_dequantize(qw, sc, qz).float()
    x = torch.randn((M, K), device=gpu, generator=g, dtype=torch.float16)
    y = sba.awq_gemm(x, qw, sc, qz, 0)
    for r0 in (0, 72448 - 256, 72448, M - 256):
        ref = x[r0:r0 + 256].float() @ W
        err = _rel(y[r0:r0 + 256], ref)
        print(f"[slabs] rows {r0}..{r0 + 255} rel_fro={err:.2e}", flush=True)
        assert err <= TOL
