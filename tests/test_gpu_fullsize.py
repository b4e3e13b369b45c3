"""Benchmark-size checks (Qwen2.5-72B layer shapes and the Qwen3-30B-A3B attention linears),
where the CPU oracle would take minutes: the dequantize kernel against the oracle on sampled
rows of the full-size matrices, then the GEMM kernels against that dequantize kernel followed by
a library matmul, plus properties that need no reference (rows independent of M, split-K
invariance)."""
import numpy as np
import pytest
import torch

from oracle import awq_ref

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


@pytest.mark.parametrize("name,K,N", LAYERS)
def test_full_size_dequantize_rows_against_the_oracle(sba, gpu, name, K, N):
    """The full-size tests below use the dequantize kernel as their reference, so the kernel itself
    is anchored here at those sizes: whole rows of its output (first and last rows of the matrix,
    both sides of group boundaries near the start, the middle and the end, the grid's last row
    slab, and a random sample) must equal the oracle's bits.  Whole rows cover every word column,
    the ragged last column block included."""
    qw, sc, qz, _ = _weights(K, N, gpu, 1)
    W = sba.awq_dequantize(qw, sc, qz)
    G, ngroups = 128, K // 128
    rows = {0, 1, 15, 16, 127, 128, 129, K - 129, K - 128, K - 17, K - 16, K - 1}
    for gidx in (ngroups // 2, ngroups - 2):
        rows |= {gidx * G - 1, gidx * G, gidx * G + 127}
    rows |= set(np.random.default_rng(K + N).integers(0, K, 48).tolist())
    rows = sorted(rows)
    ridx = torch.tensor(rows, device=gpu)
    gidx = ridx // G
    # each sampled row as a group of its own for the oracle: its packed words, its group's scales / zeros
    want = awq_ref.dequantize(qw[ridx].cpu().numpy(), sc[gidx].cpu().numpy(), qz[gidx].cpu().numpy(), 1)
    got = W[ridx].cpu().numpy()
    assert got.shape == want.shape == (len(rows), N)
    bad = np.argwhere(got.view(np.uint16) != want.view(np.uint16))
    assert bad.size == 0, f"{name}: first mismatches (sample row, column) {bad[:5].tolist()} of rows {rows}"


def _one_hot_rows(K, gpu, seed, n):
    """n row indices of K: first / last rows, first / last 128-row chunk, both sides of group
    boundaries, the tail-step rows of a 231-chunk layer, and a random sample."""
    rows = [0, 1, 31, 32, 127, 128, K - 129, K - 128, K - 97, K - 33, K - 32, K - 1]
    rows += np.random.default_rng(seed).integers(0, K, n - len(rows)).tolist()
    return sorted(set(int(r) for r in rows))


@pytest.mark.parametrize("name,K,N", LAYERS)
def test_full_size_gemm_one_hot_rows_against_the_oracle(sba, gpu, name, K, N):
    """A second anchor of the full-size GEMM checks that does not pass through the dequantize
    kernel: with a one-hot activation row e_k the skinny kernel returns row k of the dequantised
    weights exactly, so sixteen such rows per call (M = 16) must equal the oracle's dequantize of
    those rows bit for bit."""
    qw, sc, qz, _ = _weights(K, N, gpu, 6)
    rows = _one_hot_rows(K, gpu, K + N, 32)
    for r0 in range(0, len(rows), 16):
        ks = rows[r0:r0 + 16]
        x = torch.zeros((len(ks), K), dtype=torch.float16, device=gpu)
        x[torch.arange(len(ks), device=gpu), torch.tensor(ks, device=gpu)] = 1.0
        y = sba.awq_gemm(x, qw, sc, qz, 0).cpu().numpy()
        ridx = torch.tensor(ks, device=gpu)
        gidx = ridx // 128
        want = awq_ref.dequantize(qw[ridx].cpu().numpy(), sc[gidx].cpu().numpy(), qz[gidx].cpu().numpy(), 1)
        bad = np.argwhere(y.view(np.uint16) != want.view(np.uint16))
        assert bad.size == 0, f"{name}: first mismatches (row of the call, column) {bad[:5].tolist()} for k = {ks}"


@pytest.mark.parametrize("name,K,N", LAYERS)
def test_full_size_prefill_one_hot_rows_against_the_oracle(sba, gpu, name, K, N):
    """The same anchor for the many-row path (panel pass + dense kernel at 2048 rows): a one-hot
    row times exact fp16 weights is exact in the matrix pipe, so rows of a 2048-row call that are
    one-hot must equal the oracle's dequantised rows bit for bit, wherever they sit in the call
    (first / last row tile, next to random rows)."""
    qw, sc, qz, g = _weights(K, N, gpu, 7)
    M = 2048
    ks = _one_hot_rows(K, gpu, 3 * K + N, 24)
    at = np.random.default_rng(N).choice(np.arange(1, M - 1), size=len(ks), replace=False)
    at[:2] = (0, M - 1)
    x = torch.randn((M, K), device=gpu, generator=g).half()
    x[torch.tensor(at, device=gpu)] = 0
    x[torch.tensor(at, device=gpu), torch.tensor(ks, device=gpu)] = 1.0
    y = sba.awq_gemm(x, qw, sc, qz, 0)
    ridx = torch.tensor(ks, device=gpu)
    gidx = ridx // 128
    want = awq_ref.dequantize(qw[ridx].cpu().numpy(), sc[gidx].cpu().numpy(), qz[gidx].cpu().numpy(), 1)
    got = y[torch.tensor(at, device=gpu)].cpu().numpy()
    bad = np.argwhere(got.view(np.uint16) != want.view(np.uint16))
    assert bad.size == 0, f"{name}: first mismatches (sample, column) {bad[:5].tolist()}"


PREFILL_POINTS = [(n, K, N, M) for (n, K, N) in LAYERS for M in (512, 2048, 8192)]


@pytest.mark.parametrize("name,K,N,M", PREFILL_POINTS + [("qkv_proj", 8192, 10240, 100), ("down_proj", 29568, 8192, 160)])
def test_prefill_sizes_against_dequant_matmul(sba, gpu, name, K, N, M):
    """All twelve (layer, M) points of the prefill sweep and two off-grid row counts."""
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


@pytest.mark.parametrize("name,K,N", [("qwen3-30b-a3b qkv", 2048, 5120), ("qwen3-30b-a3b o", 4096, 2048)])
@pytest.mark.parametrize("M", [1, 16, 64, 8192])
def test_moe_decoder_attention_linears(sba, gpu, name, K, N, M):
    """The two dense AWQ linears of the Qwen3-30B-A3B-shaped decoder at its decode batch (64),
    its prefill pass (8 prompts x 1024 tokens) and the skinny sizes."""
    qw, sc, qz, g = _weights(K, N, gpu, 4)
    W = sba.awq_dequantize(qw, sc, qz).float()
    x = torch.randn((M, K), device=gpu, generator=g).half()
    y = sba.awq_gemm(x, qw, sc, qz, 0)
    err = _rel(y, x.float() @ W)
    print(f"[full {name} M={M}] rel_fro={err:.2e}", flush=True)
    assert err <= TOL
    assert torch.equal(y, sba.awq_gemm(x, qw, sc, qz, 0))


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


@pytest.mark.parametrize("name,K,N", [("qkv_proj", 8192, 10240), ("o_proj", 8192, 8192), ("down_proj", 29568, 8192),
                                      ("llama-70b gate_up", 8192, 57344)])
def test_full_size_layers_in_the_methods_row_pitch(sba, gpu, name, K, N):
    """Layers whose packed rows are a multiple of 1 KiB, as AWQLinearMethod holds them after
    loading (rows one 128-byte line further apart): decode, 32-row and prefill launches and
    awq_dequantize give the bits of the contiguous tensor."""
    import importlib
    ops = importlib.import_module(sba.__name__ + ".ops")
    qw, sc, qz, g = _weights(K, N, gpu, 5)
    qwp = ops.pad_qweight_rows(qw)
    assert qwp.stride() == (N // 8 + 32, 1) and tuple(qwp.shape) == tuple(qw.shape)
    for M in (1, 16, 32, 300):
        x = torch.randn((M, K), device=gpu, generator=g).half()
        y0 = sba.awq_gemm(x, qw, sc, qz, 0)
        y1 = sba.awq_gemm(x, qwp, sc, qz, 0)
        assert torch.equal(y0.view(torch.int16), y1.view(torch.int16)), (name, M)
    assert torch.equal(sba.awq_dequantize(qw, sc, qz).view(torch.int16), sba.awq_dequantize(qwp, sc, qz).view(torch.int16))
