"""Layer shapes of the other AWQ checkpoints in the harness's model list (Llama-3.3-70B,
GLM-4.5-Air, Qwen3-Coder-480B-A35B): linears against dequantize + library matmul, MoE blocks
against the dense expert evaluation, with each model's routing."""
import pytest
import torch

pytestmark = pytest.mark.gpu
TOL = 2e-3


def _triple(K, N, gpu, g, lead=()):
    qw = torch.randint(-2 ** 31, 2 ** 31, (*lead, K, N // 8), dtype=torch.int32, device=gpu, generator=g)
    qz = torch.randint(-2 ** 31, 2 ** 31, (*lead, K // 128, N // 8), dtype=torch.int32, device=gpu, generator=g)
    sc = (torch.rand((*lead, K // 128, N), device=gpu, generator=g) * 0.019 + 0.001).half()
    return qw, sc, qz


def _rel(a, b):
    a, b = a.float(), b.float()
    return float((a - b).norm() / b.norm())


@pytest.mark.parametrize("name,K,N", [
    ("llama70b gate_up", 8192, 57344), ("llama70b down", 28672, 8192),
    ("glm45air qkv", 4096, 14336), ("glm45air shared gate_up", 4096, 2816), ("glm45air shared down", 1408, 4096),
    ("qwen3-480b qkv", 6144, 14336), ("qwen3-480b o", 12288, 6144),
])
def test_model_linears(sba, gpu, name, K, N):
    g = torch.Generator(device=gpu).manual_seed(K + N)
    qw, sc, qz = _triple(K, N, gpu, g)
    W = sba.awq_dequantize(qw, sc, qz).float()
    for M in (1, 16, 40, 200):
        x = torch.randn((M, K), device=gpu, generator=g).half()
        err = _rel(sba.awq_gemm(x, qw, sc, qz, 0), x.float() @ W)
        assert err <= TOL, f"{name} M={M}: {err:.2e}"


@pytest.mark.parametrize("name,H,E,topk,I,routing", [
    ("glm45air", 4096, 128, 8, 1408, dict(scoring_func="sigmoid", bias=True, routed_scaling_factor=1.0)),
    ("qwen3-480b", 6144, 160, 8, 2560, dict(scoring_func="softmax", bias=False, routed_scaling_factor=1.0)),
])
@pytest.mark.parametrize("T", [3, 64])
def test_model_moe_blocks(sba, gpu, name, H, E, topk, I, routing, T):
    g = torch.Generator(device=gpu).manual_seed(H + E + T)
    w13, w2 = _triple(H, 2 * I, gpu, g, (E,)), _triple(I, H, gpu, g, (E,))
    x = torch.randn((T, H), device=gpu, generator=g).half()
    logits = torch.randn((T, E), device=gpu, generator=g)
    bias = (torch.randn((E,), device=gpu, generator=g) * 0.1) if routing["bias"] else None
    kw = dict(scoring_func=routing["scoring_func"], e_score_correction_bias=bias,
              routed_scaling_factor=routing["routed_scaling_factor"])
    y = sba.fused_moe_awq(x, w13, w2, logits, topk, True, **kw)
    w, ids = sba.topk_route(logits, topk, True, **kw)
    ref = torch.zeros((T, H), dtype=torch.float32, device=gpu)
    for e in torch.unique(ids).tolist():
        tok, slot = torch.nonzero(ids == e, as_tuple=True)
        W13 = sba.awq_dequantize(w13[0][e], w13[1][e], w13[2][e]).float()
        W2 = sba.awq_dequantize(w2[0][e], w2[1][e], w2[2][e]).float()
        h = (x[tok].float() @ W13).half().float()
        a = (torch.nn.functional.silu(h[:, :I]) * h[:, I:]).half().float()
        ref.index_add_(0, tok, ((a @ W2) * w[tok, slot][:, None]).half().float())
    err = _rel(y, ref)
    print(f"[{name} moe T={T}] rel_fro={err:.2e}", flush=True)
    assert err <= TOL
