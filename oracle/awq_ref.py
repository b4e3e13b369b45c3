"""CPU oracle for the AWQ W4A16 linear path.  TEST INFRASTRUCTURE, NOT PRODUCT.

Only the test-suite, the smoke check and the benchmark's CPU-baseline leg may import this
module; the shipped package never does.

What it restates.  The harness under /root/reference starts `vllm/vllm-openai:latest`
(utils/generate_compose.py:67, server command :85-93) on AWQ checkpoints
(config.yaml:36, :47, :51, :134; README.md:55, :64).  The arithmetic of that path lives in
the third-party vLLM package inside the docker image (tag `:latest`, no pinned version, not
vendored), so there is no reference source line to follow.  The normative definition is the
AutoAWQ "GEMM" checkpoint layout and the dequantize-then-matmul statement of the path:

    qweight int32 [K, N/8]   nibble i of word c holds logical column 8c + P[i],
                             P = [0, 2, 4, 6, 1, 3, 5, 7]
    qzeros  int32 [K/G, N/8] same nibble order
    scales  fp16  [K/G, N]
    W[k, n] = fp16_rn( float(w[k, n] - z[k // G, n]) * float(s[k // G, n]) )
    Y       = fp16_rn( X.float() @ W.float() )

Parity status per function (what pins it, independent of this file's own formulas):
  pack_awq / unpack_awq   hand-derived known answers, R∘P = id, round trips      PINNED
  dequantize              exact-rational brute force over every (w, z, s) triple,
                          agreement with the scalar C restatement                PINNED
  gemm                    library fp64 matmul on pinned W, one-hot / w==z cases  PINNED
  moe_align               permutation / padding invariants                       PINNED
  topk_softmax            torch.softmax + torch.topk                             PINNED
  topk_sigmoid            torch.sigmoid + torch.topk of score + bias             PINNED
  moe_forward             per-token brute force from pinned W                    PINNED
  cpu_dequantize_torch / cpu_linear_torch / cpu_moe_torch (the timed CPU baseline)
                          same bits as dequantize; gemm / moe_forward to fp32
                          summation order                                        PINNED
  behavioural choices only an import of vLLM could pin (M threshold between fused GEMM
  and dequant+matmul, sentinel/padding layout of its align kernel, [gate | up] order
  inside w13, where its grouped top-k applies the scaling factor)     PARITY UNPINNED
"""
from __future__ import annotations

import numpy as np

AWQ_PACK_ORDER = (0, 2, 4, 6, 1, 3, 5, 7)      # nibble i  -> logical column P[i]
AWQ_UNPACK_ORDER = (0, 4, 1, 5, 2, 6, 3, 7)    # logical j -> nibble R[j]


def pack_awq(vals: np.ndarray) -> np.ndarray:
    """[R, C] integers in 0..15 -> int32 [R, C/8] in AWQ nibble order."""
    vals = np.asarray(vals)
    assert vals.ndim >= 1 and vals.shape[-1] % 8 == 0
    v = vals.astype(np.uint32).reshape(*vals.shape[:-1], vals.shape[-1] // 8, 8)
    assert int(v.max(initial=0)) <= 15
    word = np.zeros(v.shape[:-1], dtype=np.uint32)
    for i, col in enumerate(AWQ_PACK_ORDER):
        word |= v[..., col] << np.uint32(4 * i)
    return word.view(np.int32)


def unpack_awq(words: np.ndarray) -> np.ndarray:
    """int32 [R, C/8] -> uint8 [R, C] logical values (logical shift: sign bit is data)."""
    w = np.ascontiguousarray(words).view(np.uint32)
    out = np.empty(w.shape + (8,), dtype=np.uint8)
    for j, nib in enumerate(AWQ_UNPACK_ORDER):
        out[..., j] = (w >> np.uint32(4 * nib)) & np.uint32(0xF)
    return out.reshape(*w.shape[:-1], w.shape[-1] * 8)


def dequantize(qweight: np.ndarray, scales: np.ndarray, qzeros: np.ndarray,
               group: int) -> np.ndarray:
    """fp16 [K, N] = fp16_rn(float(w - z) * float(s)); one rounding."""
    K = qweight.shape[-2]
    if group <= 0:
        group = K
    w = unpack_awq(qweight).astype(np.int32)
    z = np.repeat(unpack_awq(qzeros).astype(np.int32), group, axis=-2)
    s = np.repeat(np.asarray(scales, dtype=np.float16).astype(np.float32), group, axis=-2)
    return ((w - z).astype(np.float32) * s).astype(np.float16)


def gemm(x: np.ndarray, qweight, scales, qzeros, group: int, acc=np.float32) -> np.ndarray:
    """fp16 [M, N]: dequantize then matmul with `acc` accumulation, rounded once to fp16."""
    W = dequantize(qweight, scales, qzeros, group)
    return (np.asarray(x, np.float16).astype(acc) @ W.astype(acc)).astype(np.float16)


def gemm_wide(x, qweight, scales, qzeros, group: int) -> np.ndarray:
    """float64 [M, N] product of the fp16 inputs and pinned fp16 W, no final rounding."""
    W = dequantize(qweight, scales, qzeros, group)
    return np.asarray(x, np.float16).astype(np.float64) @ W.astype(np.float64)


def rel_frobenius(y, y_ref) -> float:
    y = np.asarray(y, np.float64)
    r = np.asarray(y_ref, np.float64)
    den = np.linalg.norm(r)
    return float(np.linalg.norm(y - r) / den) if den > 0 else float(np.linalg.norm(y - r))


# --------------------------------------------------------------------------- MoE

def topk_softmax(logits: np.ndarray, topk: int, renormalize: bool = True):
    """softmax over experts, top-k (ties: lowest expert id first), optional renormalise."""
    lg = np.asarray(logits, np.float32).astype(np.float64)
    p = np.exp(lg - lg.max(axis=-1, keepdims=True))
    p /= p.sum(axis=-1, keepdims=True)
    order = np.argsort(-lg, axis=-1, kind="stable")[:, :topk]   # softmax is monotonic
    w = np.take_along_axis(p, order, axis=-1)
    if renormalize:
        w = w / w.sum(axis=-1, keepdims=True)
    return order.astype(np.int32), w.astype(np.float32)


def topk_sigmoid(logits: np.ndarray, topk: int, renormalize: bool = True, bias=None, scale: float = 1.0):
    """score = sigmoid(logit); experts chosen by score + bias (ties: lowest id), weighted by the
    score, optionally renormalised over the chosen ones, times scale.  (The routing of
    sigmoid-scored MoE checkpoints with a score-correction bias and one expert group.)"""
    lg = np.asarray(logits, np.float32).astype(np.float64)
    score = 1.0 / (1.0 + np.exp(-lg))
    # the device adds the bias in fp32 to an fp32 score: choose on the same values
    key = score.astype(np.float32)
    if bias is not None:
        key = key + np.asarray(bias, np.float32)[None, :]
    order = np.argsort(-key.astype(np.float64), axis=-1, kind="stable")[:, :topk]
    w = np.take_along_axis(score, order, axis=-1)
    if renormalize:
        w = w / w.sum(axis=-1, keepdims=True)
    return order.astype(np.int32), (w * scale).astype(np.float32)


def moe_align(topk_ids: np.ndarray, num_experts: int, tile_m: int):
    """Stable sort of flat (token, slot) indices by expert, each expert's run padded to a
    multiple of tile_m with the sentinel T*topk.  Returns (sorted_ids, expert_ids,
    num_tokens_post_padded)."""
    flat = np.asarray(topk_ids, np.int64).reshape(-1)
    n = flat.size
    sorted_ids, expert_ids = [], []
    for e in range(num_experts):
        idx = np.nonzero(flat == e)[0]
        if idx.size == 0:
            continue
        nblk = -(-idx.size // tile_m)
        run = np.full(nblk * tile_m, n, dtype=np.int64)
        run[:idx.size] = idx
        sorted_ids.append(run)
        expert_ids.extend([e] * nblk)
    if sorted_ids:
        s = np.concatenate(sorted_ids)
    else:
        s = np.zeros(0, np.int64)
    return s.astype(np.int32), np.asarray(expert_ids, np.int32), int(s.size)


def silu(v):
    return v / (1.0 + np.exp(-v))


def moe_forward(x, w13, w2, topk_ids, topk_w, group: int) -> np.ndarray:
    """Per-token brute force.  w13 / w2 are (qweight[E,K,N/8], scales[E,K/G,N],
    qzeros[E,K/G,N/8]); w13 columns are [gate | up].  Intermediates are rounded to fp16
    where the device path stores fp16 (after GEMM 1, after SiLU*up, after GEMM 2), the
    slot sum is fp32.  Returns fp16 [T, H]."""
    x = np.asarray(x, np.float16)
    T = x.shape[0]
    E = w13[0].shape[0]
    W13 = [None] * E
    W2 = [None] * E
    I = w2[0].shape[1]
    H = w2[0].shape[2] * 8
    out = np.zeros((T, H), np.float32)
    for t in range(T):
        xt = x[t].astype(np.float32)
        for slot in range(topk_ids.shape[1]):
            e = int(topk_ids[t, slot])
            if W13[e] is None:
                W13[e] = dequantize(w13[0][e], w13[1][e], w13[2][e], group).astype(np.float32)
                W2[e] = dequantize(w2[0][e], w2[1][e], w2[2][e], group).astype(np.float32)
            h = (xt @ W13[e]).astype(np.float16).astype(np.float32)
            a = (silu(h[:I]) * h[I:]).astype(np.float16).astype(np.float32)
            o = (a @ W2[e]) * np.float32(topk_w[t, slot])
            out[t] += o.astype(np.float16).astype(np.float32)
    return out.astype(np.float16)


# --------------------------------------------------------------------------- baseline

def cpu_dequantize_torch(qweight_t, scales_t, qzeros_t, group: int):
    """PyTorch dequantize on the host: fp16 [K, N] = fp16((w - z) * s).  Torch CPU tensors."""
    import torch

    K = qweight_t.shape[0]
    if group <= 0:
        group = K
    shifts = torch.tensor([4 * r for r in AWQ_UNPACK_ORDER], dtype=torch.int32)

    def unpack(t):
        return ((t.unsqueeze(-1) >> shifts) & 0xF).reshape(t.shape[0], -1)

    w = unpack(qweight_t)
    z = unpack(qzeros_t).repeat_interleave(group, dim=0)
    s = scales_t.float().repeat_interleave(group, dim=0)
    return ((w - z).float() * s).half()


def cpu_matmul_torch(x_t, W_t):
    """fp16 [M, N] = fp16(X.float() @ W.float()) on the host."""
    return (x_t.float() @ W_t.float()).half()


def cpu_linear_torch(x_t, qweight_t, scales_t, qzeros_t, group: int):
    """The reference CPU path (M=16, K=N=4096 is its CPU-runnable case): PyTorch dequantize
    then matmul on the host.  Takes and returns torch CPU tensors.  Pinned against dequantize /
    gemm above (same bits for W; the product differs from numpy's only in fp32 summation
    order)."""
    return cpu_matmul_torch(x_t, cpu_dequantize_torch(qweight_t, scales_t, qzeros_t, group))


def cpu_moe_torch(x_t, w13_t, w2_t, topk_ids_t, topk_w_t, group: int):
    """The MoE block on the host with PyTorch: every expert that is hit is dequantised once and
    applied to its tokens (fp16 intermediates where the device path stores fp16, fp32 slot sum).
    Torch CPU tensors; w13 / w2 are (qweight [E, K, N/8], scales, qzeros) triples."""
    import torch

    T, H = x_t.shape
    inter = w2_t[0].shape[1]
    out = torch.zeros((T, H), dtype=torch.float32)
    for e in torch.unique(topk_ids_t).tolist():
        tok, slot = torch.nonzero(topk_ids_t == e, as_tuple=True)
        W13 = cpu_dequantize_torch(w13_t[0][e], w13_t[1][e], w13_t[2][e], group)
        W2 = cpu_dequantize_torch(w2_t[0][e], w2_t[1][e], w2_t[2][e], group)
        h = cpu_matmul_torch(x_t[tok], W13).float()
        a = (torch.nn.functional.silu(h[:, :inter]) * h[:, inter:]).half()
        o = ((a.float() @ W2.float()) * topk_w_t[tok, slot][:, None]).half().float()
        out.index_add_(0, tok, o)
    return out.half()
