"""Minimal synthetic-weight MoE decoder that drives the AWQ path the way a serving engine does.

This is the stand-in for the server the harness benchmarks
(reference benchmarks/3_vllm_benchmark.sh:151-162: `vllm bench serve --dataset-name random
--ignore-eos`, fixed input / output lengths, reported as output tokens per second) when no
vLLM is installed: a Qwen3-30B-A3B-shaped decoder (RMSNorm -> AWQ qkv -> per-head q/k norm ->
RoPE -> attention over a KV cache -> AWQ o_proj -> RMSNorm -> router -> AWQ fused MoE, with
residuals; final norm and an fp16 lm_head), random weights, random prompt ids, greedy
sampling, no end-of-sequence.

Every quantised linear and the MoE block go through `AWQLinearMethod.apply` /
`AWQMoEMethod.apply`, i.e. through the library; everything else (norms, RoPE, attention,
embedding, lm_head, argmax) is stock PyTorch and is not what this repository is about.
The decode step has fixed shapes (all sequences share one length), so it is captured once in
a HIP graph and replayed: position, cache slot and attention mask are read from device
tensors that the host bumps between replays.
"""
from __future__ import annotations

import dataclasses
import math
import time

import torch
import torch.nn.functional as F

from . import awq, ops


@dataclasses.dataclass
class DecoderConfig:
    layers: int = 48
    hidden: int = 2048
    heads: int = 32
    kv_heads: int = 4
    head_dim: int = 128
    experts: int = 128
    topk: int = 8
    inter: int = 768
    vocab: int = 151936
    group: int = 128
    rope_theta: float = 1.0e6
    eps: float = 1.0e-6


QWEN3_30B_A3B = DecoderConfig()


def _rand_awq(shape_k: int, shape_n: int, group: int, dev, gen, lead=()):
    """Uniform int4 nibbles = uniform random words; scales uniform in [0.001, 0.02]."""
    qw = torch.randint(-2 ** 31, 2 ** 31, (*lead, shape_k, shape_n // 8), dtype=torch.int32, device=dev, generator=gen)
    qz = torch.randint(-2 ** 31, 2 ** 31, (*lead, shape_k // group, shape_n // 8), dtype=torch.int32, device=dev,
                       generator=gen)
    sc = (torch.rand((*lead, shape_k // group, shape_n), device=dev, generator=gen) * 0.019 + 0.001).half()
    return qw, sc, qz


class _Layer(torch.nn.Module):
    pass


def reference_linear(sub, x: torch.Tensor) -> torch.Tensor:
    """x @ W with W from the bit-exact dequantize kernel and a library fp32 matmul: the check
    that the AWQ GEMM kernels are held against at sizes the CPU oracle does not reach."""
    W = ops.awq_dequantize(sub.qweight, sub.scales, sub.qzeros).float()
    return x.float() @ W


def reference_moe(ex, h: torch.Tensor, logits: torch.Tensor, topk: int) -> torch.Tensor:
    """The MoE block expert by expert on dequantised weights (routing from the library's top-k
    kernel, which has its own exact tests); intermediates rounded to fp16 where the kernels
    store them."""
    T, H = h.shape
    inter = ex.w2_qweight.shape[1]
    w, ids = ops.topk_softmax(logits.float().contiguous(), topk, True)
    ref = torch.zeros((T, H), dtype=torch.float32, device=h.device)
    for e in torch.unique(ids).tolist():
        tok, slot = torch.nonzero(ids == e, as_tuple=True)
        W13 = ops.awq_dequantize(ex.w13_qweight[e], ex.w13_scales[e], ex.w13_qzeros[e]).float()
        W2 = ops.awq_dequantize(ex.w2_qweight[e], ex.w2_scales[e], ex.w2_qzeros[e]).float()
        g = (h[tok].float() @ W13).half().float()
        a = (F.silu(g[:, :inter]) * g[:, inter:]).half().float()
        ref.index_add_(0, tok, ((a @ W2) * w[tok, slot][:, None]).half().float())
    return ref


class AwqOpChecker:
    """Hook for SyntheticMoEDecoder.checker: compares the output of every AWQ call of the chosen
    layers with reference_linear / reference_moe on the same input and keeps the worst relative
    Frobenius error per kind.  Eager passes only (it allocates and reads results back)."""

    def __init__(self, topk: int, layers=None):
        self.topk, self.layers, self.worst, self.calls = topk, layers, {}, 0

    def __call__(self, kind, layer_index, module, inputs, y):
        if self.layers is not None and layer_index not in self.layers:
            return
        ref = reference_moe(module, inputs[0], inputs[1], self.topk) if kind == "moe" else reference_linear(module, inputs[0])
        err = float((y.float() - ref).norm() / ref.norm())
        self.worst[kind] = max(self.worst.get(kind, 0.0), err)
        self.calls += 1


class SyntheticMoEDecoder:
    """Weights + KV cache + the two passes (prefill over whole prompts, one-token decode)."""

    def __init__(self, cfg: DecoderConfig, batch: int, max_len: int, device, seed: int = 0):
        self.cfg, self.batch, self.max_len, self.dev = cfg, batch, max_len, torch.device(device)
        dev = self.dev
        gen = torch.Generator(device=dev).manual_seed(seed)
        qcfg = awq.AWQConfig(weight_bits=4, group_size=cfg.group, zero_point=True)
        self.lin = awq.AWQLinearMethod(qcfg)
        self.moe = awq.AWQMoEMethod(qcfg)
        qkv_n = (cfg.heads + 2 * cfg.kv_heads) * cfg.head_dim
        # activations are kept at unit scale: a random (w - z) * s weight has a standard
        # deviation of about 0.077, so each projection carries a fixed rescale of
        # 1 / (0.077 * sqrt(K)); without it 48 random layers overflow fp16.  The rescales are
        # folded into the residual adds (q and k are renormalised per head anyway, so the
        # qkv factor only has to reach v, i.e. the attention output)
        self.layers = []
        for _ in range(cfg.layers):
            L = _Layer()
            for name, (K, N) in (("qkv", (cfg.hidden, qkv_n)), ("o", (cfg.heads * cfg.head_dim, cfg.hidden))):
                sub = _Layer()
                self.lin.create_weights(sub, K, [N], K, N, torch.float16, device=dev)
                qw, sc, qz = _rand_awq(K, N, cfg.group, dev, gen)
                sub.qweight.data, sub.scales.data, sub.qzeros.data = qw, sc, qz
                self.lin.process_weights_after_loading(sub)
                setattr(L, name, sub)
            ex = _Layer()
            self.moe.create_weights(ex, cfg.experts, cfg.hidden, cfg.inter, torch.float16, device=dev)
            w13 = _rand_awq(cfg.hidden, 2 * cfg.inter, cfg.group, dev, gen, lead=(cfg.experts,))
            w2 = _rand_awq(cfg.inter, cfg.hidden, cfg.group, dev, gen, lead=(cfg.experts,))
            ex.w13_qweight.data, ex.w13_scales.data, ex.w13_qzeros.data = w13
            ex.w2_qweight.data, ex.w2_scales.data, ex.w2_qzeros.data = w2
            self.moe.process_weights_after_loading(ex)
            L.experts = ex
            L.router = (torch.randn((cfg.hidden, cfg.experts), device=dev, generator=gen) / math.sqrt(cfg.hidden)).half()
            L.ln1 = torch.ones(cfg.hidden, dtype=torch.float16, device=dev)
            L.ln2 = torch.ones(cfg.hidden, dtype=torch.float16, device=dev)
            L.qn = torch.ones(cfg.head_dim, dtype=torch.float16, device=dev)
            L.kn = torch.ones(cfg.head_dim, dtype=torch.float16, device=dev)
            self.layers.append(L)
        self.s_qkv = 1.0 / (0.077 * math.sqrt(cfg.hidden))
        self.s_o = 1.0 / (0.077 * math.sqrt(cfg.heads * cfg.head_dim))
        self.s_moe = 1.0 / (0.077 * 0.077 * math.sqrt(cfg.hidden) * math.sqrt(cfg.inter))
        self.embed = torch.randn((cfg.vocab, cfg.hidden), device=dev, generator=gen).half()
        self.lm_head = (torch.randn((cfg.hidden, cfg.vocab), device=dev, generator=gen) / math.sqrt(cfg.hidden)).half()
        self.norm_f = torch.ones(cfg.hidden, dtype=torch.float16, device=dev)
        # KV cache [layer][batch, kv_heads, max_len, head_dim]
        shape = (batch, cfg.kv_heads, max_len, cfg.head_dim)
        self.kc = [torch.zeros(shape, dtype=torch.float16, device=dev) for _ in range(cfg.layers)]
        self.vc = [torch.zeros(shape, dtype=torch.float16, device=dev) for _ in range(cfg.layers)]
        # RoPE tables (neox halves)
        inv = 1.0 / (cfg.rope_theta ** (torch.arange(0, cfg.head_dim, 2, device=dev, dtype=torch.float32) / cfg.head_dim))
        ang = torch.arange(max_len, device=dev, dtype=torch.float32)[:, None] * inv[None, :]
        self.cos, self.sin = ang.cos().half(), ang.sin().half()
        # decode-step state on the device (read by the captured graph)
        self.pos = torch.zeros(1, dtype=torch.int64, device=dev)
        self.tok = torch.zeros(batch, dtype=torch.int64, device=dev)
        self.next_tok = torch.zeros(batch, dtype=torch.int64, device=dev)
        self.last_logits = torch.zeros((batch, cfg.vocab), dtype=torch.float16, device=dev)
        self._graph = None
        # optional hook(kind, layer_index, module, inputs, output) called after every AWQ op of an
        # eager pass ("qkv", "o", "moe"); must stay None while a graph is captured
        self.checker = None

    # ------------------------------------------------------------------ pieces
    def _rope(self, x, cos, sin):
        # x [..., n, head_dim]; cos / sin broadcastable [..., n, head_dim / 2]
        h = x.shape[-1] // 2
        x1, x2 = x[..., :h], x[..., h:]
        return torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin), dim=-1)

    def _moe_block(self, L, h, li=-1):
        cfg = self.cfg
        logits = (h @ L.router).float()
        y = self.moe.apply(L.experts, h, logits, cfg.topk, True)
        if self.checker is not None:
            self.checker("moe", li, L.experts, (h, logits), y)
        return y

    def _o(self, L, a, li=-1):
        y = self.lin.apply(L.o, a)
        if self.checker is not None:
            self.checker("o", li, L.o, (a,), y)
        return y

    def _qkv(self, L, x, li=-1):
        cfg = self.cfg
        qkv = self.lin.apply(L.qkv, x)
        if self.checker is not None:
            self.checker("qkv", li, L.qkv, (x,), qkv)
        q, k, v = qkv.split((cfg.heads * cfg.head_dim, cfg.kv_heads * cfg.head_dim, cfg.kv_heads * cfg.head_dim), dim=-1)
        return q, k, v

    # ------------------------------------------------------------------ prefill
    @torch.no_grad()
    def prefill(self, ids: torch.Tensor, chunk_seqs: int = 8) -> torch.Tensor:
        """ids int64 [batch, L]: fills the KV cache for positions 0..L-1 and returns the greedy
        next token of every sequence.  Sequences are processed chunk_seqs at a time (8 prompts of
        1024 tokens = 8192 tokens per pass, the size at which the MoE block switches to the MFMA
        kernel's 128-row blocks; measured 1.05 / 0.93 / 0.88 s for chunks of 4 / 8 / 16 prompts)."""
        cfg = self.cfg
        B, Lp = ids.shape
        assert B == self.batch and Lp < self.max_len
        out_tok = torch.empty(B, dtype=torch.int64, device=self.dev)
        cos, sin = self.cos[:Lp][None, None], self.sin[:Lp][None, None]
        for b0 in range(0, B, chunk_seqs):
            b1 = min(B, b0 + chunk_seqs)
            nb = b1 - b0
            x = self.embed[ids[b0:b1].reshape(-1)]                       # [nb * Lp, H]
            for li, L in enumerate(self.layers):
                h = F.rms_norm(x, (cfg.hidden,), L.ln1, cfg.eps)
                q, k, v = self._qkv(L, h, li)
                q = F.rms_norm(q.reshape(nb, Lp, cfg.heads, cfg.head_dim), (cfg.head_dim,), L.qn, cfg.eps).transpose(1, 2)
                k = F.rms_norm(k.reshape(nb, Lp, cfg.kv_heads, cfg.head_dim), (cfg.head_dim,), L.kn, cfg.eps).transpose(1, 2)
                v = v.reshape(nb, Lp, cfg.kv_heads, cfg.head_dim).transpose(1, 2)
                q, k = self._rope(q, cos, sin), self._rope(k, cos, sin)
                self.kc[li][b0:b1, :, :Lp] = k
                self.vc[li][b0:b1, :, :Lp] = v
                a = F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True)
                a = a.transpose(1, 2).reshape(nb * Lp, cfg.heads * cfg.head_dim)
                x = torch.add(x, self._o(L, a.contiguous(), li), alpha=self.s_o * self.s_qkv)
                h = F.rms_norm(x, (cfg.hidden,), L.ln2, cfg.eps)
                x = torch.add(x, self._moe_block(L, h, li), alpha=self.s_moe)
            last = x.reshape(nb, Lp, cfg.hidden)[:, -1]
            logits = F.rms_norm(last, (cfg.hidden,), self.norm_f, cfg.eps) @ self.lm_head
            self.last_logits[b0:b1] = logits
            out_tok[b0:b1] = logits.argmax(dim=-1)
        self.pos.fill_(Lp)
        self.tok.copy_(out_tok)
        return out_tok

    # ------------------------------------------------------------------ decode
    @torch.no_grad()
    def _decode_step(self):
        """One token for every sequence: reads self.tok / self.pos, writes self.next_tok and
        the cache slot self.pos.  Fixed shapes throughout."""
        cfg, B = self.cfg, self.batch
        pos = self.pos
        cos = self.cos.index_select(0, pos)[None]            # [1, 1, hd/2]
        sin = self.sin.index_select(0, pos)[None]
        mask = torch.where(torch.arange(self.max_len, device=self.dev) <= pos, 0.0, float("-inf")).half()
        grp = cfg.heads // cfg.kv_heads
        scale = 1.0 / math.sqrt(cfg.head_dim)
        x = self.embed.index_select(0, self.tok)
        for li, L in enumerate(self.layers):
            h = F.rms_norm(x, (cfg.hidden,), L.ln1, cfg.eps)
            q, k, v = self._qkv(L, h, li)
            q = F.rms_norm(q.reshape(B, cfg.heads, cfg.head_dim), (cfg.head_dim,), L.qn, cfg.eps)
            k = F.rms_norm(k.reshape(B, cfg.kv_heads, cfg.head_dim), (cfg.head_dim,), L.kn, cfg.eps)
            q, k = self._rope(q, cos, sin), self._rope(k, cos, sin)
            self.kc[li].index_copy_(2, pos, k[:, :, None])
            self.vc[li].index_copy_(2, pos, v.reshape(B, cfg.kv_heads, 1, cfg.head_dim))
            qg = q.reshape(B, cfg.kv_heads, grp, cfg.head_dim)
            s = torch.matmul(qg, self.kc[li].transpose(2, 3)) * scale + mask     # [B, kv, grp, max_len]
            p = torch.softmax(s.float(), dim=-1).half()
            a = torch.matmul(p, self.vc[li]).reshape(B, cfg.heads * cfg.head_dim)
            x = torch.add(x, self._o(L, a, li), alpha=self.s_o * self.s_qkv)
            h = F.rms_norm(x, (cfg.hidden,), L.ln2, cfg.eps)
            x = torch.add(x, self._moe_block(L, h, li), alpha=self.s_moe)
        logits = F.rms_norm(x, (cfg.hidden,), self.norm_f, cfg.eps) @ self.lm_head
        self.last_logits.copy_(logits)
        self.next_tok.copy_(logits.argmax(dim=-1))

    def capture(self):
        """Capture the decode step in a HIP graph (one warm-up step runs first, on the capture
        stream, so that every workspace the step needs exists before the capture)."""
        assert self.checker is None, "the checker hook reads results back: eager passes only"
        s = torch.cuda.Stream(self.dev)
        s.wait_stream(torch.cuda.current_stream(self.dev))
        with torch.cuda.stream(s):
            self._decode_step()
            torch.cuda.synchronize(self.dev)
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=s):
                self._decode_step()
        torch.cuda.current_stream(self.dev).wait_stream(s)
        self._graph = g

    @torch.no_grad()
    def decode(self, steps: int, use_graph: bool = True) -> torch.Tensor:
        """Generates `steps` more tokens per sequence after prefill; returns int64 [batch, steps]."""
        assert int(self.pos.item()) + steps <= self.max_len
        if use_graph and self._graph is None:
            self.capture()
        out = torch.empty((self.batch, steps), dtype=torch.int64, device=self.dev)
        for i in range(steps):
            if use_graph:
                self._graph.replay()
            else:
                self._decode_step()
            out[:, i] = self.next_tok
            self.tok.copy_(self.next_tok)
            self.pos.add_(1)
        return out


def run_serving_load(cfg: DecoderConfig = QWEN3_30B_A3B, batch: int = 64, prompt_len: int = 1024,
                     new_tokens: int = 256, device="cuda:0", seed: int = 0, use_graph: bool = True,
                     verify_prefill: bool = True) -> dict:
    """The fixed-length random-prompt load: prefill `batch` prompts, then `new_tokens - 1`
    decode steps (the first output token comes out of the prefill).  Times both phases."""
    dev = torch.device(device)
    model = SyntheticMoEDecoder(cfg, batch, prompt_len + new_tokens, dev, seed)
    gen = torch.Generator(device=dev).manual_seed(seed + 1)
    ids = torch.randint(0, cfg.vocab, (batch, prompt_len), device=dev, generator=gen)
    torch.cuda.synchronize(dev)
    t0 = time.perf_counter()
    model.prefill(ids)
    torch.cuda.synchronize(dev)
    t1 = time.perf_counter()
    if use_graph:
        saved = (model.pos.clone(), model.tok.clone())
        model.capture()                      # the warm-up / capture steps overwrite one cache slot
        model.pos.copy_(saved[0]); model.tok.copy_(saved[1])
        torch.cuda.synchronize(dev)
    t2 = time.perf_counter()
    toks = model.decode(new_tokens - 1, use_graph)
    torch.cuda.synchronize(dev)
    t3 = time.perf_counter()
    out_tokens = batch * new_tokens
    # correctness of what was just timed: one more decode step (eager) and the prefill once more,
    # with every AWQ call of the first and last layer compared with the
    # dequantize-kernel + library-matmul reference on the same inputs
    chk = AwqOpChecker(cfg.topk, layers={0, cfg.layers - 1})
    model.checker = chk
    model.pos.fill_(prompt_len + new_tokens - 1)
    model._decode_step()
    if verify_prefill:
        model.prefill(ids)
    model.checker = None
    torch.cuda.synchronize(dev)
    return {
        "batch": batch, "prompt_len": prompt_len, "new_tokens": new_tokens, "layers": cfg.layers,
        "prefill_s": round(t1 - t0, 4), "decode_s": round(t3 - t2, 4),
        "ms_per_decode_step": round((t3 - t2) * 1e3 / max(1, new_tokens - 1), 3),
        "decode_tokens_per_s": round(batch * (new_tokens - 1) / (t3 - t2), 1),
        "output_tokens_per_s": round(out_tokens / ((t1 - t0) + (t3 - t2)), 1),
        "prefill_tokens_per_s": round(batch * prompt_len / (t1 - t0), 1),
        "hip_graph": bool(use_graph),
        "distinct_last_tokens": int(torch.unique(toks[:, -1]).numel()),
        "awq_ops_checked": chk.calls,
        "awq_ops_rel_frobenius_max": {k: round(v, 6) for k, v in chk.worst.items()},
    }
