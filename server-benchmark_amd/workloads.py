"""Seeded synthetic AWQ workloads at the benchmark's layer shapes.

Value distributions follow the benchmark definition: activations fp16 N(0,1); int4 weights
and zero points uniform in 0..15, packed 8 per int32 in AWQ order; scales fp16 uniform in
[0.001, 0.02]; group 128.  Everything is drawn on the CPU generator (draw order: weights,
zeros, scales, activations) so the same seed gives the same bits on any machine, then
copied to the requested device.
"""
from __future__ import annotations

import dataclasses
import zlib

import torch

AWQ_PACK_ORDER = (0, 2, 4, 6, 1, 3, 5, 7)

# (name, K, N) of the Qwen2.5-72B AWQ linears: hidden 8192, 64 q heads / 8 kv heads of 128,
# intermediate 29568.
QWEN25_72B_LAYERS = (
    ("qkv_proj", 8192, 10240),
    ("o_proj", 8192, 8192),
    ("gate_up_proj", 8192, 59136),
    ("down_proj", 29568, 8192),
)
DECODE_M = (1, 4, 8, 16)
PREFILL_M = (512, 2048, 8192)

# Qwen3-30B-A3B MoE block
QWEN3_MOE = dict(hidden=2048, experts=128, topk=8, inter=768, group=128)
MOE_T = (1, 16, 128, 512)


def pack_int4_awq(vals: torch.Tensor) -> torch.Tensor:
    """[..., C] integers 0..15 -> int32 [..., C/8]; nibble i holds logical column P[i]."""
    assert vals.shape[-1] % 8 == 0
    v = vals.to(torch.int64).reshape(*vals.shape[:-1], vals.shape[-1] // 8, 8)
    word = torch.zeros(v.shape[:-1], dtype=torch.int64)
    for i, col in enumerate(AWQ_PACK_ORDER):
        word |= v[..., col] << (4 * i)
    word = torch.where(word >= 2 ** 31, word - 2 ** 32, word)
    return word.to(torch.int32)


def seed_for(cfg_id: int, K: int, N: int, M: int) -> int:
    return zlib.crc32(f"{cfg_id}:{K}:{N}:{M}".encode()) & 0x7FFFFFFF


@dataclasses.dataclass
class AWQLinearCase:
    x: torch.Tensor        # fp16 [M, K]
    qweight: torch.Tensor  # int32 [K, N/8]
    scales: torch.Tensor   # fp16 [K/G, N]
    qzeros: torch.Tensor   # int32 [K/G, N/8]
    group: int

    def to(self, device):
        return AWQLinearCase(self.x.to(device), self.qweight.to(device), self.scales.to(device),
                             self.qzeros.to(device), self.group)


def make_awq_weights(K: int, N: int, group: int, gen: torch.Generator, lead=()):
    G = K if group <= 0 else group
    w = torch.randint(0, 16, (*lead, K, N), generator=gen, dtype=torch.int32)
    z = torch.randint(0, 16, (*lead, K // G, N), generator=gen, dtype=torch.int32)
    s = (torch.rand((*lead, K // G, N), generator=gen) * 0.019 + 0.001).to(torch.float16)
    return pack_int4_awq(w), s, pack_int4_awq(z)


def make_linear_case(M: int, K: int, N: int, group: int = 128, seed: int = 0) -> AWQLinearCase:
    gen = torch.Generator().manual_seed(seed)
    qw, s, qz = make_awq_weights(K, N, group, gen)
    x = torch.randn((M, K), generator=gen).to(torch.float16)
    return AWQLinearCase(x, qw, s, qz, K if group <= 0 else group)


def config0() -> AWQLinearCase:
    """The CPU-runnable single linear: M=16, K=N=4096, group 128, seed 0."""
    return make_linear_case(16, 4096, 4096, 128, seed=0)


def linear_bytes(M: int, K: int, N: int, group: int = 128) -> int:
    """Algorithmic HBM bytes of one AWQ linear call: packed weights + scales + packed zeros
    + activations in + activations out."""
    G = K // group
    return K * N // 2 + G * N * 2 + G * N // 2 + 2 * M * K + 2 * M * N


def linear_flops(M: int, K: int, N: int) -> int:
    return 2 * M * K * N


@dataclasses.dataclass
class MoECase:
    x: torch.Tensor           # fp16 [T, H]
    logits: torch.Tensor      # fp32 [T, E]
    w13: tuple                # (qweight [E,H,2I/8], scales [E,H/G,2I], qzeros [E,H/G,2I/8])
    w2: tuple                 # (qweight [E,I,H/8],  scales [E,I/G,H],  qzeros [E,I/G,H/8])
    topk: int
    group: int

    def to(self, device):
        mv = lambda t: tuple(a.to(device) for a in t)
        return MoECase(self.x.to(device), self.logits.to(device), mv(self.w13), mv(self.w2),
                       self.topk, self.group)


def make_moe_case(T: int, hidden: int, experts: int, topk: int, inter: int, group: int = 128,
                  seed: int = 0) -> MoECase:
    gen = torch.Generator().manual_seed(seed)
    w13 = make_awq_weights(hidden, 2 * inter, group, gen, lead=(experts,))
    w2 = make_awq_weights(inter, hidden, group, gen, lead=(experts,))
    x = torch.randn((T, hidden), generator=gen).to(torch.float16)
    logits = torch.randn((T, experts), generator=gen)
    return MoECase(x, logits, w13, w2, topk, group)


def moe_bytes(distinct_experts: int, T: int, hidden: int, inter: int, group: int = 128) -> int:
    per_expert = (linear_bytes(0, hidden, 2 * inter, group) + linear_bytes(0, inter, hidden, group))
    return distinct_experts * per_expert + 2 * (T * hidden * 2)


def moe_flops(T: int, topk: int, hidden: int, inter: int) -> int:
    return 2 * T * topk * (hidden * 2 * inter + inter * hidden)
