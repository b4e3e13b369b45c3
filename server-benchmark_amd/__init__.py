"""MI355X-native AWQ W4A16 linear path: hand-written gfx950 kernels behind a C ABI
(libawq_mi355x.so) with the vLLM operator and layer-method surface on top."""
from . import workloads
from .awq import AWQConfig, AWQLinearMethod, AWQMoEMethod
from .ops import (awq_dequantize, awq_gemm, awq_gemm_noalloc, fused_moe_awq, moe_align_block_size, moe_awq_gemm,
                  moe_sum, silu_and_mul, topk_route, topk_softmax)

__all__ = ["AWQConfig", "AWQLinearMethod", "AWQMoEMethod", "awq_dequantize", "awq_gemm", "awq_gemm_noalloc",
           "fused_moe_awq", "moe_align_block_size", "moe_awq_gemm", "moe_sum", "silu_and_mul",
           "topk_route", "topk_softmax", "workloads"]
