"""AWQConfig / AWQLinearMethod / AWQMoEMethod: the layer-level surface a vLLM model executor
drives for an AWQ checkpoint (the servers the benchmark harness starts at reference
utils/generate_compose.py:85-93 pick this method from the checkpoint's quantization_config
because no --quantization flag is passed).  Same method names, argument meaning and registered
parameter names (`qweight`, `qzeros`, `scales`), so AWQ state dicts load unchanged; the
layers are plain torch.nn.Module objects.  vLLM is never required: the only place that looks
for it is create_weights, which wraps the parameters in vLLM's own parameter classes when those
can be imported, because vLLM's shard-aware weight loaders call methods of these classes.
"""
from __future__ import annotations

import importlib
from typing import Any, Optional

import torch
from torch.nn import Parameter

from . import ops


def _first_key(config: dict, keys, default=None, required=True):
    for k in keys:
        if k in config:
            return config[k]
    if required:
        raise ValueError(f"none of {list(keys)} found in the quantization config")
    return default


class AWQConfig:
    """weight_bits must be 4; pack_factor = 32 / weight_bits = 8; group_size -1 means one
    group spanning all of K."""

    def __init__(self, weight_bits: int, group_size: int, zero_point: bool,
                 modules_to_not_convert: Optional[list] = None):
        if weight_bits != 4:
            raise ValueError(f"AWQ here supports 4-bit weights only, got {weight_bits} bits")
        self.weight_bits = weight_bits
        self.group_size = group_size
        self.zero_point = zero_point
        self.modules_to_not_convert = list(modules_to_not_convert or [])
        self.pack_factor = 32 // weight_bits

    def __repr__(self):
        return (f"AWQConfig(weight_bits={self.weight_bits}, group_size={self.group_size}, "
                f"zero_point={self.zero_point}, modules_to_not_convert={self.modules_to_not_convert})")

    @staticmethod
    def get_name() -> str:
        return "awq"

    @staticmethod
    def get_supported_act_dtypes():
        return [torch.float16]

    @staticmethod
    def get_config_filenames():
        return ["quant_config.json", "quantize_config.json"]

    @classmethod
    def get_min_capability(cls) -> int:
        """vLLM asks every quantisation config for a minimum CUDA compute capability; on a
        ROCm build the check is a formality, so report the value vLLM's AWQ config reports."""
        return 75

    @staticmethod
    def get_scaled_act_names():
        """Activations AWQ checkpoints may carry an input scale for (same list as vLLM's)."""
        return ["gelu", "gelu_fast", "gelu_new", "gelu_pytorch_tanh"]

    @classmethod
    def from_config(cls, config: dict) -> "AWQConfig":
        bits = _first_key(config, ("w_bit", "bits"))
        group = _first_key(config, ("q_group_size", "group_size"))
        zp = _first_key(config, ("zero_point",))
        skip = _first_key(config, ("modules_to_not_convert",), default=None, required=False)
        return cls(int(bits), int(group), bool(zp), skip)

    def is_skipped(self, prefix: str) -> bool:
        return any(name in prefix for name in self.modules_to_not_convert)

    def get_quant_method(self, layer: torch.nn.Module, prefix: str = ""):
        """AWQLinearMethod for a linear layer, AWQMoEMethod for a layer flagged as fused MoE
        (`layer.is_fused_moe`), None for modules listed in modules_to_not_convert."""
        if self.is_skipped(prefix):
            return None
        if getattr(layer, "is_fused_moe", False):
            return AWQMoEMethod(self)
        return AWQLinearMethod(self)


def _register(layer, name, tensor, attrs: dict[str, Any]):
    p = Parameter(tensor, requires_grad=False)
    for k, v in attrs.items():
        setattr(p, k, v)
    layer.register_parameter(name, p)


def _vllm_parameter_classes():
    """(PackedvLLMParameter, GroupQuantScaleParameter) of vllm.model_executor.parameter, or None
    outside vLLM.  vLLM's linear layers pick their second-generation weight loader by the class
    NAME of the quantisation method, and `AWQLinearMethod` is on that list; that loader calls
    shard-loading methods (load_column_parallel_weight, load_merged_column_weight,
    load_qkv_weight, load_row_parallel_weight) that only these parameter classes have."""
    try:
        mod = importlib.import_module("vllm.model_executor.parameter")
    except ImportError:
        return None
    packed = getattr(mod, "PackedvLLMParameter", None)
    scale = getattr(mod, "GroupQuantScaleParameter", None)
    return (packed, scale) if packed is not None and scale is not None else None


class AWQLinearMethod:
    def __init__(self, quant_config: AWQConfig):
        self.quant_config = quant_config

    def create_weights(self, layer: torch.nn.Module, input_size_per_partition: int,
                       output_partition_sizes: list, input_size: int, output_size: int,
                       params_dtype: torch.dtype, **extra_weight_attrs):
        cfg = self.quant_config
        group = cfg.group_size if cfg.group_size != -1 else input_size
        if input_size_per_partition % group != 0:
            raise ValueError("The input size is not aligned with the quantized weight shape. "
                             "This can be caused by too large tensor parallel size.")
        out_pp = sum(output_partition_sizes)
        if out_pp % cfg.pack_factor != 0:
            raise ValueError("The output size is not aligned with the quantized weight shape. "
                             "This can be caused by too large tensor parallel size.")
        if params_dtype != torch.float16:
            raise ValueError("AWQ scales / activations must be float16")
        dev = extra_weight_attrs.pop("device", None)
        ngroups = input_size_per_partition // group
        qweight = torch.empty(input_size_per_partition, out_pp // cfg.pack_factor, dtype=torch.int32, device=dev)
        qzeros = torch.empty(ngroups, out_pp // cfg.pack_factor, dtype=torch.int32, device=dev)
        scales = torch.empty(ngroups, out_pp, dtype=params_dtype, device=dev)
        weight_loader = extra_weight_attrs.get("weight_loader")
        classes = _vllm_parameter_classes() if callable(weight_loader) else None
        if classes is not None:
            # inside vLLM: its parameter classes, built the way its own AWQ method builds them
            packed_cls, scale_cls = classes
            layer.register_parameter("qweight", packed_cls(
                data=qweight, input_dim=0, output_dim=1, packed_dim=1, packed_factor=cfg.pack_factor,
                weight_loader=weight_loader))
            layer.register_parameter("qzeros", packed_cls(
                data=qzeros, input_dim=0, output_dim=1, packed_dim=1, packed_factor=cfg.pack_factor,
                weight_loader=weight_loader))
            layer.register_parameter("scales", scale_cls(
                data=scales, input_dim=0, output_dim=1, weight_loader=weight_loader))
        else:
            packed = dict(input_dim=0, output_dim=1, packed_dim=1, pack_factor=cfg.pack_factor)
            _register(layer, "qweight", qweight, {**packed, **extra_weight_attrs})
            _register(layer, "qzeros", qzeros, {**packed, **extra_weight_attrs})
            _register(layer, "scales", scales, {"input_dim": 0, "output_dim": 1, **extra_weight_attrs})
        layer.input_size_per_partition = input_size_per_partition
        layer.output_size_per_partition = out_pp
        layer.output_partition_sizes = list(output_partition_sizes)

    def process_weights_after_loading(self, layer: torch.nn.Module) -> None:
        """Plain parameters in the layout the kernels stream best: qzeros and scales contiguous,
        qweight [K, N / 8] with its rows one 128-byte line further apart wherever a packed row is a
        multiple of 512 bytes and N >= 8192 (ops.pad_qweight_rows; same values, same shape, 5 - 20 %
        faster decode launches on such layers).  This is the hook in which vLLM's quantisation methods re-lay
        their weights out for their own kernels."""
        for name in ("qzeros", "scales"):
            t = getattr(layer, name)
            setattr(layer, name, Parameter(t.data.contiguous(), requires_grad=False))
        q = layer.qweight.data.contiguous()
        layer.qweight = Parameter(ops.pad_qweight_rows(q), requires_grad=False)

    def apply(self, layer: torch.nn.Module, x: torch.Tensor,
              bias: Optional[torch.Tensor] = None) -> torch.Tensor:
        qweight, scales, qzeros = layer.qweight, layer.scales, layer.qzeros
        if x.dim() == 2 and x.is_contiguous():      # the decode-step case: nothing to reshape
            out = ops.awq_gemm(x, qweight, scales, qzeros, 0)
            return out if bias is None else out.add_(bias)
        out_shape = x.shape[:-1] + (qweight.shape[-1] * self.quant_config.pack_factor,)
        x2 = x.reshape(-1, x.shape[-1])
        if not x2.is_contiguous():
            x2 = x2.contiguous()
        out = ops.awq_gemm(x2, qweight, scales, qzeros, 0)
        if bias is not None:
            out.add_(bias)
        return out.reshape(out_shape)


class AWQMoEMethod:
    """Fused-MoE counterpart: w13 ([gate | up]) and w2 expert stacks in AWQ layout."""

    def __init__(self, quant_config: AWQConfig):
        self.quant_config = quant_config

    def create_weights(self, layer: torch.nn.Module, num_experts: int, hidden_size: int,
                       intermediate_size_per_partition: int, params_dtype: torch.dtype,
                       **extra_weight_attrs):
        cfg = self.quant_config
        pf = cfg.pack_factor
        dev = extra_weight_attrs.pop("device", None)
        I = intermediate_size_per_partition

        def grp(k):
            g = cfg.group_size if cfg.group_size != -1 else k
            if k % g != 0:
                raise ValueError(f"K={k} is not a multiple of the group size {g}")
            return k // g

        shapes = {
            "w13_qweight": ((num_experts, hidden_size, 2 * I // pf), torch.int32),
            "w13_scales": ((num_experts, grp(hidden_size), 2 * I), params_dtype),
            "w13_qzeros": ((num_experts, grp(hidden_size), 2 * I // pf), torch.int32),
            "w2_qweight": ((num_experts, I, hidden_size // pf), torch.int32),
            "w2_scales": ((num_experts, grp(I), hidden_size), params_dtype),
            "w2_qzeros": ((num_experts, grp(I), hidden_size // pf), torch.int32),
        }
        # Attributes vLLM's FusedMoE.weight_loader reads off a parameter: AWQ stores a weight as
        # [K, N / 8] (input dimension first), which that loader calls "transposed" and needs to
        # know to shard gate / up along the last dimension; "group" is its name for scales and
        # zero points that come one per quantisation group.
        attrs = {"is_transposed": True, "quant_method": "group", **extra_weight_attrs}
        for name, (shape, dt) in shapes.items():
            _register(layer, name, torch.empty(shape, dtype=dt, device=dev), dict(attrs))

    def process_weights_after_loading(self, layer: torch.nn.Module) -> None:
        for name in ("w13_qweight", "w13_scales", "w13_qzeros", "w2_qweight", "w2_scales", "w2_qzeros"):
            t = getattr(layer, name)
            setattr(layer, name, Parameter(t.data.contiguous(), requires_grad=False))

    def apply(self, layer: torch.nn.Module, x: torch.Tensor, router_logits: torch.Tensor, top_k: int,
              renormalize: bool = True, use_grouped_topk: bool = False, topk_group: Optional[int] = None,
              num_expert_group: Optional[int] = None, global_num_experts: int = -1, expert_map=None,
              custom_routing_function=None, scoring_func: str = "softmax", e_score_correction_bias=None,
              activation: str = "silu", routed_scaling_factor: float = 1.0, **unused) -> torch.Tensor:
        """Same keyword surface as vLLM's fused-MoE methods.  Supported: softmax or sigmoid
        scoring, a score-correction bias (sigmoid), top-k over one expert group (optionally
        renormalised, optionally scaled), SiLU, all experts local; anything else is refused
        rather than silently computed differently."""
        if (topk_group or 1) > 1 or (num_expert_group or 1) > 1:
            raise NotImplementedError("top-k over more than one expert group is not implemented")
        if custom_routing_function is not None:
            raise NotImplementedError("custom routing functions are not implemented")
        if scoring_func not in ("softmax", "sigmoid"):
            raise NotImplementedError(f"scoring function {scoring_func!r} is not implemented")
        if e_score_correction_bias is not None and scoring_func != "sigmoid":
            raise NotImplementedError("a score-correction bias is only implemented for sigmoid scoring")
        if activation != "silu":
            raise NotImplementedError(f"activation {activation!r} is not implemented (silu only)")
        if unused.get("apply_router_weight_on_input"):
            raise NotImplementedError("routing weights applied to the expert input are not implemented")
        if expert_map is not None or (global_num_experts not in (-1, layer.w13_qweight.shape[0])):
            raise NotImplementedError("expert parallelism (expert_map / global_num_experts) is not implemented")
        shape = x.shape
        x2 = x.reshape(-1, shape[-1]).contiguous()
        out = ops.fused_moe_awq(x2, (layer.w13_qweight, layer.w13_scales, layer.w13_qzeros),
                                (layer.w2_qweight, layer.w2_scales, layer.w2_qzeros),
                                router_logits.reshape(-1, router_logits.shape[-1]), top_k, renormalize,
                                scoring_func=scoring_func,
                                e_score_correction_bias=(None if e_score_correction_bias is None
                                                         else e_score_correction_bias.float().contiguous()),
                                routed_scaling_factor=routed_scaling_factor)
        return out.reshape(shape)
