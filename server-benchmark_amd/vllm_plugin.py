"""vLLM general plugin: makes the servers the harness starts (reference
utils/generate_compose.py:85-93, AWQ checkpoints of config.yaml:36,47,51,134) run their AWQ
layers on this library.

vLLM loads every entry point of the group `vllm.general_plugins` in each worker process
before the model is built.  The entry point is declared by the `.dist-info` directory at the
root of this repository (`awq_mi355x = server_benchmark_amd.vllm_plugin:register`), so putting
that root on the server's PYTHONPATH is enough (deploy.py's `library_dir` mount does that);
no wheel has to be installed.  `register()` then does two things:

1.  It rebinds the two custom ops that vLLM's own `AWQLinearMethod.apply` calls
    (`awq_dequantize`, `awq_gemm` in `vllm._custom_ops`) to this package's functions.  vLLM's
    method passes its pack factor (8) as `split_k_iters`; this package's `awq_gemm` takes that
    argument as a hint and lets the library pick the split, so the rebound op runs the tuned
    launch.  vLLM's method sends batches of 256 rows or more through `awq_dequantize` + a
    library matmul, so with the ops alone the MFMA prefill kernel is never reached and fused
    MoE layers stay on vLLM's kernels.
2.  It registers this package's `AWQConfig` as quantisation method `awq` in vLLM's registry
    (`vllm.model_executor.layers.quantization`).  The harness passes no `--quantization` flag
    (reference utils/generate_compose.py:85-93): vLLM takes the method name from the
    checkpoint's `quantization_config`, looks it up in that registry, and the registered config
    then hands out this package's `AWQLinearMethod` (every M through `awq_gemm`, prefill on the
    MFMA kernel) and `AWQMoEMethod` (the one-call MoE block) for the model's layers.

vLLM is not part of this build's image, so nothing here is exercised against a real vLLM: both
steps are tested against stand-in modules with the attribute names given above, and step 2 is
skipped with a warning (step 1 still applies) when the registry does not look as expected.
"""
from __future__ import annotations

import importlib
import warnings

_REBOUND = ("awq_dequantize", "awq_gemm")
_QUANT_PKG = "vllm.model_executor.layers.quantization"


def _optional(module: str, attr: str):
    try:
        return getattr(importlib.import_module(module), attr, None)
    except ImportError:
        return None


def make_vllm_config_class():
    """This package's AWQConfig as a subclass of vLLM's QuantizationConfig (when that base class
    can be imported), choosing the layer method by vLLM's own layer classes: FusedMoE layers get
    AWQMoEMethod, linear layers AWQLinearMethod, everything else stays unquantised (None).  A
    linear layer listed in modules_to_not_convert gets vLLM's UnquantizedLinearMethod, as vLLM's
    own AWQ config answers: vLLM's linear layers call the returned method unconditionally."""
    from .awq import AWQConfig, AWQLinearMethod, AWQMoEMethod

    base = _optional(_QUANT_PKG + ".base_config", "QuantizationConfig")
    fused_moe_cls = _optional("vllm.model_executor.layers.fused_moe", "FusedMoE")
    linear_cls = _optional("vllm.model_executor.layers.linear", "LinearBase")
    unquantized_linear = _optional("vllm.model_executor.layers.linear", "UnquantizedLinearMethod")
    bases = (AWQConfig,) if base is None else (AWQConfig, base)

    class MI355XAWQConfig(*bases):
        def __init__(self, weight_bits, group_size, zero_point, modules_to_not_convert=None):
            if base is not None:
                base.__init__(self)
            AWQConfig.__init__(self, weight_bits, group_size, zero_point, modules_to_not_convert)

        @classmethod
        def override_quantization_method(cls, hf_quant_cfg, user_quant):
            """An `awq` checkpoint stays on this method (no upgrade to another kernel family)."""
            method = str((hf_quant_cfg or {}).get("quant_method", "")).lower()
            return "awq" if method == "awq" and user_quant in (None, "awq") else None

        def get_quant_method(self, layer, prefix=""):
            if self.is_skipped(prefix):
                if linear_cls is not None and unquantized_linear is not None and isinstance(layer, linear_cls):
                    return unquantized_linear()
                return None
            if (fused_moe_cls is not None and isinstance(layer, fused_moe_cls)) or getattr(layer, "is_fused_moe", False):
                return AWQMoEMethod(self)
            if linear_cls is None or isinstance(layer, linear_cls):
                return AWQLinearMethod(self)
            return None

    return MI355XAWQConfig


def _register_quant_config() -> bool:
    """Puts the config class under the name `awq`.  vLLM keeps out-of-tree configs in
    `_CUSTOMIZED_METHOD_TO_QUANT_CONFIG` (consulted after, and therefore over, its built-in
    table) and the known names in `QUANTIZATION_METHODS`; its public decorator
    `register_quantization_config` refuses names that exist already, so for the built-in name
    `awq` the table is written directly."""
    try:
        quant = importlib.import_module(_QUANT_PKG)
    except ImportError:
        warnings.warn("server_benchmark_amd: vLLM's quantization package is missing; only the two AWQ ops were "
                      "rebound (prefill >= 256 rows and fused-MoE layers stay on vLLM's kernels)")
        return False
    cls = make_vllm_config_class()
    table = getattr(quant, "_CUSTOMIZED_METHOD_TO_QUANT_CONFIG", None)
    names = getattr(quant, "QUANTIZATION_METHODS", None)
    registered = False
    if isinstance(table, dict):
        table["awq"] = cls
        if isinstance(names, list) and "awq" not in names:
            names.append("awq")
        registered = True
    else:
        deco = getattr(quant, "register_quantization_config", None)
        if callable(deco):
            try:
                deco("awq")(cls)
                registered = True
            except ValueError:
                pass
    if registered:
        # what vLLM hands out for the name must now be this class; a registry that resolves the
        # name some other way would leave the server on its own kernels without a word
        getter = getattr(quant, "get_quantization_config", None)
        if callable(getter):
            try:
                got = getter("awq")
            except Exception as e:           # noqa: BLE001 - any failure of the lookup is reported, not raised
                got = e
            if got is not cls:
                warnings.warn(f"server_benchmark_amd: registered the `awq` config, but vLLM's "
                              f"get_quantization_config('awq') returns {got!r}; linear and fused-MoE layers "
                              "may stay on vLLM's kernels (the two AWQ ops are rebound either way)")
                return False
        return True
    warnings.warn("server_benchmark_amd: vLLM's quantization registry does not look as expected; only the two "
                  "AWQ ops were rebound (prefill >= 256 rows and fused-MoE layers stay on vLLM's kernels)")
    return False


def register() -> list:
    """Rebinds vllm._custom_ops.{awq_dequantize, awq_gemm} and registers the `awq` quantisation
    config; returns what it did (the rebound op names, plus "quantization:awq" when the config
    was registered).  Raises ImportError when vLLM is absent and RuntimeError when the library
    cannot be loaded (there is no fallback: a server that silently kept its own kernels would
    benchmark the wrong thing)."""
    try:
        custom_ops = importlib.import_module("vllm._custom_ops")
    except ImportError as e:
        raise ImportError("server_benchmark_amd.vllm_plugin needs vLLM (vllm._custom_ops) "
                          "in the same environment") from e
    from . import _lib, ops
    _lib.load()                       # fail at start-up, not at the first request
    done = []
    for name in _REBOUND:
        setattr(custom_ops, name, getattr(ops, name))
        done.append(name)
    # vLLM on ROCm routes AWQ through Triton kernels when this switch is on; the rebound ops
    # are only reached with it off
    try:
        envs = importlib.import_module("vllm.envs")
        if getattr(envs, "VLLM_USE_TRITON_AWQ", False):
            import os
            os.environ["VLLM_USE_TRITON_AWQ"] = "0"
            if hasattr(envs, "VLLM_USE_TRITON_AWQ"):
                try:
                    setattr(envs, "VLLM_USE_TRITON_AWQ", False)
                except Exception:      # lazily evaluated env table: the variable is enough
                    pass
    except ImportError:
        pass
    if _register_quant_config():
        done.append("quantization:awq")
    return done
