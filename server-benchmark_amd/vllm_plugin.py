"""vLLM general plugin: makes the servers the harness starts (reference
utils/generate_compose.py:85-93, AWQ checkpoints of config.yaml:36,47,51,134) run their AWQ
layers on this library.

vLLM loads every entry point of the group `vllm.general_plugins` in each worker process
before the model is built.  `register()` rebinds the two custom ops that vLLM's own
`AWQLinearMethod.apply` calls (`awq_dequantize`, `awq_gemm` in `vllm._custom_ops`) to the
functions of this package, so weight loading, sharding and the layer classes stay vLLM's and
only the arithmetic changes hands.  Packaging side (pyproject.toml of the wheel that ships
this package):

    [project.entry-points."vllm.general_plugins"]
    awq_mi355x = "server_benchmark_amd.vllm_plugin:register"

vLLM is not part of this build's image, so nothing here is exercised against a real vLLM;
the rebinding itself is tested against a stand-in module.
"""
from __future__ import annotations

import importlib

_REBOUND = ("awq_dequantize", "awq_gemm")


def register() -> list:
    """Rebinds vllm._custom_ops.{awq_dequantize, awq_gemm}; returns the names it rebound.
    Raises ImportError when vLLM is absent and RuntimeError when the library cannot be
    loaded (there is no fallback: a server that silently kept its own kernels would
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
    return done
