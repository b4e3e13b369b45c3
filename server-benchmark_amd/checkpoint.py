"""AWQ checkpoint reader: `*.safetensors` + `config.json` of an AutoAWQ "GEMM" checkpoint on
a local path -> the `qweight` / `qzeros` / `scales` parameters of this package's layers.

This is the on-disk side of the linear path: the servers the harness starts read exactly such
folders (reference config.yaml:36,47,51,134 name the AWQ repositories, mounted at
/hf_models by utils/generate_compose.py:78).  Per quantised linear `<prefix>` a checkpoint
holds `<prefix>.qweight int32 [K, N/8]`, `<prefix>.qzeros int32 [K/G, N/8]` and
`<prefix>.scales fp16 [K/G, N]`; the quantisation parameters sit in `config.json` under
`quantization_config` (or in `quant_config.json` / `quantize_config.json`).  Tensors are read
with safetensors (nothing in a file is executed); no network access, local paths only.
"""
from __future__ import annotations

import json
import pathlib
from typing import Iterable, Sequence

import torch
from safetensors import safe_open

from .awq import AWQConfig

_SUFFIXES = ("qweight", "qzeros", "scales")


class CheckpointError(ValueError):
    pass


def read_awq_config(model_dir) -> AWQConfig:
    """AWQConfig of a checkpoint folder.  Raises CheckpointError when the folder is not a
    4-bit AWQ checkpoint in the GEMM layout."""
    d = pathlib.Path(model_dir)
    cfg = None
    main = d / "config.json"
    if main.is_file():
        cfg = json.loads(main.read_text()).get("quantization_config")
    if cfg is None:
        for name in AWQConfig.get_config_filenames():
            f = d / name
            if f.is_file():
                cfg = json.loads(f.read_text())
                break
    if cfg is None:
        raise CheckpointError(f"{d}: no quantization_config in config.json and no quant_config.json / "
                              "quantize_config.json")
    method = str(cfg.get("quant_method", "awq")).lower()
    if method != "awq":
        raise CheckpointError(f"{d}: quant_method is {method!r}, not 'awq'")
    version = str(cfg.get("version", "gemm")).lower()
    if version != "gemm":
        raise CheckpointError(f"{d}: AWQ layout version {version!r} is not supported (only 'gemm')")
    try:
        return AWQConfig.from_config(cfg)
    except ValueError as e:
        raise CheckpointError(f"{d}: {e}") from e


class AWQCheckpoint:
    """Index of the tensors of a checkpoint folder, read lazily, validated on read."""

    def __init__(self, model_dir):
        self.dir = pathlib.Path(model_dir)
        if not self.dir.is_dir():
            raise CheckpointError(f"{self.dir} is not a directory (local paths only)")
        self.config = read_awq_config(self.dir)
        self._where = {}
        files = sorted(self.dir.glob("*.safetensors"))
        if not files:
            raise CheckpointError(f"{self.dir}: no *.safetensors files")
        index = self.dir / "model.safetensors.index.json"
        if index.is_file():
            for name, fname in json.loads(index.read_text()).get("weight_map", {}).items():
                self._where[name] = self.dir / fname
        else:
            for f in files:
                with safe_open(str(f), framework="pt", device="cpu") as h:
                    for name in h.keys():
                        self._where[name] = f

    # ------------------------------------------------------------------ raw access
    def names(self):
        return sorted(self._where)

    def tensor(self, name: str) -> torch.Tensor:
        f = self._where.get(name)
        if f is None:
            raise CheckpointError(f"{self.dir}: tensor {name!r} not found")
        with safe_open(str(f), framework="pt", device="cpu") as h:
            return h.get_tensor(name)

    def linear_prefixes(self):
        """Prefixes of the quantised linears (those that have a .qweight)."""
        return sorted(n[: -len(".qweight")] for n in self._where if n.endswith(".qweight"))

    # ------------------------------------------------------------------ one linear
    def read_linear(self, prefix: str):
        """(qweight, scales, qzeros) of one linear, checked against the AWQ layout."""
        qw, qz, sc = (self.tensor(f"{prefix}.{s}") for s in _SUFFIXES)
        if qw.dtype != torch.int32 or qz.dtype != torch.int32:
            raise CheckpointError(f"{prefix}: qweight / qzeros must be int32, got {qw.dtype} / {qz.dtype}")
        if sc.dtype != torch.float16:
            raise CheckpointError(f"{prefix}: scales must be float16, got {sc.dtype}")
        if qw.dim() != 2 or qz.dim() != 2 or sc.dim() != 2:
            raise CheckpointError(f"{prefix}: qweight / qzeros / scales must be matrices")
        K, NW = qw.shape
        N = NW * self.config.pack_factor
        G = K if self.config.group_size == -1 else self.config.group_size
        if K % G != 0:
            raise CheckpointError(f"{prefix}: K={K} is not a multiple of the group size {G}")
        if tuple(qz.shape) != (K // G, NW):
            raise CheckpointError(f"{prefix}: qzeros shape {tuple(qz.shape)} != {(K // G, NW)}")
        if tuple(sc.shape) != (K // G, N):
            raise CheckpointError(f"{prefix}: scales shape {tuple(sc.shape)} != {(K // G, N)}")
        return qw.contiguous(), sc.contiguous(), qz.contiguous()

    def read_merged(self, prefixes: Sequence[str]):
        """Several linears over the same input, concatenated along the output dimension
        (q/k/v -> qkv_proj, gate/up -> gate_up_proj): word columns never straddle a part
        because every N is a multiple of 8."""
        parts = [self.read_linear(p) for p in prefixes]
        K = parts[0][0].shape[0]
        for p, t in zip(prefixes, parts):
            if t[0].shape[0] != K:
                raise CheckpointError(f"{p}: K={t[0].shape[0]} differs from {prefixes[0]} (K={K})")
        return tuple(torch.cat([t[i] for t in parts], dim=1).contiguous() for i in range(3))

    def load_linear(self, layer: torch.nn.Module, prefixes) -> None:
        """Fill the parameters AWQLinearMethod.create_weights registered on `layer` from one
        prefix or a list of prefixes to merge."""
        if isinstance(prefixes, str):
            prefixes = [prefixes]
        qw, sc, qz = self.read_merged(list(prefixes))
        for name, t in (("qweight", qw), ("scales", sc), ("qzeros", qz)):
            p = getattr(layer, name)
            if tuple(p.shape) != tuple(t.shape):
                raise CheckpointError(f"{'+'.join(prefixes)}.{name}: checkpoint shape {tuple(t.shape)} != layer "
                                      f"shape {tuple(p.shape)}")
            p.data.copy_(t)

    # ------------------------------------------------------------------ expert stacks
    def load_experts(self, layer: torch.nn.Module, prefix: str, num_experts: int,
                     names: Iterable[str] = ("gate_proj", "up_proj", "down_proj")) -> None:
        """Fill the w13 / w2 stacks AWQMoEMethod.create_weights registered on `layer` from
        `<prefix>.<e>.{gate_proj,up_proj,down_proj}`; w13 columns are [gate | up]."""
        gate, up, down = names
        for e in range(num_experts):
            w13 = self.read_merged([f"{prefix}.{e}.{gate}", f"{prefix}.{e}.{up}"])
            w2 = self.read_linear(f"{prefix}.{e}.{down}")
            for stack, (qw, sc, qz) in (("w13", w13), ("w2", w2)):
                for name, t in (("qweight", qw), ("scales", sc), ("qzeros", qz)):
                    p = getattr(layer, f"{stack}_{name}")
                    if tuple(p.shape[1:]) != tuple(t.shape):
                        raise CheckpointError(f"{prefix}.{e} {stack}_{name}: checkpoint shape {tuple(t.shape)} != "
                                              f"layer shape {tuple(p.shape[1:])}")
                    p.data[e].copy_(t)
