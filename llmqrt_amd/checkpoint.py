"""Loading a quantized checkpoint into the quantized Linear modules.

The reference keeps its quantization settings under ``quantization_config`` in the checkpoint's
``config.json`` (core/config.py:8-112) and loads by first swapping every ``nn.Linear`` of the model for an
empty quantized module (``from_linear(..., init_only=True)``, core/base.py:306-340) and then filling the
buffers by name from the checkpoint files (core/base.py:213-221).  The modules of this package keep the
reference's buffer names, shapes and dtypes, so the same two steps work on a reference-format checkpoint:

    cfg = QuantConfig.from_pretrained(path)
    replace_linears(model, cfg, dtype=torch.bfloat16)
    load_quantized_weights(model, path)

Only local directories and ``.safetensors`` files are read; nothing is downloaded.  FP8 checkpoints store
their weights as fp8-representable values in the model dtype; the modules cast them to fp8 once, on the
first forward, instead of on every forward (nn_models/modules/linear/linear_fp8.py:188).
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Iterable

import torch
from torch import nn

from .linear import SqW8A8BBF16OBF16PerChannel, method_to_linear


@dataclass
class QuantConfig:
    """Field names and defaults of the reference's QuantConfig (core/config.py:9-20)."""
    quant_method: str = "awq"          # "awq" | "sq" | "fp8_static_quant" | "fp8_dynamic_quant"
    zero_point: bool = False
    q_group_size: int = 0
    w_bit: int = 8
    version: str = "gemm"
    modules_to_not_convert: list = field(default_factory=lambda: ["lm_head"])
    fp8_static_quant: bool = False
    kv_cache_quant_layers: list = field(default_factory=list)
    per_tensor: bool = True

    @classmethod
    def from_dict(cls, d: dict | None = None) -> "QuantConfig":
        cfg = cls(**d) if d else cls()
        cfg.version = cfg.version.lower()
        return cfg

    @classmethod
    def from_transformers_dict(cls, d: dict) -> "QuantConfig":
        """The key names used inside config.json (core/config.py:88-112): group_size, bits."""
        known = {"quant_method": "quant_method", "zero_point": "zero_point", "group_size": "q_group_size",
                 "bits": "w_bit", "fp8_static_quant": "fp8_static_quant",
                 "kv_cache_quant_layers": "kv_cache_quant_layers",
                 "modules_to_not_convert": "modules_to_not_convert", "per_tensor": "per_tensor"}
        kwargs = {ours: d[theirs] for theirs, ours in known.items() if d.get(theirs) is not None}
        return cls.from_dict(kwargs)

    @classmethod
    def from_pretrained(cls, save_dir: str) -> "QuantConfig":
        path = os.path.join(save_dir, "config.json")
        if not os.path.isfile(path):
            raise FileNotFoundError(f"{path}: only local checkpoint directories are supported")
        with open(path, "r", encoding="utf-8") as f:
            loaded = json.load(f)
        q = loaded.get("quantization_config")
        return cls.from_transformers_dict(q) if q else cls()

    def to_transformers_dict(self) -> dict:
        return {"quant_method": self.quant_method, "zero_point": self.zero_point, "group_size": self.q_group_size,
                "bits": self.w_bit, "fp8_static_quant": self.fp8_static_quant,
                "kv_cache_quant_layers": self.kv_cache_quant_layers,
                "modules_to_not_convert": self.modules_to_not_convert, "per_tensor": self.per_tensor}


def _set_submodule(root: nn.Module, name: str, new: nn.Module) -> None:
    parent = root
    parts = name.split(".")
    for p in parts[:-1]:
        parent = parent[int(p)] if p.isdigit() and not hasattr(parent, p) else getattr(parent, p)
    setattr(parent, parts[-1], new)


def replace_linears(model: nn.Module, cfg: QuantConfig, dtype=torch.bfloat16) -> list[str]:
    """Swap every nn.Linear whose name contains none of ``cfg.modules_to_not_convert`` for an empty quantized
    module of the configured kind (buffers allocated, not filled).  -> the names that were replaced.

    ``quant_method == "sq"`` with ``per_tensor == False`` selects the per-token x per-channel SmoothQuant module,
    which the reference declares but does not implement."""
    kind = method_to_linear[cfg.quant_method]
    if cfg.quant_method == "sq" and not cfg.per_tensor:
        kind = SqW8A8BBF16OBF16PerChannel
    skip = cfg.modules_to_not_convert or []
    targets = [(n, m) for n, m in model.named_modules()
               if isinstance(m, nn.Linear) and n and not any(key in n for key in skip)]
    for name, lin in targets:
        q = kind.from_linear(lin, cfg.w_bit, cfg.q_group_size, True, dtype=dtype, per_tensor=cfg.per_tensor)
        _set_submodule(model, name, q)
    return [n for n, _ in targets]


def _checkpoint_files(path: str) -> list[str]:
    if os.path.isfile(path):
        return [path]
    index = os.path.join(path, "model.safetensors.index.json")
    if os.path.isfile(index):
        with open(index, "r", encoding="utf-8") as f:
            names = sorted(set(json.load(f)["weight_map"].values()))
        return [os.path.join(path, n) for n in names]
    files = sorted(os.path.join(path, f) for f in os.listdir(path) if f.endswith(".safetensors"))
    if not files:
        raise FileNotFoundError(f"no .safetensors files under {path}")
    return files


def load_quantized_weights(model: nn.Module, path: str, device=None) -> tuple[list[str], list[str]]:
    """Fill parameters and buffers by name from the ``.safetensors`` file(s) at ``path`` (a file, a directory,
    or a directory with a ``model.safetensors.index.json``).  Shapes and dtypes must match what the modules
    allocated (scalars may come as 0-dim or 1-element tensors).  -> (missing names, unexpected names)."""
    from safetensors import safe_open

    own = dict(model.named_parameters())
    own.update(dict(model.named_buffers()))
    seen, unexpected = set(), []
    for file in _checkpoint_files(path):
        with safe_open(file, framework="pt", device="cpu") as f:
            for key in f.keys():
                dst = own.get(key)
                if dst is None:
                    unexpected.append(key)
                    continue
                src = f.get_tensor(key)
                if src.numel() == dst.numel() and src.shape != dst.shape and dst.numel() == 1:
                    src = src.reshape(dst.shape)
                if src.shape != dst.shape:
                    raise RuntimeError(f"{key}: checkpoint shape {tuple(src.shape)} != module shape {tuple(dst.shape)}")
                if src.dtype != dst.dtype and not (src.is_floating_point() and dst.is_floating_point()):
                    raise RuntimeError(f"{key}: checkpoint dtype {src.dtype} != module dtype {dst.dtype}")
                with torch.no_grad():
                    dst.copy_(src.to(dst.dtype))
                seen.add(key)
    for m in model.modules():   # cached fp8 casts of weights that were just overwritten
        if hasattr(m, "invalidate_cache"):
            m.invalidate_cache()
    if device is not None:
        model.to(device)
    return sorted(k for k in own if k not in seen), unexpected


def named_quantized_linears(model: nn.Module) -> Iterable[tuple[str, nn.Module]]:
    kinds = tuple(set(method_to_linear.values()) | {SqW8A8BBF16OBF16PerChannel})
    return ((n, m) for n, m in model.named_modules() if isinstance(m, kinds))
