"""Fusing sibling quantized Linear modules that read the same activations (q/k/v, gate/up) into one.

Mirrors ``fuse_qkv`` / ``fuse_linears`` of the reference (utils/fused_utils.py:43-104), which fuses AWQ
modules only and leaves SmoothQuant and FP8-dynamic qkv unfused (its comment at :49 calls that homework).
With dynamic per-token activation scales and per-channel weight scales the fusion is exact for those two as
well: the scales depend only on the shared input, so the fused module's output is the concatenation of the
separate outputs bit for bit.  Modules whose activation scale is a stored per-module constant (SmoothQuant
per-tensor, FP8 static) are returned unfused, as in the reference, and so are FP8-dynamic modules with
per_tensor=True: they quantize the activations per tensor, run the tensor-wise kernel and return the module's
dtype, none of which a per-channel fused module reproduces exactly.
"""
from __future__ import annotations

import torch

from .linear import FP8DynamicLinear, FP8StaticLinear, SqW8A8BBF16OBF16PerChannel, SqW8A8BBF16OBF16PerTensor, WQLinear_GEMM


def _cat_bias(linears):
    if linears[0].bias is None:
        return None
    return torch.cat([l.bias for l in linears], dim=0)


def fuse_linears(linears):
    """-> one module computing torch.cat([l(x) for l in linears], -1), or the input list if the kind of
    module cannot be fused exactly."""
    first = linears[0]
    kind = type(first)
    if any(type(l) is not kind or l.in_features != first.in_features for l in linears):
        raise RuntimeError("fuse_linears needs modules of one class with the same in_features")
    if any((l.bias is None) != (first.bias is None) for l in linears):
        raise RuntimeError("fuse_linears needs all or none of the modules to carry a bias")
    n_out = sum(l.out_features for l in linears)
    if kind is WQLinear_GEMM:
        if any(l.group_size != first.group_size or l.w_bit != first.w_bit for l in linears):
            raise RuntimeError("AWQ modules with different group sizes cannot be fused")
        fused = WQLinear_GEMM(first.w_bit, first.group_size, first.in_features, n_out, first.bias is not None,
                              first.qweight.device)
        fused.qweight = torch.cat([l.qweight for l in linears], dim=1).contiguous()
        fused.qzeros = torch.cat([l.qzeros for l in linears], dim=1).contiguous()
        fused.scales = torch.cat([l.scales for l in linears], dim=1).contiguous()
        fused.bias = _cat_bias(linears)
        return fused
    if kind is SqW8A8BBF16OBF16PerChannel:
        fused = SqW8A8BBF16OBF16PerChannel(first.w_bit, first.group_size, first.in_features, n_out,
                                           first.bias is not None, dev=first.qweight.device, dtype=first.dtype)
        fused.qweight = torch.cat([l.qweight for l in linears], dim=0).contiguous()
        fused.weight_scale = torch.cat([l.weight_scale.reshape(-1) for l in linears], dim=0).contiguous()
        fused.bias = _cat_bias(linears)
        return fused
    if kind is FP8DynamicLinear:
        if any(l.per_tensor for l in linears):
            return list(linears)  # per-tensor activation scale + tensor-wise kernel: not reproduced by a fused module
        if any(l.dtype != first.dtype or l.qdtype != first.qdtype for l in linears):
            raise RuntimeError("FP8 modules with different dtypes cannot be fused")
        dev = first.weight.device
        fused = FP8DynamicLinear(first.in_features, n_out, first.bias is not None, dev=dev, dtype=first.dtype,
                                 qdtype=first.qdtype, per_tensor=False)
        fused.weight.data = torch.cat([l.weight.data for l in linears], dim=0).contiguous()
        fused.weight_scale.data = torch.cat([l.weight_scale.data.reshape(-1, 1) for l in linears], dim=0).contiguous()
        if first.bias is not None:
            fused.bias.data = _cat_bias(linears)
        return fused
    if kind in (SqW8A8BBF16OBF16PerTensor, FP8StaticLinear):
        return list(linears)  # per-module stored activation scales: not fusable without changing results
    raise RuntimeError(f"fuse_linears: unsupported module class {kind.__name__}")


def fuse_qkv(module, q_proj, k_proj, v_proj):
    """Reference signature (utils/fused_utils.py:43): -> the fused qkv module, or the (q, k, v) tuple when the
    module kind is not fusable.  ``module`` (the attention block) is accepted for compatibility."""
    fused = fuse_linears([q_proj, k_proj, v_proj])
    return (q_proj, k_proj, v_proj) if isinstance(fused, list) else fused
