"""RMSNorm, alone or fused with the per-token activation quantizer of the Linear that follows it.

``RMSNorm`` has the constructor and forward of the reference module
(nn_models/modules/nonlinear/norm.py:4-16).  The fused functions replace the pair
"norm, then quantize inside the next Linear" (nn_models/modules/nonlinear/block.py:68,76 followed by
linear_sq.py:55-65 or linear_fp8.py:40-63) by one kernel that reads the activations once.
"""
from __future__ import annotations

import torch
from torch import nn

from . import _abi
from .quantize import _as_rows


def _check_weight(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    if weight.dtype != x.dtype or weight.device != x.device or weight.numel() != x.shape[-1]:
        raise RuntimeError("RMSNorm weight must be a [K] tensor with the dtype and device of the activations")
    return weight.contiguous()


@torch.no_grad()
def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6, _inv_dump: torch.Tensor | None = None):
    """weight * (fp32(x) * rsqrt(mean(fp32(x)^2) + eps)).to(x.dtype), one kernel."""
    rows = _as_rows(x)
    w = _check_weight(rows, weight)
    M, K = rows.shape
    y = torch.empty((M, K), dtype=rows.dtype, device=rows.device)
    if M:
        _abi.check(_abi.lib().llmq_rmsnorm(rows.data_ptr(), _abi.dtype_code(rows.dtype), M, K,
                                           rows.stride(0) if M > 1 else K, w.data_ptr(), float(eps), y.data_ptr(),
                                           _abi.ptr(_inv_dump), _abi.stream_of(rows)), "llmq_rmsnorm")
    return y.view(x.shape)


def _fused(x, weight, eps, fp8, scale_dtype, return_normed, inv_dump):
    rows = _as_rows(x)
    w = _check_weight(rows, weight)
    M, K = rows.shape
    dev = rows.device
    q = torch.empty((M, K), dtype=torch.float8_e4m3fn if fp8 else torch.int8, device=dev)
    scale = torch.empty((M, 1), dtype=torch.float32 if fp8 else scale_dtype, device=dev)
    y = torch.empty((M, K), dtype=rows.dtype, device=dev) if return_normed else None
    if M:
        L = _abi.lib()
        ldx = rows.stride(0) if M > 1 else K
        if fp8:
            _abi.check(L.llmq_rmsnorm_quant_fp8_per_token(
                rows.data_ptr(), _abi.dtype_code(rows.dtype), M, K, ldx, w.data_ptr(), float(eps), _abi.ptr(y),
                q.data_ptr(), scale.data_ptr(), _abi.ptr(inv_dump), _abi.stream_of(rows)),
                "llmq_rmsnorm_quant_fp8_per_token")
        else:
            _abi.check(L.llmq_rmsnorm_quant_i8_per_token(
                rows.data_ptr(), _abi.dtype_code(rows.dtype), M, K, ldx, w.data_ptr(), float(eps), _abi.ptr(y),
                q.data_ptr(), scale.data_ptr(), _abi.dtype_code(scale_dtype), _abi.ptr(inv_dump),
                _abi.stream_of(rows)), "llmq_rmsnorm_quant_i8_per_token")
    out = (q.view(x.shape), scale.view(*x.shape[:-1], 1))
    return out + (y.view(x.shape),) if return_normed else out


@torch.no_grad()
def rmsnorm_quantize_activation_per_token_absmax(x, weight, eps: float = 1e-6, scale_dtype=None,
                                                 return_normed: bool = False, _inv_dump=None):
    """RMSNorm followed by quantize_activation_per_token_absmax, fused.

    -> (int8 like x, scales [.., 1] in x.dtype or ``scale_dtype``=torch.float32[, normalised activations])."""
    return _fused(x, weight, eps, False, scale_dtype or x.dtype, return_normed, _inv_dump)


@torch.no_grad()
def rmsnorm_per_token_quantize(x, weight, eps: float = 1e-6, return_normed: bool = False, _inv_dump=None):
    """RMSNorm followed by per_token_quantize (e4m3fn, fp32 scales), fused."""
    return _fused(x, weight, eps, True, torch.float32, return_normed, _inv_dump)


class RMSNorm(nn.Module):
    """Drop-in for the reference RMSNorm: same constructor (a ready weight tensor, eps) and forward."""

    def __init__(self, weight, eps=1e-6):
        super().__init__()
        self.weight = weight
        self.variance_epsilon = eps

    def forward(self, hidden_states):
        return rmsnorm(hidden_states, self.weight, self.variance_epsilon)

    def forward_quantized(self, hidden_states, fp8: bool = False, return_normed: bool = False):
        """Normalise and quantize per token in one pass, for a W8A8 / FP8 Linear that accepts (q, scale)."""
        if fp8:
            return rmsnorm_per_token_quantize(hidden_states, self.weight, self.variance_epsilon, return_normed)
        return rmsnorm_quantize_activation_per_token_absmax(hidden_states, self.weight, self.variance_epsilon,
                                                            torch.float32, return_normed)
