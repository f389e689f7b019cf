"""Activation quantizers of the quantized Linear modules, one HIP kernel each.

Same names, arguments and return values as the reference's eager-torch helpers:
``quantize_activation_per_token_absmax`` / ``quantize_activation_per_tensor_absmax``
(nn_models/modules/linear/linear_sq.py:44-65) and ``per_token_quantize`` /
``per_tensor_quantize`` / ``static_per_tensor_quantize``
(nn_models/modules/linear/linear_fp8.py:11-63).  Results are bit-identical to those
functions evaluated by torch on the same input.
"""
from __future__ import annotations

import torch

from . import _abi


def _as_rows(t: torch.Tensor) -> torch.Tensor:
    if t.dtype not in (torch.bfloat16, torch.float16):
        raise RuntimeError(f"activation dtype must be bf16 or fp16, got {t.dtype}")
    if not t.is_cuda:
        raise RuntimeError("activation must live on the GPU")
    x = t.reshape(-1, t.shape[-1])
    if x.stride(-1) != 1 or (x.shape[0] > 1 and x.stride(0) % 8) or x.data_ptr() % 16:
        x = x.contiguous()
    if x.shape[-1] % 8:
        raise RuntimeError("the last dimension must be a multiple of 8")
    return x


def _int8_per_token(t: torch.Tensor, scale_dtype, floor: float = 1e-5):
    x = _as_rows(t)
    M, K = x.shape
    q = torch.empty((M, K), dtype=torch.int8, device=x.device)
    scale = torch.empty((M, 1), dtype=scale_dtype, device=x.device)
    if M:
        _abi.check(_abi.lib().llmq_quant_i8_per_token_floor(
            x.data_ptr(), _abi.dtype_code(x.dtype), M, K, x.stride(0) if M > 1 else K, q.data_ptr(),
            scale.data_ptr(), _abi.dtype_code(scale_dtype), floor, _abi.stream_of(x)), "llmq_quant_i8_per_token_floor")
    return q.view(*t.shape), scale.view(*t.shape[:-1], 1)


def _int8_per_tensor(t: torch.Tensor, floor: float):
    x = _as_rows(t)
    M, K = x.shape
    q = torch.empty((M, K), dtype=torch.int8, device=x.device)
    scale = torch.empty((), dtype=t.dtype, device=x.device)
    ws_bytes = _abi.lib().llmq_quant_workspace_bytes()
    ws = _abi.workspaces.get(x.device, ws_bytes)
    _abi.check(_abi.lib().llmq_quant_i8_per_tensor_floor(
        x.data_ptr(), _abi.dtype_code(x.dtype), M, K, x.stride(0) if M > 1 else K, q.data_ptr(),
        scale.data_ptr(), _abi.dtype_code(t.dtype), floor, ws.data_ptr(), ws.numel(), _abi.stream_of(x)),
        "llmq_quant_i8_per_tensor_floor")
    return q.view(*t.shape), scale


@torch.no_grad()
def quantize_activation_per_token_absmax(t: torch.Tensor, n_bits: int = 8):
    """-> (int8 tensor like t, scales [.., 1] in t.dtype)."""
    assert n_bits == 8
    return _int8_per_token(t, t.dtype)


@torch.no_grad()
def quantize_activation_per_token_absmax_f32(t: torch.Tensor):
    """Same quantizer, scales widened to fp32 (the form the GEMM epilogue consumes)."""
    return _int8_per_token(t, torch.float32)


@torch.no_grad()
def quantize_activation_per_tensor_absmax(t: torch.Tensor, n_bits: int = 8):
    """-> (int8 tensor like t, 0-dim scale in t.dtype)."""
    assert n_bits == 8
    return _int8_per_tensor(t, 1e-5)


@torch.no_grad()
def dynamic_quantize_activation_per_token_absmax(t: torch.Tensor):
    """utils/quantization_utils.py:65-71: the per-token quantizer with the absmax clamped at 1e-8 instead of 1e-5.
    -> (int8 tensor like t, scales [.., 1] in t.dtype).  The reference also overwrites ``t`` with the rounded
    quotients (in-place ``div_().round_().clamp_()``); here ``t`` is left as it was."""
    return _int8_per_token(t, t.dtype, 1e-8)


@torch.no_grad()
def dynamic_quantize_activation_per_tensor_absmax(t: torch.Tensor):
    """utils/quantization_utils.py:57-62: one global absmax clamped at 1e-8.  -> (int8 like t, 0-dim scale in t.dtype)."""
    return _int8_per_tensor(t, 1e-8)


@torch.no_grad()
def per_token_quantize(tensor: torch.Tensor):
    """-> (float8_e4m3fn tensor like `tensor`, fp32 scales [.., 1])."""
    if tensor.numel() == 0:
        return (torch.empty_like(tensor, dtype=torch.float8_e4m3fn),
                torch.ones((*tensor.shape[:-1], 1), dtype=torch.float32))
    x = _as_rows(tensor)
    M, K = x.shape
    q = torch.empty((M, K), dtype=torch.float8_e4m3fn, device=x.device)
    scale = torch.empty((M, 1), dtype=torch.float32, device=x.device)
    _abi.check(_abi.lib().llmq_quant_fp8_per_token(
        x.data_ptr(), _abi.dtype_code(x.dtype), M, K, x.stride(0) if M > 1 else K, q.data_ptr(),
        scale.data_ptr(), _abi.stream_of(x)), "llmq_quant_fp8_per_token")
    return q.view(*tensor.shape), scale.view(*tensor.shape[:-1], 1)


@torch.no_grad()
def per_tensor_quantize(tensor: torch.Tensor):
    """-> (float8_e4m3fn tensor, 0-dim fp32 scale)."""
    if tensor.numel() == 0:
        amax = torch.tensor(16.0, dtype=tensor.dtype)
        scale = (amax.clamp(min=1e-12) / 448.0).float().to(tensor.device)
        return torch.empty_like(tensor, dtype=torch.float8_e4m3fn), scale
    x = _as_rows(tensor)
    M, K = x.shape
    q = torch.empty((M, K), dtype=torch.float8_e4m3fn, device=x.device)
    scale = torch.empty((), dtype=torch.float32, device=x.device)
    ws = _abi.workspaces.get(x.device, _abi.lib().llmq_quant_workspace_bytes())
    _abi.check(_abi.lib().llmq_quant_fp8_per_tensor(
        x.data_ptr(), _abi.dtype_code(x.dtype), M, K, x.stride(0) if M > 1 else K, q.data_ptr(),
        scale.data_ptr(), ws.data_ptr(), ws.numel(), _abi.stream_of(x)), "llmq_quant_fp8_per_tensor")
    return q.view(*tensor.shape), scale


@torch.no_grad()
def static_per_tensor_quantize(tensor: torch.Tensor, scale) -> torch.Tensor:
    """`scale`: fp32 tensor with one element (the quotient is then formed in fp32, as torch's
    type promotion does for tensor / fp32-tensor) or a Python float / 0-dim tensor (quotient
    rounded to tensor.dtype)."""
    if tensor.numel() == 0:
        return torch.empty_like(tensor, dtype=torch.float8_e4m3fn)
    x = _as_rows(tensor)
    M, K = x.shape
    if isinstance(scale, torch.Tensor):
        promote = scale.dim() > 0 and scale.dtype == torch.float32
        sdev = scale.detach().reshape(-1)[:1].to(device=x.device, dtype=torch.float32)
    else:
        promote = False
        sdev = torch.tensor([float(scale)], dtype=torch.float32, device=x.device)
    q = torch.empty((M, K), dtype=torch.float8_e4m3fn, device=x.device)
    _abi.check(_abi.lib().llmq_quant_fp8_static(
        x.data_ptr(), _abi.dtype_code(x.dtype), M, K, x.stride(0) if M > 1 else K, q.data_ptr(),
        sdev.data_ptr(), int(promote), _abi.stream_of(x)), "llmq_quant_fp8_static")
    return q.view(*tensor.shape)


@torch.no_grad()
def quantize_weight_per_channel_absmax(w: torch.Tensor):
    """Replaces quantize_weight_per_channel_absmax (utils/quantization_utils.py:27-38): w [N, K] bf16 / fp16 / fp32 on
    the GPU -> (int8 [N, K], scales [N, 1] in w.dtype).  Unlike the reference it leaves w untouched."""
    assert w.dim() == 2 and w.is_cuda and w.dtype in (torch.bfloat16, torch.float16, torch.float32)
    if w.stride(1) != 1:
        w = w.contiguous()
    N, K = w.shape
    q = torch.empty((N, K), dtype=torch.int8, device=w.device)
    scale = torch.empty((N, 1), dtype=w.dtype, device=w.device)
    if N:
        _abi.check(_abi.lib().llmq_quant_i8_weight_per_channel(
            w.data_ptr(), _abi.dtype_code(w.dtype), N, K, w.stride(0), q.data_ptr(), scale.data_ptr(),
            _abi.stream_of(w)), "llmq_quant_i8_weight_per_channel")
    return q, scale
