"""HIP-backed drop-in for the reference's pybind extension ``runtime.sq_fp8_kernels``
(csrc/bindings.cpp:7-14): same op names, positional signatures, tensor contracts and error
behaviour (RuntimeError on a violated check), computing on gfx950 MFMA kernels through the
C ABI of libllmq_gfx950.so.

Tensor contracts (as the reference checks them, csrc/fp8/sm89_fp8_rowwise_fbgemm.cu:526-575):
``input`` [M, K] row-major, ``weight`` a [K, N] view with stride (1, ld) of an [N, K]
row-major tensor, ``bias`` 1-D [N].
"""
from __future__ import annotations

from typing import Optional

import torch

from . import _abi

_FP8_FORMATS = {torch.float8_e4m3fn: _abi.E4M3, torch.float8_e5m2: _abi.E5M2}
_STR_TO_DTYPE = {"bfloat16": torch.bfloat16, "float16": torch.float16}


def _check(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


def _check_operands(x: torch.Tensor, w: torch.Tensor, what: str):
    _check(x.is_cuda, f"{what}: input must be a GPU tensor")
    _check(x.device == w.device, f"{what}: input and weight must be on the same device")
    _check(x.dim() == 2 and w.dim() == 2, f"{what}: input and weight must be 2-D")
    _check(x.size(1) == w.size(0), f"{what}: input is [M, K], weight must be [K, N]")
    _check(x.stride(1) == 1 and x.stride(0) >= x.size(1), f"{what}: input must be row-major")
    _check(w.stride(0) == 1 and w.stride(1) >= w.size(0),
           f"{what}: weight must be column-major, i.e. the .t() view of an [N, K] row-major tensor")
    M, K = x.shape
    N = w.size(1)
    _check(K % 16 == 0, f"{what}: K must be a multiple of 16")
    return M, N, K


def _check_bias(bias: Optional[torch.Tensor], w: torch.Tensor, N: int, allowed, what: str):
    if bias is None:
        return
    _check(bias.device == w.device, f"{what}: bias must be on the weight's device")
    _check(bias.dtype in allowed, f"{what}: unsupported bias dtype {bias.dtype}")
    _check(bias.dim() == 1 and bias.size(0) == N and bias.stride(0) == 1, f"{what}: bias must be a contiguous [N] vector")


def _scalar(value, device):
    """Python number -> (float, None); GPU tensor -> (1.0, fp32 device scalar) without a host sync."""
    if isinstance(value, torch.Tensor):
        if value.is_cuda:
            return 1.0, value.detach().reshape(-1)[:1].to(device=device, dtype=torch.float32)
        return float(value), None
    return float(value), None


def _run(fp8: bool, x, w, a_scale, w_scale, alpha, alpha_dev, bias, beta, out_dtype, acc_dump=None):
    M, K = x.shape
    N = w.size(1)
    out = torch.empty((M, N), dtype=out_dtype, device=x.device)
    if M == 0 or N == 0:
        return out
    L = _abi.lib()
    ws_bytes = L.llmq_gemm_workspace_bytes(M, N, K)
    ws = _abi.workspaces.get(x.device, ws_bytes)
    common = (_abi.ptr(a_scale), _abi.ptr(w_scale), float(alpha), _abi.ptr(alpha_dev), _abi.ptr(bias),
              _abi.dtype_code(bias.dtype) if bias is not None else _abi.BF16, float(beta), out.data_ptr(),
              _abi.dtype_code(out_dtype), out.stride(0), M, N, K, _abi.ptr(acc_dump), _abi.ptr(ws),
              ws.numel() if ws is not None else 0, _abi.stream_of(x))
    if fp8:
        st = L.llmq_gemm_fp8(x.data_ptr(), _FP8_FORMATS[x.dtype], x.stride(0), w.data_ptr(), w.stride(1), *common)
        _abi.check(st, "llmq_gemm_fp8")
    else:
        st = L.llmq_gemm_w8a8(x.data_ptr(), x.stride(0), w.data_ptr(), w.stride(1), *common)
        _abi.check(st, "llmq_gemm_w8a8")
    return out


@torch.no_grad()
def w8a8_int8_linear_bbf16_obf16_per_tensor(input: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor,
                                            alpha, beta, *, _acc_dump=None) -> torch.Tensor:
    """out = bias.dtype(alpha * (input @ weight) + beta * bias)   (csrc/smoothquant/sq_gemm.cu:36-160).

    ``alpha`` / ``beta``: Python floats; ``alpha`` may also be a 0-dim GPU tensor (the reference's
    caller builds it as ``input_scale * weight_scale.item()``), which is then read on the device
    instead of being synchronised to the host.  The output has ``bias.dtype`` (bf16 or fp16) and
    really holds values of that dtype (the reference writes fp16 bits whatever the bias dtype).
    """
    what = "w8a8_int8_linear_bbf16_obf16_per_tensor"
    _check(input.dtype == torch.int8 and weight.dtype == torch.int8, f"{what}: input and weight must be int8")
    M, N, K = _check_operands(input, weight, what)
    _check(bias is not None, f"{what}: bias is required (pass zeros for a bias-free layer)")
    _check_bias(bias, weight, N, (torch.bfloat16, torch.float16), what)
    a, a_dev = _scalar(alpha, input.device)
    return _run(False, input, weight, None, None, a, a_dev, bias, float(beta), bias.dtype, _acc_dump)


@torch.no_grad()
def w8a8_int8_linear_bbf16_obf16_per_channel(input: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor,
                                             alpha: torch.Tensor, beta: torch.Tensor, *, _acc_dump=None) -> torch.Tensor:
    """Per-token x per-channel dequant GEMM, the op the reference declares at
    csrc/smoothquant/sq_gemm.h:19-24 without defining it.  ``alpha``: activation scales [M, 1]
    (fp32, or the bf16/fp16 scales the quantizer returns), ``beta``: weight scales [1, N] / [N, 1]
    / [N]; out = bias.dtype((acc * alpha[m]) * beta[n] + bias[n])
    (math of utils/quantization_utils.py:89-97 plus bias)."""
    what = "w8a8_int8_linear_bbf16_obf16_per_channel"
    _check(input.dtype == torch.int8 and weight.dtype == torch.int8, f"{what}: input and weight must be int8")
    M, N, K = _check_operands(input, weight, what)
    _check(bias is not None, f"{what}: bias is required (pass zeros for a bias-free layer)")
    _check_bias(bias, weight, N, (torch.bfloat16, torch.float16), what)
    _check(isinstance(alpha, torch.Tensor) and alpha.numel() == M, f"{what}: alpha must hold one scale per token")
    _check(isinstance(beta, torch.Tensor) and beta.numel() == N, f"{what}: beta must hold one scale per channel")
    a = alpha.detach().reshape(-1).to(device=input.device, dtype=torch.float32).contiguous()
    b = beta.detach().reshape(-1).to(device=input.device, dtype=torch.float32).contiguous()
    return _run(False, input, weight, a, b, 1.0, None, bias, 1.0, bias.dtype, _acc_dump)


@torch.no_grad()
def cutlass_f8f8bf16_tensorwise_sm89(XQ: torch.Tensor, WQ: torch.Tensor, bias: Optional[torch.Tensor], alpha, beta,
                                     dtype_str: str, *, _acc_dump=None) -> torch.Tensor:
    """out = dtype(alpha * (XQ @ WQ) + beta * bias)  (csrc/fp8/sm89_fp8_tensorwise_cutlassgemm.cu:316-334).
    The name is kept for drop-in compatibility; the kernel is a gfx950 MFMA kernel."""
    what = "cutlass_f8f8bf16_tensorwise_sm89"
    _check(XQ.dtype in _FP8_FORMATS, f"{what}: XQ must be float8_e4m3fn or float8_e5m2")
    _check(WQ.dtype == torch.float8_e4m3fn, f"{what}: WQ must be float8_e4m3fn")
    M, N, K = _check_operands(XQ, WQ, what)
    _check(dtype_str in _STR_TO_DTYPE,
           f"{what}: currently only support bf16 or fp16 output dtype, the passed dtype is {dtype_str}")
    out_dtype = _STR_TO_DTYPE[dtype_str]
    _check_bias(bias, WQ, N, (torch.bfloat16, torch.float16), what)
    if bias is not None:
        _check(bias.dtype == out_dtype, f"{what}: if bias has value, dtype passed in should same as bias dtype")
    a, a_dev = _scalar(alpha, XQ.device)
    return _run(True, XQ, WQ, None, None, a, a_dev, bias, float(beta), out_dtype, _acc_dump)


@torch.no_grad()
def f8f8_tensorwise_quantized_output(XQ: torch.Tensor, WQ: torch.Tensor, bias: Optional[torch.Tensor], alpha, beta,
                                     dtype_str: str, output_scale: torch.Tensor) -> torch.Tensor:
    """cutlass_f8f8bf16_tensorwise_sm89 followed by the output quantization of FP8StaticLinear.forward
    (nn_models/modules/linear/linear_fp8.py:309-311) in one launch: the ``dtype_str`` result makes a round trip
    through e4m3fn on ``output_scale`` (a one-element fp32 GPU tensor) inside the GEMM epilogue.  -> fp32 [M, N],
    the dtype the reference's ``qoutput.to(dtype) * output_scale`` has.  No counterpart among the reference's ops."""
    what = "f8f8_tensorwise_quantized_output"
    _check(XQ.dtype in _FP8_FORMATS, f"{what}: XQ must be float8_e4m3fn or float8_e5m2")
    _check(WQ.dtype == torch.float8_e4m3fn, f"{what}: WQ must be float8_e4m3fn")
    M, N, K = _check_operands(XQ, WQ, what)
    _check(dtype_str in _STR_TO_DTYPE,
           f"{what}: currently only support bf16 or fp16 output dtype, the passed dtype is {dtype_str}")
    inter = _STR_TO_DTYPE[dtype_str]
    _check_bias(bias, WQ, N, (torch.bfloat16, torch.float16), what)
    if bias is not None:
        _check(bias.dtype == inter, f"{what}: if bias has value, dtype passed in should same as bias dtype")
    _check(isinstance(output_scale, torch.Tensor) and output_scale.numel() == 1 and output_scale.dtype == torch.float32
           and output_scale.device == XQ.device, f"{what}: output_scale must be a one-element fp32 tensor on the GPU")
    a, a_dev = _scalar(alpha, XQ.device)
    out = torch.empty((M, N), dtype=torch.float32, device=XQ.device)
    if M == 0 or N == 0:
        return out
    L = _abi.lib()
    ws = _abi.workspaces.get(XQ.device, L.llmq_gemm_fp8_quantized_output_workspace_bytes(M, N, K))
    st = L.llmq_gemm_fp8_quantized_output(
        XQ.data_ptr(), _FP8_FORMATS[XQ.dtype], XQ.stride(0), WQ.data_ptr(), WQ.stride(1), None, None, float(a),
        _abi.ptr(a_dev), _abi.ptr(bias), _abi.dtype_code(bias.dtype) if bias is not None else _abi.BF16, float(beta),
        output_scale.data_ptr(), out.data_ptr(), _abi.dtype_code(inter), out.stride(0), M, N, K, _abi.ptr(ws),
        ws.numel() if ws is not None else 0, _abi.stream_of(XQ))
    _abi.check(st, "llmq_gemm_fp8_quantized_output")
    return out


@torch.no_grad()
def cutlass_f8f8bf16_rowwise_sm89(XQ: torch.Tensor, WQ: torch.Tensor, bias: Optional[torch.Tensor],
                                  x_scale: torch.Tensor, w_scale: torch.Tensor, use_fast_accum: bool = True,
                                  *, _acc_dump=None) -> torch.Tensor:
    """out = bf16(((XQ @ WQ) * x_scale[m]) * w_scale[n] + bias[n])
    (csrc/fp8/sm89_fp8_rowwise_fbgemm.cu:582-606).  ``use_fast_accum`` is accepted and has no
    effect: the MFMA accumulates in fp32 natively."""
    what = "cutlass_f8f8bf16_rowwise_sm89"
    _check(XQ.dtype in _FP8_FORMATS, f"{what}: XQ must be float8_e4m3fn or float8_e5m2")
    _check(WQ.dtype == torch.float8_e4m3fn, f"{what}: WQ must be float8_e4m3fn")
    M, N, K = _check_operands(XQ, WQ, what)
    _check(x_scale.device == XQ.device and w_scale.device == WQ.device, f"{what}: scales must be on the GPU")
    _check(x_scale.dtype == torch.float32 and w_scale.dtype == torch.float32, f"{what}: scales must be fp32")
    _check(x_scale.dim() == 2 and w_scale.dim() == 2, f"{what}: scales must be 2-D")
    _check(x_scale.size(0) == M and x_scale.size(1) == 1, f"{what}: x_scale must be [M, 1]")
    _check(w_scale.size(0) == 1, f"Expected scale_b.size(0) == 1, but got {w_scale.size(0)}")
    _check(w_scale.size(1) == N, f"{what}: w_scale must be [1, N]")
    _check(M <= 1 or x_scale.stride(0) == 1, f"{what}: x_scale must be contiguous")
    _check(N <= 1 or w_scale.stride(1) == 1, f"{what}: w_scale must be contiguous")
    _check_bias(bias, WQ, N, (torch.bfloat16, torch.float32), what)
    return _run(True, XQ, WQ, x_scale, w_scale, 1.0, None, bias, 1.0, torch.bfloat16, _acc_dump)


# ---- one-launch linears for a few tokens (no counterpart among the reference's ops: they fuse the
# quantizer call and the GEMM op of linear_sq.py:97-138 / linear_fp8.py:199-221) ------------------------------

def dynamic_linear_max_tokens(in_features: int) -> int:
    """Largest token count the one-launch linears accept for this K (the quantized rows must fit in LDS)."""
    return int(_abi.lib().llmq_linear_dynamic_max_tokens(int(in_features)))


def _run_dynamic(fp8: bool, x, w, bias, w_scale, out_dtype, q_dump, scale_dump, acc_dump, what: str):
    _check(x.dtype in (torch.bfloat16, torch.float16), f"{what}: activations must be bf16 or fp16")
    M, N, K = _check_operands(x, w, what)
    _check(M <= dynamic_linear_max_tokens(K), f"{what}: at most {dynamic_linear_max_tokens(K)} tokens at K = {K}")
    _check(x.stride(0) % 8 == 0, f"{what}: the activation row stride must be a multiple of 8")
    _check(w_scale is None or (w_scale.dtype == torch.float32 and w_scale.numel() == N and w_scale.is_contiguous()
                               and w_scale.device == x.device), f"{what}: w_scale must hold one fp32 scale per channel")
    out = torch.empty((M, N), dtype=out_dtype, device=x.device)
    if M == 0 or N == 0:
        return out
    L = _abi.lib()
    fn = L.llmq_linear_fp8_dynamic if fp8 else L.llmq_linear_i8_dynamic
    st = fn(x.data_ptr(), _abi.dtype_code(x.dtype), x.stride(0), w.data_ptr(), w.stride(1), _abi.ptr(w_scale), _abi.ptr(bias),
            _abi.dtype_code(bias.dtype) if bias is not None else _abi.BF16, out.data_ptr(), _abi.dtype_code(out_dtype),
            out.stride(0), M, N, K, _abi.ptr(q_dump), _abi.ptr(scale_dump), _abi.ptr(acc_dump), _abi.stream_of(x))
    _abi.check(st, what)
    return out


@torch.no_grad()
def w8a8_int8_linear_dynamic_per_token(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, w_scale: torch.Tensor,
                                       *, _q_dump=None, _scale_dump=None, _acc_dump=None) -> torch.Tensor:
    """quantize_activation_per_token_absmax (linear_sq.py:55-65) + w8a8_int8_linear_bbf16_obf16_per_channel in one
    launch, for up to dynamic_linear_max_tokens(K) tokens; bit-identical to the two calls.  ``x``: bf16 / fp16 [M, K];
    ``weight``: int8 [K, N] view of an [N, K] row-major tensor; ``bias``: [N], its dtype is the output dtype."""
    what = "w8a8_int8_linear_dynamic_per_token"
    _check(weight.dtype == torch.int8, f"{what}: weight must be int8")
    _check(bias is not None, f"{what}: bias is required (pass zeros for a bias-free layer)")
    _check_bias(bias, weight, weight.size(1), (torch.bfloat16, torch.float16), what)
    return _run_dynamic(False, x, weight, bias, w_scale, bias.dtype, _q_dump, _scale_dump, _acc_dump, what)


@torch.no_grad()
def f8f8bf16_linear_dynamic_per_token(x: torch.Tensor, WQ: torch.Tensor, bias: Optional[torch.Tensor],
                                      w_scale: torch.Tensor, *, _q_dump=None, _scale_dump=None,
                                      _acc_dump=None) -> torch.Tensor:
    """per_token_quantize (linear_fp8.py:40-63) + cutlass_f8f8bf16_rowwise_sm89 in one launch, for up to
    dynamic_linear_max_tokens(K) tokens; bit-identical to the two calls.  Output bf16."""
    what = "f8f8bf16_linear_dynamic_per_token"
    _check(WQ.dtype == torch.float8_e4m3fn, f"{what}: WQ must be float8_e4m3fn")
    _check_bias(bias, WQ, WQ.size(1), (torch.bfloat16, torch.float32), what)
    return _run_dynamic(True, x, WQ, bias, w_scale, torch.bfloat16, _q_dump, _scale_dump, _acc_dump, what)
