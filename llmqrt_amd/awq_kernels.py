"""HIP-backed drop-in for ``runtime.triton_kernels.awq_kernels`` (awq_kernels.py:273-378):
``awq_gemm_triton`` and ``awq_dequantize_triton`` keep their names and signatures; the block-size
and split-K arguments are accepted (and validated as the reference validates them) but the
gfx950 kernels choose their own tiling."""
from __future__ import annotations

import torch

from . import _abi

AWQ_TRITON_SUPPORTED_GROUP_SIZES = [-1, 32, 64, 128]


def _check_layout(qweight, scales, zeros, K, N, group_size):
    assert qweight.dtype == torch.int32 and zeros.dtype == torch.int32 and scales.dtype == torch.float16
    assert qweight.is_cuda and scales.device == qweight.device and zeros.device == qweight.device
    assert qweight.is_contiguous() and scales.is_contiguous() and zeros.is_contiguous()
    assert qweight.shape[0] == K and qweight.shape[1] == N // 8
    assert zeros.shape[0] == K // group_size and zeros.shape[1] == N // 8
    assert scales.shape[0] == K // group_size and scales.shape[1] == N
    assert group_size <= K
    assert group_size in AWQ_TRITON_SUPPORTED_GROUP_SIZES or group_size == K


@torch.no_grad()
def awq_dequantize_triton(qweight: torch.Tensor, scales: torch.Tensor, zeros: torch.Tensor,
                          block_size_x: int = 32, block_size_y: int = 32) -> torch.Tensor:
    """qweight [K, N/8] i32, scales [K/G, N] fp16, zeros [K/G, N/8] i32 -> fp16 [K, N]."""
    K = qweight.shape[0]
    N = scales.shape[1]
    group_size = qweight.shape[0] // scales.shape[0]
    assert K > 0 and N > 0
    _check_layout(qweight, scales, zeros, K, N, group_size)
    result = torch.empty(K, N, device=qweight.device, dtype=scales.dtype)
    _abi.check(_abi.lib().llmq_awq_dequant(qweight.data_ptr(), scales.data_ptr(), zeros.data_ptr(),
                                           result.data_ptr(), K, N, group_size, _abi.stream_of(qweight)),
               "llmq_awq_dequant")
    return result


@torch.no_grad()
def awq_dequantize_transposed(qweight: torch.Tensor, scales: torch.Tensor, zeros: torch.Tensor) -> torch.Tensor:
    """The same dequantized weights as awq_dequantize_triton, written as fp16 [N, K] (K contiguous): the weight operand
    of ``gemm_f16``.  No counterpart in the reference (its torch.matmul takes the [K, N] tensor)."""
    K = qweight.shape[0]
    N = scales.shape[1]
    group_size = qweight.shape[0] // scales.shape[0]
    assert K > 0 and N > 0 and group_size % 8 == 0
    _check_layout(qweight, scales, zeros, K, N, group_size)
    result = torch.empty(N, K, device=qweight.device, dtype=scales.dtype)
    _abi.check(_abi.lib().llmq_awq_dequant_t(qweight.data_ptr(), scales.data_ptr(), zeros.data_ptr(),
                                             result.data_ptr(), K, N, group_size, _abi.stream_of(qweight)),
               "llmq_awq_dequant_t")
    return result


@torch.no_grad()
def gemm_f16(x: torch.Tensor, w_nk: torch.Tensor, bias: torch.Tensor | None = None, *, _acc_dump=None) -> torch.Tensor:
    """x fp16 [M, K] times w_nk^T (fp16 [N, K]) -> fp16 [M, N], fp32 accumulation on the matrix cores (+ bias).
    Replaces the torch.matmul of the reference's many-token path (linear_awq.py:51-53)."""
    assert x.dtype == torch.float16 and w_nk.dtype == torch.float16 and x.dim() == 2 and w_nk.dim() == 2
    assert x.is_cuda and w_nk.device == x.device and x.shape[1] == w_nk.shape[1]
    M, K = x.shape
    N = w_nk.shape[0]
    assert K % 8 == 0
    if x.stride(1) != 1 or x.stride(0) % 8 or x.data_ptr() % 16:
        x = x.contiguous()
    if w_nk.stride(1) != 1 or w_nk.stride(0) % 8 or w_nk.data_ptr() % 16:
        w_nk = w_nk.contiguous()
    out = torch.empty((M, N), dtype=torch.float16, device=x.device)
    if M == 0 or N == 0:
        return out
    L = _abi.lib()
    ws = _abi.workspaces.get(x.device, L.llmq_gemm_f16_workspace_bytes(M, N, K))
    _abi.check(L.llmq_gemm_f16(x.data_ptr(), x.stride(0), w_nk.data_ptr(), w_nk.stride(0), 1.0, _abi.ptr(bias),
                               _abi.dtype_code(bias.dtype) if bias is not None else 0, 1.0, out.data_ptr(), _abi.F16, N,
                               M, N, K, _abi.ptr(_acc_dump), _abi.ptr(ws), ws.numel() if ws is not None else 0,
                               _abi.stream_of(x)), "llmq_gemm_f16")
    return out


@torch.no_grad()
def awq_gemm_triton(input: torch.Tensor, qweight: torch.Tensor, scales: torch.Tensor, qzeros: torch.Tensor,
                    split_k_iters: int, block_size_m: int = 32, block_size_n: int = 32,
                    block_size_k: int = 32, *, bias: torch.Tensor | None = None) -> torch.Tensor:
    """input fp16 [M, K] x dequant(qweight) -> fp16 [M, N] (fp32 accumulation, deterministic)."""
    M, K = input.shape
    N = qweight.shape[1] * 8
    group_size = qweight.shape[0] // qzeros.shape[0]
    assert N > 0 and K > 0 and M > 0
    assert split_k_iters & (split_k_iters - 1) == 0 and split_k_iters != 0
    assert split_k_iters <= 32
    _check_layout(qweight, scales, qzeros, K, N, group_size)
    assert input.dtype == torch.float16 and input.device == qweight.device
    x = input
    if x.stride(1) != 1 or x.stride(0) % 8 or x.data_ptr() % 16:
        x = x.contiguous()
    result = torch.empty((M, N), dtype=scales.dtype, device=input.device)
    L = _abi.lib()
    ws = _abi.awq_workspaces.get(x.device, L.llmq_awq_gemm_workspace_bytes(M, N, K))
    _abi.check(L.llmq_awq_gemm(x.data_ptr(), x.stride(0), qweight.data_ptr(), scales.data_ptr(), qzeros.data_ptr(),
                               _abi.ptr(bias), result.data_ptr(), M, N, K, group_size, _abi.ptr(ws),
                               ws.numel() if ws is not None else 0, _abi.stream_of(x)), "llmq_awq_gemm")
    return result
