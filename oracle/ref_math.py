"""CPU oracle for the quantized-linear hot path.  TEST INFRASTRUCTURE ONLY.

This module restates, with torch CPU ops, the arithmetic of the reference's
quantized-linear path.  Only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import it; the product package
``llmqrt_amd`` never does.  Every function cites the reference lines it follows
(paths relative to the reference checkout's ``runtime/`` directory).

Pins (what each function is checked against, all in ``tests/test_oracle_*.py``):

* int8 quantizers        - the scalar C restatement ``oracle/llmq_oracle.c`` (independent
                           bit-twiddled bf16/fp16 rounding), exhaustive over all bf16
                           patterns, closed-form special cases (zero row, arg-max -> +-127
                           in fp32 semantics, half-to-even ties).
* e4m3fn codec           - the 256-entry decode table built from the OCP format definition
                           (``tests/golden/e4m3fn_table.json``), encode->decode round trip,
                           tie/saturation cases.
* exact integer GEMM     - int64 triple loop in C on small shapes; known-answer vectors.
* scale epilogues        - linearity / all-ones invariants and the recipe of
                           ``unittest/test_sq_linear.py:8-34`` (atol 0.1).
* AWQ pack / unpack      - ``R[O[i]] == i``, pack->unpack identity over all nibble slots,
                           hand-built words in ``tests/golden/awq_kat.json``.
* AWQ fused GEMM (the Triton boundary ``awq_gemm_triton``): **parity unpinned** by the
  reference's own tests (it has none for AWQ, and the Triton kernel is fp16-accumulated with
  non-deterministic atomics); pinned here on the dequantize-then-matmul math the reference
  itself uses as its fallback (``nn_models/modules/linear/linear_awq.py:64-65``).
"""
from __future__ import annotations

import torch

AWQ_ORDER = (0, 2, 4, 6, 1, 3, 5, 7)          # utils/packing_utils.py:4, linear_awq.py:194
AWQ_REVERSE_ORDER = (0, 4, 1, 5, 2, 6, 3, 7)  # utils/packing_utils.py:5, awq_kernels.py:76-84
E4M3_MAX = 448.0                              # torch.finfo(torch.float8_e4m3fn).max


# --------------------------------------------------------------------------------------
# SmoothQuant int8 quantizers
# --------------------------------------------------------------------------------------
@torch.no_grad()
def quantize_activation_per_token_absmax(t: torch.Tensor):
    """nn_models/modules/linear/linear_sq.py:55-65.

    All arithmetic happens in ``t.dtype`` (bf16/fp16): the per-row absmax is clamped at
    1e-5 *rounded to t.dtype*, divided by 127 (result rounded to t.dtype), the quotient
    x/scale is rounded to t.dtype, then rounded half-to-even, clamped to [-128, 127] and
    narrowed to int8.  Returns (q int8 [.., K], scale t.dtype [.., 1]).
    """
    amax = t.abs().max(dim=-1, keepdim=True).values
    scale = amax.clamp(min=1e-5) / 127
    q = (t / scale).round().clamp(-128, 127).to(torch.int8)
    return q, scale


@torch.no_grad()
def quantize_activation_per_tensor_absmax(t: torch.Tensor):
    """nn_models/modules/linear/linear_sq.py:44-53: one global absmax, 0-dim scale."""
    scale = t.abs().max().clamp(min=1e-5) / 127
    q = (t / scale).round().clamp(-128, 127).to(torch.int8)
    return q, scale


@torch.no_grad()
def dynamic_quantize_activation_per_token_absmax(t: torch.Tensor):
    """utils/quantization_utils.py:65-71: as quantize_activation_per_token_absmax with the clamp at 1e-8
    (which is 0 in fp16).  The reference works in place on t (div_, round_, clamp_); this restatement returns the same
    (q, scale) without touching t."""
    max_val = t.abs().max(dim=-1, keepdim=True)[0]
    max_val = torch.clamp(max_val, min=1e-8) / 127
    q = (t / max_val).round().clamp(-128, 127).to(torch.int8)
    return q, max_val


@torch.no_grad()
def dynamic_quantize_activation_per_tensor_absmax(t: torch.Tensor):
    """utils/quantization_utils.py:57-62."""
    max_val = t.abs().max()
    max_val = torch.clamp(max_val, min=1e-8) / 127
    q = (t / max_val).round().clamp(-128, 127).to(torch.int8)
    return q, max_val


@torch.no_grad()
def quantize_weight_per_channel_absmax(w: torch.Tensor, native_dtype: bool = False):
    """utils/quantization_utils.py:27-38 (weights [N, K] -> int8 [N, K], scales [N, 1]).

    native_dtype=False: fp32 arithmetic (what a module built from fp32 master weights sees).  native_dtype=True: every
    tensor op in ``w.dtype``, as the reference's ops run on a GPU tensor (scale = absmax / 127 and w / scale each rounded
    to w.dtype, true division, no floor on the scale; the quotient is then rounded half-to-even and clamped)."""
    if not native_dtype:
        w = w.float()
    scale = (w.abs().max(dim=1).values / 127).view(-1, 1)
    q = (w / scale).round().clamp(-128, 127).to(torch.int8)
    return q, scale


# --------------------------------------------------------------------------------------
# W8A8 GEMM: exact accumulators + the two epilogues
# --------------------------------------------------------------------------------------
@torch.no_grad()
def int8_gemm_exact(qx: torch.Tensor, qw_nk: torch.Tensor) -> torch.Tensor:
    """acc[m, n] = sum_k qx[m, k] * qw[n, k] as int32 (csrc/smoothquant/sq_gemm.cu:67-76,
    A row-major [M,K], B column-major [K,N] == row-major [N,K]).

    fp64 BLAS is exact here: every partial sum is an integer below 2**53
    (|acc| <= K * 2**14 and K < 2**38).
    """
    acc = qx.double() @ qw_nk.double().t()
    return acc.to(torch.int64).to(torch.int32)


@torch.no_grad()
def w8a8_epilogue_per_tensor(acc, bias, alpha: float, beta: float, out_dtype):
    """D = out_dtype(alpha * float(acc) + beta * float(bias[n])): CUTLASS LinearCombination as
    instantiated at csrc/smoothquant/sq_gemm.cu:71-75,126-132 (C = bias broadcast over rows).
    The reference stores fp16 bits whatever the bias dtype (sq_gemm.cu:53 vs :112); this
    restatement rounds to the dtype the caller asked for."""
    y = acc.float() * torch.tensor(alpha, dtype=torch.float32)
    if bias is not None:
        y = y + torch.tensor(beta, dtype=torch.float32) * bias.float().view(1, -1)
    return y.to(out_dtype)


@torch.no_grad()
def w8a8_epilogue_per_token_per_channel(acc, a_scale, w_scale, bias, out_dtype):
    """Epilogue of the per-token x per-channel op declared at csrc/smoothquant/sq_gemm.h:19-24 (body absent in
    the reference).  Its semantics follow the reference's working per-token x per-channel op, the row-wise fp8
    GEMM: ((float(acc) * a_scale[m]) * w_scale[n]) + bias[n], every node rounded to fp32, one rounding to
    out_dtype at the end (the EVT tree at csrc/fp8/sm89_fp8_rowwise_fbgemm.cu:193-245).
    dequantize_activation_w_per_channel_a_per_token below is the torch helper with the other multiplication
    order; the two differ by at most one fp32 rounding before the final narrowing."""
    y = (acc.float() * a_scale.float().view(-1, 1)) * w_scale.float().view(1, -1)
    if bias is not None:
        y = y + bias.float().view(1, -1)
    return y.to(out_dtype)


@torch.no_grad()
def dequantize_activation_w_per_channel_a_per_token(q_act, w_scales, a_scales):
    """utils/quantization_utils.py:89-97, line by line: (float(acc) * w_scale[n]) * a_scale[m] -> a_scales.dtype."""
    dtype = a_scales.dtype
    q_act = q_act.to(torch.float32)
    q_act = q_act.mul(w_scales.reshape(1, -1)).mul(a_scales.reshape(-1, 1))
    return q_act.to(dtype)


@torch.no_grad()
def w8a8_linear_naive(qx, a_scale, qw_nk, w_scale, bias, out_dtype):
    """Dequantize-then-matmul ("naive impl", linear_sq.py:117-125): the CPU baseline."""
    y = (qx.float() * a_scale.float().view(-1, 1)) @ (qw_nk.float() * w_scale.float().view(-1, 1)).t()
    if bias is not None:
        y = y + bias.float().view(1, -1)
    return y.to(out_dtype)


# --------------------------------------------------------------------------------------
# FP8 (OCP e4m3fn)
# --------------------------------------------------------------------------------------
@torch.no_grad()
def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float):
    """RMSNorm.forward, nn_models/modules/nonlinear/norm.py:10-16, line by line.  -> (y in x.dtype, inv fp32 [.., 1]).

    The mean is whatever order torch's CPU reduction uses: `inv` is pinned only to a few fp32 ulps (see
    rmsnorm_given_inv for the part that is pinned bit for bit)."""
    h = x.to(torch.float32)
    variance = h.pow(2).mean(-1, keepdim=True)
    inv = torch.rsqrt(variance + eps)
    return weight * (h * inv).to(x.dtype), inv


def rmsnorm_given_inv(x: torch.Tensor, weight: torch.Tensor, inv: torch.Tensor) -> torch.Tensor:
    """Lines 14-16 of the same function with the reciprocal RMS supplied: y = weight * (fp32(x) * inv).to(dtype)."""
    return weight * (x.to(torch.float32) * inv.to(torch.float32).reshape(*x.shape[:-1], 1)).to(x.dtype)


def fp8_per_token_quantize(t: torch.Tensor):
    """nn_models/modules/linear/linear_fp8.py:40-63: scale = clamp(amax, 1e-12) / 448 in
    t.dtype, q = e4m3fn(clamp(t / scale, -448, 448)), scale returned as fp32 [.., 1]."""
    if t.numel() == 0:
        return (torch.empty_like(t, dtype=torch.float8_e4m3fn),
                torch.ones((*t.shape[:-1], 1), dtype=torch.float32))
    amax = t.abs().amax(dim=-1, keepdim=True)
    scale = amax.clamp(min=1e-12) / E4M3_MAX
    q = (t / scale).clamp(min=-E4M3_MAX, max=E4M3_MAX).to(torch.float8_e4m3fn)
    return q, scale.float()


@torch.no_grad()
def fp8_per_tensor_quantize(t: torch.Tensor):
    """linear_fp8.py:11-32 (global aminmax -> scalar scale; empty tensor -> amax 16)."""
    if t.numel() == 0:
        amax = torch.tensor(16.0, dtype=t.dtype)
    else:
        lo, hi = t.aminmax()
        amax = torch.maximum(lo.abs(), hi.abs())
    scale = amax.clamp(min=1e-12) / E4M3_MAX
    q = (t / scale).clamp(min=-E4M3_MAX, max=E4M3_MAX).to(torch.float8_e4m3fn)
    return q, scale.float()


@torch.no_grad()
def fp8_static_per_tensor_quantize(t: torch.Tensor, scale):
    """linear_fp8.py:34-37 (scale: fp32 1-element tensor or float; a fp32 tensor operand
    promotes the division to fp32, a Python float keeps it in t.dtype)."""
    return (t / scale).clamp(min=-E4M3_MAX, max=E4M3_MAX).to(torch.float8_e4m3fn)


@torch.no_grad()
def fp8_gemm_acc(xq: torch.Tensor, wq_nk: torch.Tensor) -> torch.Tensor:
    """fp64 accumulation of the decoded fp8 operands: the products are exact, so this is the
    mathematically exact accumulator the fp32 MFMA sum approximates."""
    return xq.double() @ wq_nk.double().t()


@torch.no_grad()
def fp8_epilogue_rowwise(acc, x_scale, w_scale, bias, out_dtype=torch.bfloat16):
    """((acc * x_scale[m]) * w_scale[n]) + bias[n] -> bf16, the EVT tree at
    csrc/fp8/sm89_fp8_rowwise_fbgemm.cu:193-245."""
    y = (acc.float() * x_scale.float().view(-1, 1)) * w_scale.float().view(1, -1)
    if bias is not None:
        y = y + bias.float().view(1, -1)
    return y.to(out_dtype)


@torch.no_grad()
def fp8_epilogue_tensorwise(acc, bias, alpha: float, beta: float, out_dtype):
    """alpha * acc + beta * bias[n] (csrc/fp8/sm89_fp8_tensorwise_cutlassgemm.cu:55-64,100-135)."""
    y = acc.float() * torch.tensor(alpha, dtype=torch.float32)
    if bias is not None:
        y = y + torch.tensor(beta, dtype=torch.float32) * bias.float().view(1, -1)
    return y.to(out_dtype)


@torch.no_grad()
def fp8_linear_naive(xq, x_scale, wq_nk, w_scale, bias, out_dtype=torch.bfloat16):
    """Dequantize-then-matmul (linear_fp8.py:97-101) in fp32: the CPU baseline."""
    y = (xq.float() * x_scale.float().view(-1, 1)) @ (wq_nk.float() * w_scale.float().view(-1, 1)).t()
    if bias is not None:
        y = y + bias.float().view(1, -1)
    return y.to(out_dtype)


# --------------------------------------------------------------------------------------
# AWQ W4A16
# --------------------------------------------------------------------------------------
@torch.no_grad()
def awq_pack(intw: torch.Tensor) -> torch.Tensor:
    """Pack uint4 values [R, C] (C % 8 == 0) into int32 [R, C/8]: nibble i of word c holds
    logical column 8c + AWQ_ORDER[i] (linear_awq.py:192-202, same for zeros :212-220)."""
    R, C = intw.shape
    v = intw.to(torch.int64).view(R, C // 8, 8)
    word = torch.zeros(R, C // 8, dtype=torch.int64)
    for i, o in enumerate(AWQ_ORDER):
        word |= (v[:, :, o] & 0xF) << (4 * i)
    word = torch.where(word >= 2 ** 31, word - 2 ** 32, word)
    return word.to(torch.int32)


@torch.no_grad()
def awq_unpack(packed: torch.Tensor) -> torch.Tensor:
    """int32 [R, C/8] -> uint4 values [R, C] in logical column order: logical column j of a
    word is nibble AWQ_REVERSE_ORDER[j] (utils/packing_utils.py:9-43)."""
    R, Cw = packed.shape
    w = packed.to(torch.int64) & 0xFFFFFFFF
    out = torch.empty(R, Cw, 8, dtype=torch.int32)
    for j, r in enumerate(AWQ_REVERSE_ORDER):
        out[:, :, j] = ((w >> (4 * r)) & 0xF).to(torch.int32)
    return out.view(R, Cw * 8)


@torch.no_grad()
def awq_dequantize(qweight, qzeros, scales, group_size: int) -> torch.Tensor:
    """fp16 W[k, n] = fp16(q[k, n] - z[k // G, n]) * s[k // G, n]  (utils/packing_utils.py:65-80;
    the difference is exact in fp16, the product is one fp16 RNE multiply)."""
    iw = awq_unpack(qweight)
    iz = awq_unpack(qzeros).repeat_interleave(group_size, dim=0)
    s = scales.repeat_interleave(group_size, dim=0)
    return (iw - iz).to(scales.dtype) * s


@torch.no_grad()
def awq_quantize_weight(w_nk: torch.Tensor, group_size: int):
    """Asymmetric uint4 group quantization of fp32 weights [N, K] along K, then the packer
    of linear_awq.py:133-222.  Returns (qweight [K, N/8] i32, qzeros [K/G, N/8] i32,
    scales [K/G, N] fp16)."""
    N, K = w_nk.shape
    G = group_size
    wg = w_nk.float().t().contiguous().view(K // G, G, N)
    mx, mn = wg.amax(dim=1), wg.amin(dim=1)
    s = ((mx - mn) / 15).clamp(min=1e-5).half()                      # [K/G, N]
    z = (-mn / s.float()).round().clamp(0, 15)                       # [K/G, N]
    q = ((wg / s.float().unsqueeze(1)).round() + z.unsqueeze(1)).clamp(0, 15)
    return awq_pack(q.view(K, N).to(torch.int32)), awq_pack(z.to(torch.int32)), s


@torch.no_grad()
def awq_gemm(x, qweight, qzeros, scales, group_size: int) -> torch.Tensor:
    """x @ dequantize(W) with fp32 accumulation, rounded to fp16 (linear_awq.py:64-65)."""
    w = awq_dequantize(qweight, qzeros, scales, group_size)
    return (x.float() @ w.float()).to(torch.float16)
