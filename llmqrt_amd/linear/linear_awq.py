"""AWQ W4A16 Linear module (nn_models/modules/linear/linear_awq.py:25-267): same buffers
(``qweight`` int32 [K, N/8], ``qzeros`` int32 [K/G, N/8], ``scales`` fp16 [K/G, N], ``bias`` fp16),
same two paths (fused decode GEMM, dequantize + matmul) with the switch point measured on MI355X."""
from __future__ import annotations

import torch

from ..awq_kernels import awq_dequantize_transposed, awq_dequantize_triton, awq_gemm_triton, gemm_f16
from .linear_base import LinearBase

AWQ_ORDER = (0, 2, 4, 6, 1, 3, 5, 7)


def _pack_rows(values: torch.Tensor, w_bit: int = 4) -> torch.Tensor:
    """uint4 [R, C] -> int32 [R, C/8]; nibble i of a word = column 8c + AWQ_ORDER[i] (linear_awq.py:192-202)."""
    pack_num = 32 // w_bit
    v = values.to(torch.int64).view(values.shape[0], -1, pack_num)
    word = torch.zeros(v.shape[:2], dtype=torch.int64, device=values.device)
    for i, o in enumerate(AWQ_ORDER):
        word |= (v[:, :, o] & 0xF) << (w_bit * i)
    return torch.where(word >= 2 ** 31, word - 2 ** 32, word).to(torch.int32)


# Set to False to keep every token count on the fused kernels (llmq_awq_gemm) instead of switching to dequantize +
# fp16 GEMM for long prompts.
USE_DEQUANT_MATMUL = True


def dequant_matmul_token_threshold(in_features: int, out_features: int = 0) -> int:
    """Token count from which dequantize (transposed, llmq_awq_dequant_t) + fp16 MFMA GEMM (llmq_gemm_f16) beats the
    fused kernels on MI355X.

    The reference switches to dequantize + torch.matmul at 1024 tokens (linear_awq.py:22,47).  Here both sides are
    this library's kernels; measured on the Qwen2-7B shapes (us, fused / dequantize + GEMM) the fused path (few-token
    kernel up to 64 tokens, tile kernel with in-loop dequantization above) is ahead up to ~256 tokens for qkv / o
    (K = 3584; o 31 / 33 at 256 tokens, 36 / 34 at 320), ~224 for down (K = 18944; 79 / 83 at 192, 92 / 90 at 256,
    122 / 102 at 320) and ~550 for gate_up (N = 37888, where the dequantizer's 63 us take longest to amortize:
    138 / 185 at 256 tokens, 222 / 237 at 512, 264 / 247 at 640).  Both paths are within 1e-2 (max relative) of
    dequantize-then-matmul in fp32."""
    if in_features > 8192:
        return 256
    return 576 if out_features > 8192 else 288


def awq_linear_forward(x, qweight, qzeros, scales, w_bit=4, group_size=128, bias=None, out_features=0):
    """WQLinearMMFunction.forward (linear_awq.py:25-74): x fp16 [.., K] -> fp16 [.., N] (3-D at least)."""
    out_shape = x.shape[:-1] + (out_features,)
    if x.shape[0] == 0:
        return torch.zeros(out_shape, dtype=x.dtype, device=x.device)
    tokens = x.numel() // x.shape[-1]
    if USE_DEQUANT_MATMUL and tokens >= dequant_matmul_token_threshold(x.shape[-1], out_features):
        if group_size % 8 == 0 and x.dtype == torch.float16:
            # dequantize (transposed, fp16 [N, K]) + this package's own fp16 MFMA GEMM: no vendor library on the path
            out = gemm_f16(x.reshape(-1, x.shape[-1]), awq_dequantize_transposed(qweight, scales, qzeros), bias)
        else:
            w = awq_dequantize_triton(qweight, scales, qzeros)
            out = torch.matmul(x, w.to(x.dtype))
            out = out + bias if bias is not None else out
    else:
        out = awq_gemm_triton(x.reshape(-1, x.shape[-1]), qweight, scales, qzeros, split_k_iters=8, bias=bias)
    out = out.reshape(out_shape)
    if len(out.shape) == 2:
        out = out.unsqueeze(0)
    return out


class WQLinear_GEMM(LinearBase):
    def __init__(self, w_bit, group_size, in_features, out_features, bias, dev, training=False):
        super().__init__()
        if w_bit not in [4]:
            raise NotImplementedError("Only 4-bit are supported for now.")
        self.in_features = in_features
        self.out_features = out_features
        self.w_bit = w_bit
        self.group_size = group_size if group_size != -1 else in_features
        self.training = training
        assert self.in_features % self.group_size == 0
        assert out_features % (32 // self.w_bit) == 0
        pack = 32 // self.w_bit
        self.register_buffer("qweight", torch.zeros((in_features, out_features // pack), dtype=torch.int32, device=dev))
        self.register_buffer("qzeros", torch.zeros((in_features // self.group_size, out_features // pack),
                                                   dtype=torch.int32, device=dev))
        self.register_buffer("scales", torch.zeros((in_features // self.group_size, out_features),
                                                   dtype=torch.float16, device=dev))
        if bias:
            self.register_buffer("bias", torch.zeros(out_features, dtype=torch.float16, device=dev))
        else:
            self.bias = None

    @classmethod
    def from_linear(cls, linear, w_bit, group_size, init_only=False, dtype=torch.bfloat16, scales=None, zeros=None,
                    per_tensor=False):
        awq_linear = cls(w_bit, group_size, linear.in_features, linear.out_features, linear.bias is not None,
                         linear.weight.device)
        if init_only:
            return awq_linear
        assert scales is not None and zeros is not None
        # scales, zeros: [K/G, N], the orientation the reference indexes (scale_zeros[idx // group_size] is a
        # row of N values; zeros are packed along dim 1): intw[k, n] = round((W[n, k] + z * s) / s)
        # (linear_awq.py:165-186)
        G = awq_linear.group_size
        want = (linear.in_features // G, linear.out_features)
        if tuple(scales.shape) != want or tuple(zeros.shape) != want:
            raise RuntimeError(f"from_linear: scales and zeros must be [in_features // group_size, out_features] = "
                               f"{list(want)}, got {list(scales.shape)} and {list(zeros.shape)}")
        awq_linear.scales = scales.clone().half()
        if linear.bias is not None:
            awq_linear.bias = linear.bias.clone().half()
        sz = zeros * scales                                # [K/G, N]
        w_kn = linear.weight.data.t()                      # [K, N]
        intw = torch.round((w_kn + sz.repeat_interleave(G, dim=0)) /
                           awq_linear.scales.repeat_interleave(G, dim=0)).to(torch.int32)
        awq_linear.qweight = _pack_rows(intw, w_bit)
        awq_linear.qzeros = _pack_rows(zeros.to(torch.int32), w_bit)
        return awq_linear

    def forward(self, x):
        assert x.device == self.qweight.device, "when awq linear fwd, input and qweight must be same device!"
        assert self.qzeros.device == self.qweight.device, "when awq linear fwd, qzeros and qweight must be same device!"
        assert self.scales.device == self.qweight.device, "when awq linear fwd, scales and qweight must be same device!"
        out_shape = x.shape[:-1] + (self.out_features,)
        if x.shape[0] == 0:
            return torch.zeros(out_shape, dtype=x.dtype, device=x.device)
        input_dtype = x.dtype
        if input_dtype != torch.float16:
            x = x.to(torch.float16)
        with torch.no_grad():
            out = awq_linear_forward(x, self.qweight, self.qzeros, self.scales, self.w_bit, self.group_size,
                                     self.bias, self.out_features)
        if input_dtype != torch.float16:
            out = out.to(dtype=input_dtype)
        return out.reshape(out_shape)

    def extra_repr(self) -> str:
        return "in_features={}, out_features={}, bias={}, w_bit={}, group_size={}".format(
            self.in_features, self.out_features, self.bias is not None, self.w_bit, self.group_size)
