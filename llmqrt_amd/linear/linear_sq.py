"""SmoothQuant W8A8 Linear modules (nn_models/modules/linear/linear_sq.py:69-214).

Buffer names, shapes and dtypes match the reference so its checkpoints load unchanged:
``qweight`` int8 [N, K], ``bias`` [N] (model dtype), ``weight_scale`` / ``input_scale``.
The forward pass is two HIP kernels (activation quantizer, int8 MFMA GEMM with fused
dequant epilogue) and no host synchronisation.
"""
from __future__ import annotations

import torch

from ..quantize import (quantize_activation_per_tensor_absmax, quantize_weight_per_channel_absmax,
                        quantize_activation_per_token_absmax,
                        quantize_activation_per_token_absmax_f32)
from ..sq_fp8_kernels import (dynamic_linear_max_tokens, w8a8_int8_linear_bbf16_obf16_per_channel,
                              w8a8_int8_linear_bbf16_obf16_per_tensor, w8a8_int8_linear_dynamic_per_token)
from .linear_base import LinearBase

__all__ = ["SqW8A8BBF16OBF16PerTensor", "SqW8A8BBF16OBF16PerChannel",
           "quantize_activation_per_tensor_absmax", "quantize_activation_per_token_absmax"]


# Up to this many tokens (and K < 8192) the one-launch linear is as fast on the GPU as quantizer + GEMM and saves a
# launch on the host; beyond, the two launches are faster (measured on MI355X at the Qwen2-7B shapes).
ONE_LAUNCH_MAX_TOKENS = 4


def _fusable(x2: torch.Tensor) -> bool:
    """Layout the one-launch linear takes: 16-bit activations, contiguous rows, K % 16 == 0, 16-byte aligned."""
    return (x2.is_cuda and x2.dtype in (torch.bfloat16, torch.float16) and x2.stride(-1) == 1 and x2.shape[-1] % 16 == 0
            and x2.shape[-1] < 8192
            and x2.stride(0) % 8 == 0 and x2.data_ptr() % 16 == 0)


class SqW8A8BBF16OBF16PerTensor(LinearBase):
    """Per-tensor weight scale, dynamic per-tensor activation scale (linear_sq.py:69-153)."""

    def __init__(self, w_bit, group_size, in_features, out_features, bias, dev="cuda:0", dtype=torch.float16,
                 weight_scale=1.0, input_scale=1.0, alpha=1.0, beta=1.0):
        super().__init__()
        self.w_bit = w_bit
        self.group_size = group_size
        self.in_features = in_features
        self.out_features = out_features
        self.dtype = dtype
        self.register_buffer("qweight", torch.randint(-127, 127, (out_features, in_features), dtype=torch.int8,
                                                      device=dev, requires_grad=False))
        if bias:
            self.register_buffer("bias", torch.zeros(out_features, dtype=dtype, device=dev, requires_grad=False))
        else:
            self.bias = None
        self.register_buffer("weight_scale", torch.tensor(weight_scale, device=dev))
        self.register_buffer("input_scale", torch.tensor(input_scale, device=dev))
        self._zero_bias = None

    def _bias_or_zeros(self, dtype, device):
        if self.bias is not None:
            return self.bias
        z = self._zero_bias
        if z is None or z.dtype != dtype or z.device != device:
            z = self._zero_bias = torch.zeros(self.out_features, dtype=dtype, device=device)
        return z

    @torch.no_grad()
    def forward(self, x):
        assert x.device == self.qweight.device, "when sq linear fwd, input and qweight must be same device!"
        assert self.weight_scale.device == self.qweight.device, "when sq linear fwd, scale and qweight must be same device!"
        assert self.input_scale.device == self.qweight.device, "when sq linear fwd, scale and qweight must be same device!"
        x_shape = x.shape
        x2 = x.reshape(-1, x_shape[-1])
        qx, input_scale = quantize_activation_per_tensor_absmax(x2)
        # alpha stays on the device: the product is rounded to the activation dtype as the
        # reference's `input_scale * weight_scale.item()` is, then read by the kernel
        alpha = (input_scale.float() * self.weight_scale.float()).to(input_scale.dtype)
        y = w8a8_int8_linear_bbf16_obf16_per_tensor(qx, self.qweight.t(), self._bias_or_zeros(x.dtype, x.device),
                                                    alpha, 1.0)
        return y.view(*x_shape[:-1], -1)

    @classmethod
    def from_linear(cls, module: torch.nn.Linear, w_bit, group_size, init_only=True, dtype=torch.float16,
                    per_tensor=True):
        sq_linear = cls(w_bit=w_bit, group_size=group_size, in_features=module.in_features,
                        out_features=module.out_features, bias=module.bias is not None,
                        dev=module.weight.device, dtype=dtype)
        if init_only:
            return sq_linear
        w = module.weight.data.float()
        scale = w.abs().max() / 127
        sq_linear.qweight = (w / scale).round().clamp(-128, 127).to(torch.int8)
        sq_linear.weight_scale = scale.to(sq_linear.weight_scale.dtype)
        if module.bias is not None:
            sq_linear.bias = module.bias.data.to(dtype)
        return sq_linear


class SqW8A8BBF16OBF16PerChannel(LinearBase):
    """Per-output-channel weight scales, dynamic per-token activation scales: the variant the
    reference sketches at linear_sq.py:155-214 (non-functional there).  ``weight_scale`` is fp32 [N]."""

    def __init__(self, w_bit, group_size, in_features, out_features, bias, dev="cuda:0", dtype=torch.float16):
        super().__init__()
        self.w_bit = w_bit
        self.group_size = group_size
        self.in_features = in_features
        self.out_features = out_features
        self.dtype = dtype
        self.register_buffer("qweight", torch.randint(-127, 127, (out_features, in_features), dtype=torch.int8,
                                                      device=dev, requires_grad=False))
        if bias:
            self.register_buffer("bias", torch.zeros(out_features, dtype=dtype, device=dev, requires_grad=False))
        else:
            self.bias = None
        self.register_buffer("weight_scale", torch.ones(out_features, dtype=torch.float32, device=dev))
        self._zero_bias = None

    _bias_or_zeros = SqW8A8BBF16OBF16PerTensor._bias_or_zeros

    @torch.no_grad()
    def forward(self, x):
        assert x.device == self.qweight.device, "when sq linear fwd, input and qweight must be same device!"
        assert self.weight_scale.device == self.qweight.device, "when sq linear fwd, scale and qweight must be same device!"
        x_shape = x.shape
        x2 = x.reshape(-1, x_shape[-1])
        if 0 < x2.shape[0] <= min(ONE_LAUNCH_MAX_TOKENS, dynamic_linear_max_tokens(x2.shape[-1])) and _fusable(x2):
            # a few tokens: quantizer and GEMM in one launch (same bits as the two calls below)
            y = w8a8_int8_linear_dynamic_per_token(x2, self.qweight.t(), self._bias_or_zeros(x.dtype, x.device),
                                                   self.weight_scale)
            return y.view(*x_shape[:-1], -1)
        qx, input_scale = quantize_activation_per_token_absmax_f32(x2)
        y = w8a8_int8_linear_bbf16_obf16_per_channel(qx, self.qweight.t(), self._bias_or_zeros(x.dtype, x.device),
                                                     input_scale, self.weight_scale)
        return y.view(*x_shape[:-1], -1)

    @torch.no_grad()
    def forward_quantized(self, qx, input_scale, out_dtype):
        """Same as forward for activations that are already quantized per token (int8 qx, fp32 scales
        [.., 1]), e.g. by the fused RMSNorm + quantizer kernel; no counterpart in the reference."""
        q2 = qx.reshape(-1, qx.shape[-1])
        y = w8a8_int8_linear_bbf16_obf16_per_channel(q2, self.qweight.t(), self._bias_or_zeros(out_dtype, qx.device),
                                                     input_scale.reshape(-1, 1), self.weight_scale)
        return y.view(*qx.shape[:-1], -1)

    @classmethod
    def from_linear(cls, module: torch.nn.Linear, w_bit, group_size, init_only=True, dtype=torch.float16,
                    per_tensor=False):
        sq_linear = cls(w_bit=w_bit, group_size=group_size, in_features=module.in_features,
                        out_features=module.out_features, bias=module.bias is not None,
                        dev=module.weight.device, dtype=dtype)
        if init_only:
            return sq_linear
        w = module.weight.data.float()
        if w.is_cuda:
            sq_linear.qweight, scale = quantize_weight_per_channel_absmax(w)   # utils/quantization_utils.py:27-38
            scale = scale.view(-1)
        else:  # a module assembled on the host: the same arithmetic in torch
            scale = w.abs().max(dim=1).values / 127
            sq_linear.qweight = (w / scale.view(-1, 1)).round().clamp(-128, 127).to(torch.int8)
        sq_linear.weight_scale = scale.float()
        if module.bias is not None:
            sq_linear.bias = module.bias.data.to(dtype)
        return sq_linear
