"""FP8 (OCP e4m3fn) Linear modules (nn_models/modules/linear/linear_fp8.py:134-313).

Parameter names/shapes/dtypes follow the reference (``weight`` is kept in the model dtype holding
fp8-representable values, ``weight_scale`` fp32 [1] or [N, 1], ``bias``, static: ``input_scale``,
``output_scale``).  Unlike the reference, the fp8 copy of the weight is made once and reused
until the parameter changes, instead of being re-cast on every forward.
"""
from __future__ import annotations

import torch

from ..quantize import per_tensor_quantize, per_token_quantize, static_per_tensor_quantize
from ..sq_fp8_kernels import (cutlass_f8f8bf16_rowwise_sm89, cutlass_f8f8bf16_tensorwise_sm89,
                              dynamic_linear_max_tokens, f8f8_tensorwise_quantized_output,
                              f8f8bf16_linear_dynamic_per_token)
from .linear_base import LinearBase
from .linear_sq import ONE_LAUNCH_MAX_TOKENS, _fusable

__all__ = ["FP8DynamicLinear", "FP8StaticLinear", "per_tensor_quantize", "per_token_quantize",
           "static_per_tensor_quantize"]

dtype_to_str = {torch.bfloat16: "bfloat16", torch.float16: "float16"}


class _FP8LinearBase(LinearBase):
    def _init_common(self, in_features, out_features, bias, dev, dtype, qdtype, per_channel_scale):
        self.dtype = dtype
        self.qdtype = qdtype
        self.in_features = in_features
        self.out_features = out_features
        self.weight = torch.nn.Parameter(torch.randn((out_features, in_features), dtype=dtype, device=dev),
                                         requires_grad=False)
        shape = (out_features, 1) if per_channel_scale else (1,)
        self.weight_scale = torch.nn.Parameter(torch.randn(shape, dtype=torch.float32, device=dev),
                                               requires_grad=False)
        if bias:
            self.bias = torch.nn.Parameter(torch.zeros(out_features, dtype=dtype, device=dev), requires_grad=False)
        else:
            self.bias = None
        self._q_cache = None
        self._s_cache = None

    def _wscale_flat(self):
        """The per-channel weight scales as a contiguous fp32 [N] vector, made once and kept like the fp8 weight."""
        s = self.weight_scale
        key = (id(s), s.data_ptr(), s._version, s.device)
        if self._s_cache is None or self._s_cache[0] != key:
            self._s_cache = (key, s.detach().to(torch.float32).reshape(-1).contiguous())
        return self._s_cache[1]

    def _qweight_t(self):
        """[K, N] column-major fp8 view of the weight.  The cast is made once and kept until the parameter is
        replaced, moved, re-versioned (an in-place op on the Parameter) or a state dict is loaded; a write
        through ``weight.data`` changes none of these and needs an explicit ``invalidate_cache()``."""
        w = self.weight
        key = (id(w), w.data_ptr(), w._version, w.device)
        if self._q_cache is None or self._q_cache[0] != key:
            self._q_cache = (key, w.detach().to(self.qdtype).contiguous())
        return self._q_cache[1].t()

    def invalidate_cache(self):
        """Drop the cached fp8 copy of the weight and the flat copy of its scales; the next forward makes them again."""
        self._q_cache = None
        self._s_cache = None

    def _load_from_state_dict(self, *args, **kwargs):
        self._q_cache = self._s_cache = None   # loaders fill parameters through .data.copy_(), which bumps no version
        return super()._load_from_state_dict(*args, **kwargs)

    def _apply(self, fn, *args, **kwargs):
        self._q_cache = self._s_cache = None   # .to() / .cuda() / .half() replace or rewrite the parameter storage
        return super()._apply(fn, *args, **kwargs)


class FP8DynamicLinear(_FP8LinearBase):
    def __init__(self, in_features, out_features, bias, dev="cuda:0", dtype=torch.bfloat16,
                 qdtype=torch.float8_e4m3fn, per_tensor=True):
        super().__init__()
        self.per_tensor = per_tensor
        self._init_common(in_features, out_features, bias, dev, dtype, qdtype, not per_tensor)

    @classmethod
    def from_linear(cls, module: torch.nn.Linear, w_bit=8, group_size=0, init_only=True, dtype=torch.bfloat16,
                    per_tensor=True):
        assert group_size == 0, "not support group wise fp8 quant yet! pls set group_size = 0"
        lin = cls(in_features=module.in_features, out_features=module.out_features,
                  bias=module.bias is not None, dev=module.weight.device, dtype=dtype, per_tensor=per_tensor)
        if init_only:
            return lin
        w = module.weight.data.float()
        amax = w.abs().amax() if per_tensor else w.abs().amax(dim=1, keepdim=True)
        scale = amax.clamp(min=1e-12) / 448.0
        lin.weight.data = (w / scale).clamp(-448, 448).to(torch.float8_e4m3fn).to(dtype)
        lin.weight_scale.data = scale.reshape(lin.weight_scale.shape).float()
        if module.bias is not None:
            lin.bias.data = module.bias.data.to(dtype)
        return lin

    @torch.no_grad()
    def forward(self, x):
        assert x.device == self.weight.device, "when fp8 linear fwd, input and qweight must be same device!"
        assert self.weight_scale.device == self.weight.device, "when fp8 linear fwd, scale and qweight must be same device!"
        x_shape = x.shape
        out_shape = x.shape[:-1] + (self.out_features,)
        if x.shape[0] == 0:
            return torch.zeros(out_shape, dtype=x.dtype, device=x.device)
        qweight = self._qweight_t()
        if self.per_tensor:
            qinput, x_scale = per_tensor_quantize(x)
            alpha = self.weight_scale * x_scale
            output = cutlass_f8f8bf16_tensorwise_sm89(qinput.view(-1, x_shape[-1]), qweight, self.bias, alpha, 1.0,
                                                      dtype_to_str.get(self.dtype))
        else:
            x2 = x.reshape(-1, x_shape[-1])
            if (self.qdtype == torch.float8_e4m3fn and _fusable(x2)
                    and x2.shape[0] <= min(ONE_LAUNCH_MAX_TOKENS, dynamic_linear_max_tokens(x2.shape[-1]))):
                # a few tokens: quantizer and GEMM in one launch (same bits as the two calls below)
                output = f8f8bf16_linear_dynamic_per_token(x2, qweight, self.bias, self._wscale_flat())
                return output.view(*x_shape[:-1], -1)
            qinput, x_scale = per_token_quantize(x)
            output = cutlass_f8f8bf16_rowwise_sm89(qinput.view(-1, x_shape[-1]), qweight, self.bias,
                                                   x_scale.view(-1, 1), self.weight_scale.to(torch.float32).t(), True)
        return output.view(*x_shape[:-1], -1)

    @torch.no_grad()
    def forward_quantized(self, qinput, x_scale):
        """Per-channel forward for activations already quantized per token (e4m3fn qinput, fp32 scales
        [.., 1]), e.g. by the fused RMSNorm + quantizer kernel; no counterpart in the reference."""
        assert not self.per_tensor, "pre-quantized activations carry per-token scales"
        output = cutlass_f8f8bf16_rowwise_sm89(qinput.reshape(-1, qinput.shape[-1]), self._qweight_t(), self.bias,
                                               x_scale.reshape(-1, 1), self.weight_scale.to(torch.float32).t(), True)
        return output.view(*qinput.shape[:-1], -1)


class FP8StaticLinear(_FP8LinearBase):
    def __init__(self, in_features, out_features, bias, dev="cuda:0", dtype=torch.bfloat16,
                 qdtype=torch.float8_e4m3fn, per_tensor=True, quantize_output=False):
        super().__init__()
        self.per_tensor = per_tensor
        self._init_common(in_features, out_features, bias, dev, dtype, qdtype, False)
        self.input_scale = torch.nn.Parameter(torch.randn((1,), dtype=torch.float32, device=dev), requires_grad=False)
        self.quantize_output = quantize_output
        self.output_scale = torch.nn.Parameter(torch.randn((1,), dtype=torch.float32, device=dev), requires_grad=False)

    @classmethod
    def from_linear(cls, module: torch.nn.Linear, w_bit=8, group_size=0, init_only=True, dtype=torch.bfloat16,
                    per_tensor=True, quantize_output=False):
        assert group_size == 0, "not support group wise fp8 quant yet! pls set group_size = 0"
        lin = cls(in_features=module.in_features, out_features=module.out_features,
                  bias=module.bias is not None, dev=module.weight.device, dtype=dtype, per_tensor=True,
                  quantize_output=quantize_output)
        if init_only:
            return lin
        w = module.weight.data.float()
        scale = w.abs().amax().clamp(min=1e-12) / 448.0
        lin.weight.data = (w / scale).clamp(-448, 448).to(torch.float8_e4m3fn).to(dtype)
        lin.weight_scale.data = scale.reshape(1).float()
        if module.bias is not None:
            lin.bias.data = module.bias.data.to(dtype)
        return lin

    @torch.no_grad()
    def forward(self, x):
        assert x.device == self.weight.device, "when fp8 linear fwd, input and qweight must be same device!"
        assert self.weight_scale.device == self.weight.device, "when fp8 linear fwd, scale and qweight must be same device!"
        x_shape = x.shape
        out_shape = x.shape[:-1] + (self.out_features,)
        if x.shape[0] == 0:
            return torch.zeros(out_shape, dtype=x.dtype, device=x.device)
        assert self.per_tensor, "[error!!] static activation quant only support per tensor!"
        qinput = static_per_tensor_quantize(x, self.input_scale)
        alpha = self.weight_scale * self.input_scale
        if self.quantize_output:
            # output / output_scale -> e4m3fn -> * output_scale (linear_fp8.py:309-311) inside the GEMM epilogue:
            # one launch, fp32 result as the reference's `qoutput.to(dtype) * output_scale`
            output = f8f8_tensorwise_quantized_output(qinput.view(-1, x_shape[-1]), self._qweight_t(), self.bias, alpha,
                                                      1.0, dtype_to_str.get(self.dtype), self.output_scale)
        else:
            output = cutlass_f8f8bf16_tensorwise_sm89(qinput.view(-1, x_shape[-1]), self._qweight_t(), self.bias, alpha,
                                                      1.0, dtype_to_str.get(self.dtype))
        return output.view(*x_shape[:-1], -1)
