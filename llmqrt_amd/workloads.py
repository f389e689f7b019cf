"""Seeded synthetic inputs for the benchmark / parity configurations.

Everything is drawn with a CPU generator (so a CPU checker and the GPU see identical bits) and
moved to the requested device afterwards.  Shapes are the Qwen2-7B linear projections; the
activation distribution is N(0,1) with 1 % of the channels scaled x20 (the outlier channels
SmoothQuant is designed around); weights are 0.02 * N(0,1).
"""
from __future__ import annotations

import math

import torch

from .linear.linear_awq import _pack_rows

# name -> (K, N)
QWEN2_7B_PROJ = {
    "qkv": (3584, 4608),
    "o": (3584, 3584),
    "gate_up": (3584, 37888),
    "down": (18944, 3584),
}
CONFIG0_SHAPE = (16, 896, 4864)  # M, K, N: Qwen2-0.5B MLP up-proj

W8A8_M = (1, 16, 128, 2048, 8192)
FP8_M = (16, 512, 4096)
AWQ_M = (1, 4, 16, 64)


def seed_for(config: int, index: int) -> int:
    return 1000 * config + index


def _gen(seed: int) -> torch.Generator:
    return torch.Generator(device="cpu").manual_seed(seed)


def activations(M: int, K: int, seed: int, dtype=torch.bfloat16, outliers: bool = True, device="cpu"):
    g = _gen(seed)
    x = torch.randn(M, K, generator=g, dtype=torch.float32)
    if outliers:
        idx = torch.randperm(K, generator=g)[: math.ceil(0.01 * K)]
        x[:, idx] *= 20.0
    return x.to(dtype).to(device)


def dense_weights(N: int, K: int, seed: int) -> torch.Tensor:
    return 0.02 * torch.randn(N, K, generator=_gen(seed), dtype=torch.float32)


def int8_weights(N: int, K: int, seed: int, device="cpu"):
    """Per-output-channel symmetric int8: (qweight int8 [N, K], w_scale fp32 [N])."""
    w = dense_weights(N, K, seed)
    scale = w.abs().amax(dim=1) / 127
    q = (w / scale.view(-1, 1)).round_().clamp_(-128, 127).to(torch.int8)
    return q.to(device), scale.to(device)


def fp8_weights(N: int, K: int, seed: int, device="cpu"):
    """Per-output-channel e4m3fn: (qweight fp8 [N, K], w_scale fp32 [N])."""
    w = dense_weights(N, K, seed)
    scale = w.abs().amax(dim=1).clamp_(min=1e-12) / 448.0
    q = (w / scale.view(-1, 1)).clamp_(-448.0, 448.0).to(torch.float8_e4m3fn)
    return q.to(device), scale.to(device)


def awq_weights(N: int, K: int, seed: int, group: int = 128, device="cpu"):
    """Asymmetric uint4, groups of `group` along K, AWQ packing:
    (qweight int32 [K, N/8], qzeros int32 [K/G, N/8], scales fp16 [K/G, N])."""
    w = dense_weights(N, K, seed)
    wg = w.t().contiguous().view(K // group, group, N)
    mx, mn = wg.amax(dim=1), wg.amin(dim=1)
    s = ((mx - mn) / 15).clamp_(min=1e-5).half()
    sf = s.float()
    z = (-mn / sf).round_().clamp_(0, 15)
    q = (wg / sf.unsqueeze(1)).round_().add_(z.unsqueeze(1)).clamp_(0, 15)
    qweight = _pack_rows(q.view(K, N).to(torch.int32))
    qzeros = _pack_rows(z.to(torch.int32))
    return qweight.to(device), qzeros.to(device), s.to(device)


def smoothquant_factors(x_absmax: torch.Tensor, w_absmax: torch.Tensor, alpha: float = 0.5) -> torch.Tensor:
    """s_j = max|X_j|^alpha / max|W_j|^(1-alpha) per input channel j (SmoothQuant); activations are
    divided by s (folded into the preceding RMSNorm weight), weights multiplied by s."""
    return (x_absmax.clamp(min=1e-5).pow(alpha) / w_absmax.clamp(min=1e-5).pow(1 - alpha)).clamp(min=1e-5)


# ---- algorithmic work per linear (what the roofline figures are computed from) ---------------
def gemm_ops(M, N, K) -> int:
    return 2 * M * N * K


def w8a8_gemm_bytes(M, N, K) -> int:
    """int8 A + int8 B + bf16 out + fp32 scales."""
    return M * K + K * N + 2 * M * N + 4 * (M + N)


def quant_bytes(M, K) -> int:
    """bf16 in + 1-byte out + fp32 scale."""
    return 2 * M * K + M * K + 4 * M


def awq_gemm_bytes(M, N, K, group=128) -> int:
    return K * N // 2 + 2 * (K // group) * N + 4 * (K // group) * (N // 8) + 2 * M * K + 2 * M * N
