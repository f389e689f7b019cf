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


LAYER_M = (2048, 32)          # prefill tokens, decode batch
LAYER_NORM_EPS = 1e-6
# the two projections that read the output of an RMSNorm (input_layernorm -> qkv, post_attention_layernorm
# -> gate_up); o and down read the attention / activation-function output, whose smoothing factors live in
# the weights of the producer (v_proj, up_proj) and so arrive already divided
LAYER_NORMED = ("qkv", "gate_up")


def smoothquant_layer(alpha: float = 0.5, calib_tokens: int = 256, dtype=torch.bfloat16):
    """One Qwen2-7B-shaped decoder layer's linears in SmoothQuant W8A8 form (all tensors on the CPU).

    Per projection: dense fp32 weights W [N, K]; a seeded calibration batch gives max|X_j|; s from
    smoothquant_factors; the int8 weights are the per-channel quantization of W * s; for the projections
    behind an RMSNorm the norm weight g is stored both plain and folded (g / s, rounded to `dtype`), so that
    norm_folded(x) = norm(x) / s feeds the quantizer directly.
    -> {name: {K, N, w (fp32), s, qweight, w_scale, norm_weight, norm_weight_folded}}"""
    layer = {}
    for pi, (pname, (K, N)) in enumerate(QWEN2_7B_PROJ.items()):
        w = dense_weights(N, K, seed_for(4, 100 + pi))
        calib = activations(calib_tokens, K, seed_for(4, 200 + pi)).float()
        g = gf = None
        if pname in LAYER_NORMED:
            g = (1.0 + 0.1 * torch.randn(K, generator=_gen(seed_for(4, 300 + pi)))).to(dtype)
            inv = torch.rsqrt(calib.pow(2).mean(-1, keepdim=True) + LAYER_NORM_EPS)
            calib = g.float() * (calib * inv)
        s = smoothquant_factors(calib.abs().amax(0), w.abs().amax(0), alpha)
        if g is not None:
            gf = (g.float() / s).to(dtype)
        ws = w * s.view(1, -1)
        scale = ws.abs().amax(dim=1) / 127
        qw = (ws / scale.view(-1, 1)).round_().clamp_(-128, 127).to(torch.int8)
        layer[pname] = {"K": K, "N": N, "w": w, "s": s, "qweight": qw, "w_scale": scale,
                        "norm_weight": g, "norm_weight_folded": gf}
    return layer


def layer_input(pname: str, M: int, s: torch.Tensor, dtype=torch.bfloat16) -> torch.Tensor:
    """Input of projection `pname` of the layer stack for M tokens: the residual stream (in front of the
    RMSNorm) for qkv / gate_up, the producer's output already divided by s for o / down."""
    pi = list(QWEN2_7B_PROJ).index(pname)
    K = QWEN2_7B_PROJ[pname][0]
    x = activations(M, K, seed_for(4, 10 * pi + (0 if M > 64 else 1)), dtype=torch.float32)
    if pname not in LAYER_NORMED:
        x = x / s.view(1, -1)
    return x.to(dtype)


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
