"""CPU: the SmoothQuant smoothing used by the decoder-layer stack (the decoder-layer workload of the benchmark contract).

The smoothing formula is not in the reference repository (it ships pre-smoothed checkpoints); it is pinned
here by what the mathematics fixes: the identity (X / s)(s W)^T = X W^T, the balance point
max|X_j / s_j| = max|W_j s_j| = sqrt(max|X_j| max|W_j|) at alpha = 0.5, and the two limits alpha = 0 / 1."""
import torch

from llmqrt_amd import workloads as W


def _xw(seed, M=64, K=96, N=40):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g, dtype=torch.float64)
    x[:, ::17] *= 20
    w = 0.02 * torch.randn(N, K, generator=g, dtype=torch.float64)
    return x, w


def test_smoothing_is_an_identity_on_the_product():
    x, w = _xw(1)
    s = W.smoothquant_factors(x.abs().amax(0), w.abs().amax(0), 0.5)
    y0 = x @ w.t()
    y1 = (x / s) @ (w * s).t()
    assert (y0 - y1).abs().max() <= 1e-12 * y0.abs().max()


def test_alpha_half_balances_activation_and_weight_ranges():
    x, w = _xw(2)
    ax, aw = x.abs().amax(0), w.abs().amax(0)
    s = W.smoothquant_factors(ax, aw, 0.5)
    assert torch.allclose(ax / s, aw * s, rtol=1e-12)
    assert torch.allclose(ax / s, (ax * aw).sqrt(), rtol=1e-12)


def test_alpha_limits():
    x, w = _xw(3)
    ax, aw = x.abs().amax(0), w.abs().amax(0)
    # alpha = 1: all the range moves into the weights (activations end with unit range);
    # alpha = 0: the weights end with unit range
    assert torch.allclose(ax / W.smoothquant_factors(ax, aw, 1.0), torch.ones_like(ax), rtol=1e-12)
    assert torch.allclose(aw * W.smoothquant_factors(ax, aw, 0.0), torch.ones_like(aw), rtol=1e-12)


def test_layer_builder_folds_the_factors_into_norm_weight_and_weights():
    small = dict(W.QWEN2_7B_PROJ)
    try:
        W.QWEN2_7B_PROJ.clear()
        W.QWEN2_7B_PROJ.update({"qkv": (128, 96), "o": (128, 64), "gate_up": (128, 160), "down": (256, 128)})
        layer = W.smoothquant_layer(alpha=0.5, calib_tokens=32)
    finally:
        W.QWEN2_7B_PROJ.clear()
        W.QWEN2_7B_PROJ.update(small)
    for name, p in layer.items():
        normed = name in W.LAYER_NORMED
        assert (p["norm_weight_folded"] is not None) == normed
        if normed:
            want = (p["norm_weight"].float() / p["s"]).bfloat16()
            assert torch.equal(p["norm_weight_folded"], want)
        # int8 weights dequantize back to W * s within half a step per channel
        deq = p["qweight"].float() * p["w_scale"].view(-1, 1)
        assert ((deq - p["w"] * p["s"].view(1, -1)).abs() <= 0.5 * p["w_scale"].view(-1, 1) * (1 + 1e-5)).all()
        assert p["qweight"].abs().max() <= 127
