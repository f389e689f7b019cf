"""GPU: reference-format AWQ, SmoothQuant and FP8 checkpoints loaded by name run through the HIP kernels and
match the oracle."""
import json

import pytest
import torch
from torch import nn

from oracle import ref_math as R

pytestmark = pytest.mark.gpu


class _Mlp(nn.Module):
    def __init__(self, d, h):
        super().__init__()
        self.up_proj, self.down_proj = nn.Linear(d, h, bias=False), nn.Linear(h, d, bias=False)


def test_awq_checkpoint_end_to_end(cuda, tmp_path):
    from safetensors.torch import save_file
    from llmqrt_amd import workloads as W
    from llmqrt_amd.checkpoint import QuantConfig, load_quantized_weights, replace_linears
    d, h = 256, 1024
    up = W.awq_weights(h, d, 61)
    down = W.awq_weights(d, h, 62)
    sd = {"up_proj.qweight": up[0], "up_proj.qzeros": up[1], "up_proj.scales": up[2],
          "down_proj.qweight": down[0], "down_proj.qzeros": down[1], "down_proj.scales": down[2]}
    save_file({k: v.contiguous() for k, v in sd.items()}, str(tmp_path / "model.safetensors"))
    (tmp_path / "config.json").write_text(json.dumps({"quantization_config": {
        "quant_method": "awq", "bits": 4, "group_size": 128, "zero_point": True, "modules_to_not_convert": None}}))
    cfg = QuantConfig.from_pretrained(str(tmp_path))
    model = _Mlp(d, h)
    assert replace_linears(model, cfg, dtype=torch.float16) == ["up_proj", "down_proj"]
    missing, unexpected = load_quantized_weights(model, str(tmp_path), device=cuda)
    assert missing == [] and unexpected == []
    x = W.activations(5, d, 63, dtype=torch.float16, outliers=False)
    y = model.down_proj(model.up_proj(x.to(cuda)))
    mid = R.awq_gemm(x, *up[:2], up[2], 128)
    ref = R.awq_gemm(mid, *down[:2], down[2], 128)
    rel = ((y.float().cpu() - ref.float()).abs().max() / ref.float().abs().max()).item()
    assert rel <= 1e-2


def _write_ckpt(tmp_path, sd, qcfg):
    from safetensors.torch import save_file
    save_file({k: v.contiguous() for k, v in sd.items()}, str(tmp_path / "model.safetensors"))
    (tmp_path / "config.json").write_text(json.dumps({"quantization_config": qcfg}))


def test_smoothquant_per_channel_checkpoint_end_to_end(cuda, tmp_path):
    """A SmoothQuant checkpoint in the reference's buffer naming (qweight int8 [N, K], weight_scale, no bias)
    loaded by name, run through quantizer + int8 GEMM, against the oracle composition."""
    from llmqrt_amd import workloads as W
    from llmqrt_amd.checkpoint import QuantConfig, load_quantized_weights, replace_linears
    from llmqrt_amd.linear import SqW8A8BBF16OBF16PerChannel
    d, h = 256, 1024
    up_q, up_s = W.int8_weights(h, d, 71)
    dn_q, dn_s = W.int8_weights(d, h, 72)
    _write_ckpt(tmp_path, {"up_proj.qweight": up_q, "up_proj.weight_scale": up_s,
                           "down_proj.qweight": dn_q, "down_proj.weight_scale": dn_s},
                {"quant_method": "sq", "bits": 8, "group_size": 0, "per_tensor": False, "modules_to_not_convert": None})
    cfg = QuantConfig.from_pretrained(str(tmp_path))
    model = _Mlp(d, h)
    replace_linears(model, cfg, dtype=torch.bfloat16)
    assert isinstance(model.up_proj, SqW8A8BBF16OBF16PerChannel)
    missing, unexpected = load_quantized_weights(model, str(tmp_path), device=cuda)
    assert missing == [] and unexpected == []
    x = W.activations(7, d, 73)
    mid = model.up_proj(x.to(cuda))
    y = model.down_proj(mid)

    def oracle(inp, q, s):
        qx, sx = R.quantize_activation_per_token_absmax(inp)
        return R.w8a8_epilogue_per_token_per_channel(R.int8_gemm_exact(qx, q), sx, s, None, torch.bfloat16)
    mid_ref = oracle(x, up_q, up_s)
    assert ((mid.float().cpu() - mid_ref.float()).abs().max() / mid_ref.float().abs().max()) <= 1e-2
    # second stage on the GPU's own intermediate, so that the check does not compound two tolerances
    ref = oracle(mid.cpu(), dn_q, dn_s)
    assert ((y.float().cpu() - ref.float()).abs().max() / ref.float().abs().max()) <= 1e-2


def test_fp8_checkpoint_casts_once_and_follows_reloads(cuda, tmp_path):
    """An FP8 checkpoint stores fp8-representable values in bf16 (`weight`) plus `weight_scale`.  The module casts
    the weight to fp8 once (same cached tensor on the second forward), matches the oracle, and a second
    checkpoint loaded over the same module changes the result (the cached cast is dropped by the loader and by
    load_state_dict; a raw write through .data needs invalidate_cache())."""
    from llmqrt_amd import workloads as W
    from llmqrt_amd.checkpoint import QuantConfig, load_quantized_weights, replace_linears
    from llmqrt_amd.linear import FP8DynamicLinear
    d, h = 256, 512

    class _One(nn.Module):
        def __init__(self):
            super().__init__()
            self.up_proj = nn.Linear(d, h, bias=False)

    def ckpt(seed, path):
        q, s = W.fp8_weights(h, d, seed)
        path.mkdir()
        _write_ckpt(path, {"up_proj.weight": q.to(torch.bfloat16), "up_proj.weight_scale": s.view(-1, 1)},
                    {"quant_method": "fp8_dynamic_quant", "bits": 8, "group_size": 0, "per_tensor": False,
                     "modules_to_not_convert": None})
        return q, s
    q1, s1 = ckpt(81, tmp_path / "a")
    q2, s2 = ckpt(82, tmp_path / "b")
    model = _One()
    replace_linears(model, QuantConfig.from_pretrained(str(tmp_path / "a")), dtype=torch.bfloat16)
    lin = model.up_proj
    assert isinstance(lin, FP8DynamicLinear) and not lin.per_tensor
    load_quantized_weights(model, str(tmp_path / "a"), device=cuda)
    x = W.activations(9, d, 83)

    def oracle(q, s):
        xq, xs = R.fp8_per_token_quantize(x)
        return R.fp8_epilogue_rowwise(R.fp8_gemm_acc(xq, q), xs, s, None)

    def rel(y, ref):
        return ((y.float().cpu() - ref.float()).abs().max() / ref.float().abs().max()).item()
    y1 = lin(x.to(cuda))
    cached = lin._q_cache[1]
    assert cached.dtype == torch.float8_e4m3fn and torch.equal(cached.cpu().view(torch.uint8), q1.view(torch.uint8))
    y1b = lin(x.to(cuda))
    assert lin._q_cache[1] is cached and torch.equal(y1, y1b)          # cast once
    assert rel(y1, oracle(q1, s1)) <= 1e-2
    # reload other weights into the same module through the loader
    load_quantized_weights(model, str(tmp_path / "b"), device=cuda)
    y2 = lin(x.to(cuda))
    assert rel(y2, oracle(q2, s2)) <= 1e-2 and not torch.equal(y1, y2)
    # ... through load_state_dict
    sd = {"up_proj.weight": q1.to(torch.bfloat16).to(cuda), "up_proj.weight_scale": s1.view(-1, 1).to(cuda)}
    model.load_state_dict(sd)
    assert rel(lin(x.to(cuda)), oracle(q1, s1)) <= 1e-2
    # ... and a raw .data write, which nothing can observe: explicit invalidation
    lin.weight.data.copy_(q2.to(torch.bfloat16))
    lin.weight_scale.data.copy_(s2.view(-1, 1))
    lin.invalidate_cache()
    assert rel(lin(x.to(cuda)), oracle(q2, s2)) <= 1e-2
