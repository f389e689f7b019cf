"""Host logic of the checkpoint loader: QuantConfig parsing, module replacement, filling buffers by name from
safetensors files written in the reference's buffer naming.  CPU only (no kernels run)."""
import json

import pytest
import torch
from torch import nn


class _Attn(nn.Module):
    def __init__(self, d):
        super().__init__()
        self.q_proj, self.k_proj, self.v_proj = nn.Linear(d, d), nn.Linear(d, d // 4), nn.Linear(d, d // 4)
        self.o_proj = nn.Linear(d, d, bias=False)


class _Tiny(nn.Module):
    def __init__(self, d=256, layers=2):
        super().__init__()
        self.layers = nn.ModuleList([nn.ModuleDict({"self_attn": _Attn(d)}) for _ in range(layers)])
        self.lm_head = nn.Linear(d, 64, bias=False)


def test_quant_config_round_trip(tmp_path):
    from llmqrt_amd.checkpoint import QuantConfig
    cfg = QuantConfig.from_dict({"quant_method": "awq", "q_group_size": 128, "w_bit": 4, "version": "GEMM",
                                 "zero_point": True})
    assert cfg.version == "gemm" and cfg.modules_to_not_convert == ["lm_head"] and cfg.per_tensor is True
    (tmp_path / "config.json").write_text(json.dumps({"hidden_size": 256,
                                                      "quantization_config": cfg.to_transformers_dict()}))
    back = QuantConfig.from_pretrained(str(tmp_path))
    assert (back.quant_method, back.q_group_size, back.w_bit, back.zero_point) == ("awq", 128, 4, True)
    (tmp_path / "config.json").write_text(json.dumps({"hidden_size": 256}))
    assert QuantConfig.from_pretrained(str(tmp_path)) == QuantConfig()
    with pytest.raises(FileNotFoundError):
        QuantConfig.from_pretrained(str(tmp_path / "nowhere"))


@pytest.mark.parametrize("method,per_tensor,cls_name,names", [
    ("awq", True, "WQLinear_GEMM", {"qweight", "qzeros", "scales", "bias"}),
    ("sq", True, "SqW8A8BBF16OBF16PerTensor", {"qweight", "bias", "weight_scale", "input_scale"}),
    ("sq", False, "SqW8A8BBF16OBF16PerChannel", {"qweight", "bias", "weight_scale"}),
    ("fp8_dynamic_quant", False, "FP8DynamicLinear", {"weight", "weight_scale", "bias"}),
    ("fp8_static_quant", True, "FP8StaticLinear", {"weight", "weight_scale", "bias", "input_scale"}),
])
def test_replace_and_load_by_name(tmp_path, method, per_tensor, cls_name, names):
    from safetensors.torch import save_file
    from llmqrt_amd.checkpoint import QuantConfig, load_quantized_weights, named_quantized_linears, replace_linears
    cfg = QuantConfig(quant_method=method, q_group_size=128 if method == "awq" else 0, w_bit=4 if method == "awq" else 8,
                      per_tensor=per_tensor)
    model = _Tiny()
    replaced = replace_linears(model, cfg, dtype=torch.bfloat16)
    assert len(replaced) == 8 and "lm_head" not in replaced and isinstance(model.lm_head, nn.Linear)
    q = model.layers[1]["self_attn"].q_proj
    assert type(q).__name__ == cls_name
    own = {n.split(".")[-1] for n, _ in list(q.named_buffers()) + list(q.named_parameters())}
    assert names <= own, own
    # a checkpoint in the reference's naming: random contents of the right shape/dtype, split over two files
    g = torch.Generator().manual_seed(5)
    sd = {}
    for n, t in list(model.named_buffers()) + list(model.named_parameters()):
        if t.dtype in (torch.int8, torch.int32):
            sd[n] = torch.randint(-100, 100, t.shape, generator=g).to(t.dtype)
        else:
            sd[n] = torch.randn(t.shape, generator=g).to(t.dtype)
    keys = sorted(sd)
    save_file({k: sd[k].contiguous() for k in keys[::2]}, str(tmp_path / "model-00001-of-00002.safetensors"))
    save_file({k: sd[k].contiguous() for k in keys[1::2]} | {"rotary.inv_freq": torch.ones(4)},
              str(tmp_path / "model-00002-of-00002.safetensors"))
    missing, unexpected = load_quantized_weights(model, str(tmp_path))
    assert missing == [] and unexpected == ["rotary.inv_freq"]
    now = dict(model.named_buffers()) | dict(model.named_parameters())
    assert all(torch.equal(now[k], sd[k]) for k in keys)
    assert len(list(named_quantized_linears(model))) == 8


def test_load_rejects_wrong_shapes(tmp_path):
    from safetensors.torch import save_file
    from llmqrt_amd.checkpoint import QuantConfig, load_quantized_weights, replace_linears
    model = _Tiny(layers=1)
    replace_linears(model, QuantConfig(quant_method="awq", q_group_size=128, w_bit=4))
    save_file({"layers.0.self_attn.q_proj.qweight": torch.zeros(256, 8, dtype=torch.int32)}, str(tmp_path / "m.safetensors"))
    with pytest.raises(RuntimeError, match="shape"):
        load_quantized_weights(model, str(tmp_path / "m.safetensors"))
    save_file({"layers.0.self_attn.q_proj.qweight": torch.zeros(256, 32)}, str(tmp_path / "m.safetensors"))
    with pytest.raises(RuntimeError, match="dtype"):
        load_quantized_weights(model, str(tmp_path / "m.safetensors"))
