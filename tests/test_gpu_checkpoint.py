"""GPU: a reference-format AWQ / SmoothQuant checkpoint loaded by name runs through the HIP kernels and
matches the oracle."""
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
