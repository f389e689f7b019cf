"""GPU: fused q/k/v (and gate/up) modules give exactly the concatenation of the separate modules' outputs."""
import pytest
import torch

pytestmark = pytest.mark.gpu

K, NS = 896, (896, 128, 128)   # Qwen2-0.5B-like q / k / v widths


def _dense(n, k, seed):
    lin = torch.nn.Linear(k, n, bias=True)
    g = torch.Generator().manual_seed(seed)
    lin.weight.data = 0.02 * torch.randn(n, k, generator=g)
    lin.bias.data = 0.1 * torch.randn(n, generator=g)
    return lin


def _x(M, dtype, cuda):
    from llmqrt_amd import workloads as W
    return W.activations(M, K, 4242, dtype=dtype).to(cuda)


@pytest.mark.parametrize("M", [1, 16, 300])
def test_fuse_sq_per_channel(cuda, M):
    from llmqrt_amd.fused_utils import fuse_qkv
    from llmqrt_amd.linear import SqW8A8BBF16OBF16PerChannel
    mods = [SqW8A8BBF16OBF16PerChannel.from_linear(_dense(n, K, 10 + i).to(cuda), 8, 0, init_only=False,
                                                   dtype=torch.bfloat16) for i, n in enumerate(NS)]
    x = _x(M, torch.bfloat16, cuda)
    want = torch.cat([m(x) for m in mods], dim=-1)
    fused = fuse_qkv(None, *mods)
    assert isinstance(fused, SqW8A8BBF16OBF16PerChannel) and fused.out_features == sum(NS)
    assert torch.equal(fused(x), want)


@pytest.mark.parametrize("per_tensor", [True, False])
def test_fuse_fp8_dynamic(cuda, per_tensor):
    from llmqrt_amd.fused_utils import fuse_linears
    from llmqrt_amd.linear import FP8DynamicLinear
    mods = [FP8DynamicLinear.from_linear(_dense(n, K, 20 + i).to(cuda), init_only=False, dtype=torch.bfloat16,
                                         per_tensor=False) for i, n in enumerate(NS)]
    x = _x(33, torch.bfloat16, cuda)
    want = torch.cat([m(x) for m in mods], dim=-1)
    if per_tensor:
        # per-tensor weight scales, evaluated through the row-wise op so that the activation scales are
        # the same per-token ones the fused module uses
        for m in mods:
            m.weight_scale.data = m.weight_scale.data.max().reshape(1, 1).expand(m.out_features, 1).contiguous()
        want = torch.cat([m(x) for m in mods], dim=-1)
    fused = fuse_linears(mods)
    assert isinstance(fused, FP8DynamicLinear) and not fused.per_tensor
    assert torch.equal(fused(x), want)


def test_fuse_awq(cuda):
    from llmqrt_amd import workloads as W
    from llmqrt_amd.fused_utils import fuse_qkv
    from llmqrt_amd.linear import WQLinear_GEMM
    mods = []
    for i, n in enumerate(NS):
        qw, qz, sc = W.awq_weights(n, K, 30 + i)
        m = WQLinear_GEMM(4, 128, K, n, True, cuda)
        m.qweight, m.qzeros, m.scales = qw.to(cuda), qz.to(cuda), sc.to(cuda)
        m.bias = (0.1 * torch.randn(n, generator=torch.Generator().manual_seed(40 + i))).half().to(cuda)
        mods.append(m)
    x = _x(4, torch.float16, cuda).view(1, 4, K)
    want = torch.cat([m(x) for m in mods], dim=-1)
    fused = fuse_qkv(None, *mods)
    assert isinstance(fused, WQLinear_GEMM) and fused.qweight.shape == (K, sum(NS) // 8)
    assert torch.equal(fused(x), want)


def test_static_activation_scales_are_left_unfused(cuda):
    from llmqrt_amd.fused_utils import fuse_qkv
    from llmqrt_amd.linear import FP8StaticLinear, SqW8A8BBF16OBF16PerTensor
    sq = [SqW8A8BBF16OBF16PerTensor(8, 0, K, n, True, dev=cuda, dtype=torch.bfloat16) for n in NS]
    assert fuse_qkv(None, *sq) == tuple(sq)
    st = [FP8StaticLinear(K, n, True, dev=cuda) for n in NS]
    assert fuse_qkv(None, *st) == tuple(st)
