"""GPU: fused q/k/v (and gate/up) modules give exactly the concatenation of the separate modules' outputs,
and that concatenation matches the oracle composition (quantizer -> exact GEMM -> epilogue) on the fused buffers."""
import pytest
import torch

from oracle import ref_math as R

pytestmark = pytest.mark.gpu
OUT_TOL = 1e-2


def _rel(got, ref):
    return ((got.float().cpu() - ref.float()).abs().max() / ref.float().abs().max()).item()

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
    got = fused(x)
    assert torch.equal(got, want)
    # oracle composition on the fused module's own buffers
    qx, sx = R.quantize_activation_per_token_absmax(x.cpu())
    acc = R.int8_gemm_exact(qx, fused.qweight.cpu())
    ref = R.w8a8_epilogue_per_token_per_channel(acc, sx, fused.weight_scale.cpu(), fused.bias.cpu(), torch.bfloat16)
    assert _rel(got, ref) <= OUT_TOL


def test_fuse_fp8_dynamic_per_channel(cuda):
    # bf16 only: the row-wise op returns bf16 and takes a bf16 / fp32 bias, as the reference's does
    # (csrc/fp8/sm89_fp8_rowwise_fbgemm.cu:286-287,560-566)
    dtype = torch.bfloat16
    from llmqrt_amd.fused_utils import fuse_linears
    from llmqrt_amd.linear import FP8DynamicLinear
    mods = [FP8DynamicLinear.from_linear(_dense(n, K, 20 + i).to(cuda), init_only=False, dtype=dtype,
                                         per_tensor=False) for i, n in enumerate(NS)]
    x = _x(33, dtype, cuda)
    want = torch.cat([m(x) for m in mods], dim=-1)
    fused = fuse_linears(mods)
    assert isinstance(fused, FP8DynamicLinear) and not fused.per_tensor and fused.dtype == dtype
    got = fused(x)
    assert torch.equal(got, want)
    xq, xs = R.fp8_per_token_quantize(x.cpu())
    acc = R.fp8_gemm_acc(xq.float(), fused.weight.data.cpu().float())
    ref = R.fp8_epilogue_rowwise(acc, xs, fused.weight_scale.data.cpu().view(-1), fused.bias.data.cpu(), torch.bfloat16)
    assert _rel(got, ref) <= OUT_TOL


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fp8_dynamic_per_tensor_modules_stay_unfused(cuda, dtype):
    """per_tensor=True modules quantize the activations per tensor and return the module dtype through the
    tensor-wise kernel; a fused per-channel module would change both, so they come back unfused - and each one
    still matches the oracle's per-tensor composition."""
    from llmqrt_amd.fused_utils import fuse_linears, fuse_qkv
    from llmqrt_amd.linear import FP8DynamicLinear
    mods = [FP8DynamicLinear.from_linear(_dense(n, K, 50 + i).to(cuda), init_only=False, dtype=dtype,
                                         per_tensor=True) for i, n in enumerate(NS)]
    assert all(m.per_tensor and m.weight_scale.shape == (1,) for m in mods)
    out = fuse_linears(mods)
    assert isinstance(out, list) and all(a is b for a, b in zip(out, mods))
    assert fuse_qkv(None, *mods) == tuple(mods)
    x = _x(33, dtype, cuda)
    xq, xs = R.fp8_per_tensor_quantize(x.cpu())
    for m in mods:
        y = m(x)
        assert y.dtype == dtype
        acc = R.fp8_gemm_acc(xq.float(), m.weight.data.cpu().float())
        alpha = float(m.weight_scale.data.cpu().float() * xs)
        ref = R.fp8_epilogue_tensorwise(acc, m.bias.data.cpu(), alpha, 1.0, dtype)
        assert _rel(y, ref) <= OUT_TOL


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
    got = fused(x)
    assert torch.equal(got, want)
    ref = R.awq_gemm(x.cpu().view(4, K), fused.qweight.cpu(), fused.qzeros.cpu(), fused.scales.cpu(), 128)
    ref = (ref.float() + fused.bias.cpu().float()).half()
    assert _rel(got.view(4, -1), ref) <= OUT_TOL


def test_static_activation_scales_are_left_unfused(cuda):
    from llmqrt_amd.fused_utils import fuse_qkv
    from llmqrt_amd.linear import FP8StaticLinear, SqW8A8BBF16OBF16PerTensor
    sq = [SqW8A8BBF16OBF16PerTensor(8, 0, K, n, True, dev=cuda, dtype=torch.bfloat16) for n in NS]
    assert fuse_qkv(None, *sq) == tuple(sq)
    st = [FP8StaticLinear(K, n, True, dev=cuda) for n in NS]
    assert fuse_qkv(None, *st) == tuple(st)
