"""GPU parity: RMSNorm and RMSNorm fused with the per-token quantizers vs the CPU oracle.

The reciprocal RMS depends on the fp32 summation order, so it is compared within a few fp32 ulps; every
other output is compared BIT-EXACTLY against the oracle evaluated with the kernel's own reciprocal RMS,
and end to end against the oracle's own within one rounding step on a vanishing fraction of elements."""
import pytest
import torch

from oracle import ref_math as R

pytestmark = pytest.mark.gpu

INV_RTOL = 5e-7  # ~4 ulp of fp32: summation order + one sqrt + one division
# (258, 896) .. (257, 520) take the wavefront-per-row kernels (256 rows or more of at most 1024 elements), the last three
# the half-size blocks with four chunks per thread (256 rows or more of 2056 .. 4096 elements)
SHAPES = [(1, 896), (16, 896), (7, 3584), (128, 3584), (33, 18944), (3, 8), (5, 24576), (2, 40960),
          (258, 896), (1027, 1024), (300, 8), (257, 520), (300, 3584), (257, 2056), (256, 4096)]


def _inputs(M, K, dtype, seed):
    from llmqrt_amd import workloads as W
    x = W.activations(M, K, seed, dtype=dtype)
    if M > 2:
        x[2] = 0  # all-zero row: inv = 1/sqrt(eps), y = 0, quantizer floor scale
    g = torch.Generator().manual_seed(seed + 1)
    w = (1.0 + 0.2 * torch.randn(K, generator=g)).to(dtype)
    return x, w


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,K", SHAPES)
def test_rmsnorm(cuda, M, K, dtype):
    from llmqrt_amd.norm import rmsnorm
    x, w = _inputs(M, K, dtype, 5 * M + K)
    eps = 1e-6
    inv = torch.empty(M, dtype=torch.float32, device=cuda)
    y = rmsnorm(x.to(cuda), w.to(cuda), eps, _inv_dump=inv)
    y_ref, inv_ref = R.rmsnorm(x, w, eps)
    assert y.dtype == dtype and y.shape == x.shape
    assert torch.allclose(inv.cpu(), inv_ref.view(-1), rtol=INV_RTOL, atol=0)
    assert torch.equal(y.cpu().view(torch.int16), R.rmsnorm_given_inv(x, w, inv.cpu()).view(torch.int16))
    # end to end: a different last bit of inv can move x * inv across a rounding boundary, rarely; one step
    # of the normalised value (up to 2^-7 relative for bf16) then passes through the product with weight
    diff = (y.cpu().float() - y_ref.float()).abs()
    ulp = 2.0 ** (-6 if dtype == torch.bfloat16 else -9)
    assert (diff <= ulp * y_ref.float().abs() + 1e-30).all()
    assert (diff > 0).float().mean() < 2e-3


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,K", SHAPES)
def test_rmsnorm_int8_fused(cuda, M, K, dtype):
    from llmqrt_amd.norm import rmsnorm_quantize_activation_per_token_absmax as fused
    x, w = _inputs(M, K, dtype, 7 * M + K)
    eps = 1e-6
    inv = torch.empty(M, dtype=torch.float32, device=cuda)
    q, s, y = fused(x.to(cuda), w.to(cuda), eps, return_normed=True, _inv_dump=inv)
    y_ref = R.rmsnorm_given_inv(x, w, inv.cpu())
    q_ref, s_ref = R.quantize_activation_per_token_absmax(y_ref)
    assert torch.allclose(inv.cpu(), R.rmsnorm(x, w, eps)[1].view(-1), rtol=INV_RTOL, atol=0)
    assert torch.equal(y.cpu().view(torch.int16), y_ref.view(torch.int16))
    assert s.dtype == dtype and torch.equal(s.cpu().view(torch.int16), s_ref.view(torch.int16))
    assert torch.equal(q.cpu(), q_ref)
    # without the normalised output, with fp32 scales: same codes
    q2, s2 = fused(x.to(cuda), w.to(cuda), eps, scale_dtype=torch.float32)
    assert torch.equal(q2.cpu(), q_ref) and torch.equal(s2.cpu(), s_ref.float())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,K", SHAPES)
def test_rmsnorm_fp8_fused(cuda, M, K, dtype):
    from llmqrt_amd.norm import rmsnorm_per_token_quantize as fused
    x, w = _inputs(M, K, dtype, 9 * M + K)
    eps = 1e-5
    inv = torch.empty(M, dtype=torch.float32, device=cuda)
    q, s, y = fused(x.to(cuda), w.to(cuda), eps, return_normed=True, _inv_dump=inv)
    y_ref = R.rmsnorm_given_inv(x, w, inv.cpu())
    q_ref, s_ref = R.fp8_per_token_quantize(y_ref)
    assert torch.equal(y.cpu().view(torch.int16), y_ref.view(torch.int16))
    assert torch.equal(s.cpu(), s_ref)
    assert torch.equal(q.cpu().view(torch.uint8), q_ref.view(torch.uint8))


def test_strided_rows_and_3d(cuda):
    from llmqrt_amd.norm import RMSNorm
    x = torch.randn(2, 5, 1024, generator=torch.Generator().manual_seed(3)).bfloat16()
    w = torch.ones(512, dtype=torch.bfloat16)
    xs = x[..., :512]  # row stride 1024
    m = RMSNorm(w.to(cuda), 1e-6)
    y = m(xs.to(cuda))
    y_ref, _ = R.rmsnorm(xs, w, 1e-6)
    assert y.shape == (2, 5, 512)
    assert (y.cpu().float() - y_ref.float()).abs().max() <= 2.0 ** -7 * y_ref.float().abs().max()
    q, s = m.forward_quantized(xs.to(cuda))
    assert q.shape == (2, 5, 512) and s.shape == (2, 5, 1) and s.dtype == torch.float32
    assert m(torch.empty(0, 512, dtype=torch.bfloat16, device=cuda)).shape == (0, 512)


def test_norm_then_linear_matches_unfused(cuda):
    """The fused norm+quant feeding the W8A8 Linear gives exactly what norm -> Linear.forward gives."""
    from llmqrt_amd import workloads as W
    from llmqrt_amd.linear import SqW8A8BBF16OBF16PerChannel
    from llmqrt_amd.norm import RMSNorm
    K, N, M = 896, 4864, 16
    x = W.activations(M, K, 77, dtype=torch.bfloat16).to(cuda)
    norm = RMSNorm(torch.ones(K, dtype=torch.bfloat16, device=cuda) * 1.5, 1e-6)
    lin = SqW8A8BBF16OBF16PerChannel(8, 0, K, N, True, dev=cuda, dtype=torch.bfloat16)
    qw, ws = W.int8_weights(N, K, 78)
    lin.qweight.copy_(qw.to(cuda)); lin.weight_scale.copy_(ws.to(cuda))
    unfused = lin(norm(x))
    q, s = norm.forward_quantized(x)
    fused = lin.forward_quantized(q, s, torch.bfloat16)
    assert torch.equal(unfused, fused)
