"""GPU parity of the one-launch few-token linears (per-token dynamic quantizer + GEMM + epilogue):
codes, scales and raw accumulators against the oracle, outputs bit-identical to the two-launch form."""
import pytest
import torch

from oracle import ref_math as R

pytestmark = pytest.mark.gpu

# (K, N): Qwen2-7B qkv and down, a ragged channel edge with an odd number of K steps plus a 16-byte tail, one step
SHAPES = [(3584, 4608), (18944, 3584), (1040, 264), (64, 40)]


@pytest.fixture
def force_variant():
    from llmqrt_amd import _abi
    yield lambda v: _abi.check(_abi.lib().llmq_linear_dynamic_force_variant(v), "force_variant")
    _abi.lib().llmq_linear_dynamic_force_variant(-1)


@pytest.mark.parametrize("variant", [0, 1])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M", [1, 3, 16])
@pytest.mark.parametrize("K,N", SHAPES)
def test_int8_dynamic_linear(cuda, force_variant, variant, dtype, M, K, N):
    from llmqrt_amd import workloads as W
    from llmqrt_amd.sq_fp8_kernels import dynamic_linear_max_tokens
    if M > dynamic_linear_max_tokens(K):
        pytest.skip("the quantized rows of this many tokens do not fit in LDS at this K")
    from llmqrt_amd.quantize import quantize_activation_per_token_absmax_f32
    from llmqrt_amd.sq_fp8_kernels import w8a8_int8_linear_bbf16_obf16_per_channel, w8a8_int8_linear_dynamic_per_token
    x = W.activations(M, 2 * K, 900 + M + K, dtype=dtype)[:, :K]   # row stride 2K
    qw, sw = W.int8_weights(N, K, 901 + N)
    bias = (0.1 * torch.randn(N, generator=torch.Generator().manual_seed(N))).to(dtype)
    q_ref, s_ref = R.quantize_activation_per_token_absmax(x)
    acc_ref = R.int8_gemm_exact(q_ref, qw)
    xd = W.activations(M, 2 * K, 900 + M + K, dtype=dtype).to(cuda)[:, :K]
    assert xd.stride(0) == 2 * K
    args = (qw.to(cuda).t(), bias.to(cuda), sw.to(cuda))
    force_variant(variant)
    qd = torch.full((M, K), 99, dtype=torch.int8, device=cuda)
    sd = torch.zeros(M, dtype=torch.float32, device=cuda)
    ad = torch.full((M, N), -5, dtype=torch.int32, device=cuda)
    y = w8a8_int8_linear_dynamic_per_token(xd, *args, _q_dump=qd, _scale_dump=sd, _acc_dump=ad)
    assert y.dtype == dtype and y.shape == (M, N)
    assert torch.equal(qd.cpu(), q_ref), "codes"
    assert torch.equal(sd.cpu(), s_ref.float().view(-1)), "scales"
    assert torch.equal(ad.cpu(), acc_ref), "int32 accumulators"
    q2, s2 = quantize_activation_per_token_absmax_f32(xd.contiguous())
    two = w8a8_int8_linear_bbf16_obf16_per_channel(q2, args[0], args[1], s2, args[2])
    assert torch.equal(y.view(torch.int16), two.view(torch.int16)), "same bits as quantizer + GEMM"
    assert torch.equal(y, w8a8_int8_linear_dynamic_per_token(xd, *args)), "deterministic, dumps optional"


@pytest.mark.parametrize("variant", [0, 1])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M", [1, 3, 16])
@pytest.mark.parametrize("K,N", SHAPES)
def test_fp8_dynamic_linear(cuda, force_variant, variant, dtype, M, K, N):
    from llmqrt_amd import _abi, workloads as W
    from llmqrt_amd.sq_fp8_kernels import dynamic_linear_max_tokens
    if M > dynamic_linear_max_tokens(K):
        pytest.skip("the quantized rows of this many tokens do not fit in LDS at this K")
    from llmqrt_amd.quantize import per_token_quantize
    from llmqrt_amd.sq_fp8_kernels import cutlass_f8f8bf16_rowwise_sm89, f8f8bf16_linear_dynamic_per_token
    x = W.activations(M, K, 910 + M + K, dtype=dtype)
    wq, ws = W.fp8_weights(N, K, 911 + N)
    bias = (0.1 * torch.randn(N, generator=torch.Generator().manual_seed(N))).bfloat16()
    q_ref, s_ref = R.fp8_per_token_quantize(x)
    xd = x.to(cuda)
    wsd = ws.to(cuda).float().reshape(-1).contiguous()
    force_variant(variant)
    qd = torch.zeros((M, K), dtype=torch.uint8, device=cuda)
    sd = torch.zeros(M, dtype=torch.float32, device=cuda)
    ad = torch.zeros((M, N), dtype=torch.float32, device=cuda)
    y = f8f8bf16_linear_dynamic_per_token(xd, wq.to(cuda).t(), bias.to(cuda), wsd, _q_dump=qd, _scale_dump=sd, _acc_dump=ad)
    assert y.dtype == torch.bfloat16 and y.shape == (M, N)
    assert torch.equal(qd.cpu(), q_ref.view(torch.uint8)), "codes"
    assert torch.equal(sd.cpu(), s_ref.view(-1)), "scales"
    q2, s2 = per_token_quantize(xd)
    ad2 = torch.zeros((M, N), dtype=torch.float32, device=cuda)
    # the few-token GEMM with the same channel tiles per wavefront and wavefronts along K adds in the same order
    _abi.check(_abi.lib().llmq_gemm_force_plan(101 if variant == 0 else 102, 1), "force_plan")
    try:
        two = cutlass_f8f8bf16_rowwise_sm89(q2, wq.to(cuda).t(), bias.to(cuda), s2.view(-1, 1), wsd.view(1, -1), True, _acc_dump=ad2)
    finally:
        _abi.lib().llmq_gemm_force_plan(-1, 1)
    assert torch.equal(ad, ad2), "same fp32 accumulators as the few-token GEMM"
    assert torch.equal(y.view(torch.int16), two.view(torch.int16)), "same bits as quantizer + GEMM"
    y_ref = R.fp8_linear_naive(q_ref, s_ref, wq, ws, bias)
    assert ((y.float().cpu() - y_ref.float()).abs().max() / y_ref.float().abs().max()).item() <= 1e-2


def test_dynamic_linear_rejects_more_tokens_and_bad_layout(cuda):
    from llmqrt_amd import workloads as W
    from llmqrt_amd.sq_fp8_kernels import dynamic_linear_max_tokens, w8a8_int8_linear_dynamic_per_token
    mt = dynamic_linear_max_tokens(128)
    assert mt == 16 and dynamic_linear_max_tokens(18944) == 3 and dynamic_linear_max_tokens(3584) == 16
    qw, sw = W.int8_weights(64, 128, 5)
    bias = torch.zeros(64, dtype=torch.bfloat16, device=cuda)
    x = torch.zeros((mt + 1, 128), dtype=torch.bfloat16, device=cuda)
    with pytest.raises(RuntimeError):
        w8a8_int8_linear_dynamic_per_token(x, qw.to(cuda).t(), bias, sw.to(cuda))
    with pytest.raises(RuntimeError):
        w8a8_int8_linear_dynamic_per_token(x[:2].float(), qw.to(cuda).t(), bias, sw.to(cuda))
    empty = w8a8_int8_linear_dynamic_per_token(x[:0], qw.to(cuda).t(), bias, sw.to(cuda))
    assert empty.shape == (0, 64)


@pytest.mark.parametrize("tokens", [1, 4, 5])
def test_modules_take_the_one_launch_path_with_identical_results(cuda, tokens):
    """SqW8A8BBF16OBF16PerChannel and FP8DynamicLinear (per token) switch to the one-launch kernel up to 4 tokens:
    the result must not depend on which side of the switch a batch falls (rows of a 17-token batch = the same rows
    computed alone)."""
    from llmqrt_amd.linear import FP8DynamicLinear, SqW8A8BBF16OBF16PerChannel
    torch.manual_seed(3)
    dense = torch.nn.Linear(512, 384, bias=True).to(cuda)
    x = torch.randn(17, 512, device=cuda).to(torch.bfloat16)
    sq = SqW8A8BBF16OBF16PerChannel.from_linear(dense, 8, 0, init_only=False, dtype=torch.bfloat16)
    f8 = FP8DynamicLinear.from_linear(dense, init_only=False, dtype=torch.bfloat16, per_tensor=False)
    full, part = sq(x), sq(x[:tokens])    # 17 tokens: quantizer + GEMM; up to 4: one launch
    assert torch.equal(part, full[:tokens])   # int32 accumulation is exact, the epilogue arithmetic is shared
    full, part = f8(x), f8(x[:tokens])    # fp32 accumulation: the two kernels add in different orders
    assert ((part.float() - full[:tokens].float()).abs().max() / full.float().abs().max()).item() <= 1e-2
