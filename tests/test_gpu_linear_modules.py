"""GPU parity of the Linear module classes (the reference's drop-in level) against the CPU oracle.

Each module is built from a dense nn.Linear with ``from_linear(..., init_only=False)``, run on the GPU, and
compared with the oracle's composition of the same steps (activation quantizer -> exact GEMM -> epilogue) on
the module's own quantized buffers: max |y - y_ref| / max |y_ref| <= 1e-2.  A second, loose check against the
dense fp32 Linear catches a wrong scale or a transposed weight, which the first check alone would also catch
only if the oracle composition were right: W8A8 / FP8 outputs stay within 6 % of the dense result.
"""
import pytest
import torch
from torch import nn

from oracle import ref_math as R

pytestmark = pytest.mark.gpu
REL_TOL = 1e-2
DENSE_TOL = 6e-2


def rel_err(y, ref):
    y, ref = y.float().cpu(), ref.float()
    return ((y - ref).abs().max() / ref.abs().max().clamp(min=1e-30)).item()


def _dense(N, K, seed, bias=True):
    g = torch.Generator().manual_seed(seed)
    lin = nn.Linear(K, N, bias=bias)
    with torch.no_grad():
        lin.weight.copy_(0.05 * torch.randn(N, K, generator=g))
        if bias:
            lin.bias.copy_(0.1 * torch.randn(N, generator=g))
    return lin


def _acts(shape, seed, dtype):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)).to(dtype)


def _dense_out(lin, x):
    return nn.functional.linear(x.float(), lin.weight.float(), None if lin.bias is None else lin.bias.float())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("bias", [True, False])
def test_sq_per_tensor_module(cuda, dtype, bias):
    from llmqrt_amd.linear import SqW8A8BBF16OBF16PerTensor
    lin = _dense(264, 512, 1, bias)
    m = SqW8A8BBF16OBF16PerTensor.from_linear(lin.to(cuda), 8, 0, init_only=False, dtype=dtype)
    x = _acts((2, 19, 512), 2, dtype)
    y = m(x.to(cuda))
    assert y.shape == (2, 19, 264) and y.dtype == dtype
    qx, sx = R.quantize_activation_per_tensor_absmax(x.view(-1, 512))
    alpha = float((sx.float() * m.weight_scale.float().cpu()).to(dtype))
    acc = R.int8_gemm_exact(qx, m.qweight.cpu())
    b = m.bias.cpu() if bias else torch.zeros(264, dtype=dtype)
    ref = R.w8a8_epilogue_per_tensor(acc, b, alpha, 1.0, dtype)
    assert rel_err(y.view(-1, 264), ref) <= REL_TOL
    assert rel_err(y.view(-1, 264), _dense_out(lin.cpu(), x.view(-1, 512))) <= DENSE_TOL


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_sq_per_channel_module(cuda, dtype):
    from llmqrt_amd.linear import SqW8A8BBF16OBF16PerChannel
    lin = _dense(520, 384, 3)
    m = SqW8A8BBF16OBF16PerChannel.from_linear(lin.to(cuda), 8, 0, init_only=False, dtype=dtype)
    x = _acts((37, 384), 4, dtype)
    y = m(x.to(cuda))
    assert y.shape == (37, 520) and y.dtype == dtype
    qx, sx = R.quantize_activation_per_token_absmax(x)
    ref = R.w8a8_epilogue_per_token_per_channel(R.int8_gemm_exact(qx, m.qweight.cpu()), sx.float().view(-1),
                                                m.weight_scale.cpu(), m.bias.cpu(), dtype)
    assert rel_err(y, ref) <= REL_TOL
    assert rel_err(y, _dense_out(lin.cpu(), x)) <= DENSE_TOL


@pytest.mark.parametrize("per_tensor", [True, False])
def test_fp8_dynamic_module(cuda, per_tensor):
    from llmqrt_amd.linear import FP8DynamicLinear
    lin = _dense(264, 512, 5)
    m = FP8DynamicLinear.from_linear(lin.to(cuda), init_only=False, dtype=torch.bfloat16, per_tensor=per_tensor)
    x = _acts((3, 11, 512), 6, torch.bfloat16)
    y = m(x.to(cuda))
    assert y.shape == (3, 11, 264) and y.dtype == torch.bfloat16
    wq = m.weight.data.cpu().to(torch.float8_e4m3fn)
    x2 = x.view(-1, 512)
    if per_tensor:
        xq, xs = R.fp8_per_tensor_quantize(x2)
        alpha = float(xs.float().view(-1)[0] * m.weight_scale.float().cpu().view(-1)[0])
        ref = R.fp8_epilogue_tensorwise(R.fp8_gemm_acc(xq, wq), m.bias.cpu(), alpha, 1.0, torch.bfloat16)
    else:
        xq, xs = R.fp8_per_token_quantize(x2)
        ref = R.fp8_epilogue_rowwise(R.fp8_gemm_acc(xq, wq), xs, m.weight_scale.float().cpu().view(-1), m.bias.cpu())
    assert rel_err(y.view(-1, 264), ref) <= REL_TOL
    assert rel_err(y.view(-1, 264), _dense_out(lin.cpu(), x2)) <= DENSE_TOL


@pytest.mark.parametrize("quantize_output", [False, True])
def test_fp8_static_module(cuda, quantize_output):
    """Static input scale, and with ``quantize_output`` the output rounded to fp8 on a stored scale and
    scaled back (linear_fp8.py:309-311, the KV-cache scale)."""
    from llmqrt_amd.linear import FP8StaticLinear
    lin = _dense(264, 512, 7)
    m = FP8StaticLinear.from_linear(lin.to(cuda), init_only=False, dtype=torch.bfloat16,
                                    quantize_output=quantize_output)
    x = _acts((23, 512), 8, torch.bfloat16)
    in_scale = (x.float().abs().max() / 448.0).reshape(1)
    dense = _dense_out(lin.cpu(), x)
    out_scale = (dense.abs().max() / 448.0).reshape(1)
    m.input_scale.data = in_scale.to(cuda)
    m.output_scale.data = out_scale.to(cuda)
    y = m(x.to(cuda))
    # `fp8.to(bf16) * output_scale` with a 1-element fp32 tensor promotes to fp32, in the reference as here
    assert y.shape == (23, 264) and y.dtype == (torch.float32 if quantize_output else torch.bfloat16)
    wq = m.weight.data.cpu().to(torch.float8_e4m3fn)
    xq = R.fp8_static_per_tensor_quantize(x, in_scale)
    alpha = float(m.weight_scale.float().cpu().view(-1)[0] * in_scale[0])
    ref = R.fp8_epilogue_tensorwise(R.fp8_gemm_acc(xq, wq), m.bias.cpu(), alpha, 1.0, torch.bfloat16)
    if quantize_output:
        # fp8 rounding of the output: an input one bf16 ulp apart may land on the neighbouring fp8 value, so
        # the bound is one fp8 step (2^-3 relative at e4m3's 3 mantissa bits) of the largest output.
        ref = R.fp8_static_per_tensor_quantize(ref, out_scale).to(torch.bfloat16) * out_scale
        assert rel_err(y, ref) <= 2.0 ** -3
        q = (y.float().cpu() / out_scale).to(torch.float8_e4m3fn).float() * out_scale
        assert rel_err(y, q.to(torch.bfloat16).float()) <= 2.0 ** -7, "outputs must sit on the fp8 grid of output_scale"
    else:
        assert rel_err(y, ref) <= REL_TOL
    assert rel_err(y, dense) <= (0.1 if quantize_output else DENSE_TOL)


@pytest.mark.parametrize("dtype_str", ["bfloat16", "float16"])
@pytest.mark.parametrize("M,N,K", [(23, 264, 512), (300, 392, 1040), (512, 768, 384), (64, 3584, 18944)])
def test_fp8_output_quantization_in_the_epilogue_is_bit_exact(cuda, M, N, K, dtype_str):
    """f8f8_tensorwise_quantized_output (one launch) against the reference's three steps on the same GEMM result
    (linear_fp8.py:309-311): the e4m3fn codes and the fp32 outputs must agree bit for bit, on ragged and interior
    tiles and with a K split (the last shape)."""
    from llmqrt_amd.sq_fp8_kernels import cutlass_f8f8bf16_tensorwise_sm89, f8f8_tensorwise_quantized_output
    dt = {"bfloat16": torch.bfloat16, "float16": torch.float16}[dtype_str]
    g = torch.Generator().manual_seed(M + N)
    xq = torch.randn(M, K, generator=g).clamp(-3, 3).to(torch.float8_e4m3fn)
    wq = torch.randn(N, K, generator=g).clamp(-3, 3).to(torch.float8_e4m3fn)
    bias = torch.randn(N, generator=g).to(dt)
    alpha = 0.37 / K ** 0.5
    plain = cutlass_f8f8bf16_tensorwise_sm89(xq.to(cuda), wq.to(cuda).t(), bias.to(cuda), alpha, 1.0, dtype_str).cpu()
    out_scale = (plain.float().abs().max() / 600.0).reshape(1)   # some outputs beyond +-448 * scale: the clamp matters
    fused = f8f8_tensorwise_quantized_output(xq.to(cuda), wq.to(cuda).t(), bias.to(cuda), alpha, 1.0, dtype_str,
                                             out_scale.to(cuda))
    assert fused.dtype == torch.float32 and fused.shape == (M, N)
    q_ref = R.fp8_static_per_tensor_quantize(plain, out_scale)
    assert (q_ref.float().abs() == 448).any(), "the case is meant to reach the clamp"
    ref = q_ref.to(dt) * out_scale
    assert ref.dtype == torch.float32
    assert torch.equal(fused.cpu().view(torch.int32), ref.view(torch.int32))
    codes = (fused.cpu() / out_scale).to(torch.float8_e4m3fn)
    assert torch.equal(codes.view(torch.uint8), q_ref.view(torch.uint8))


def test_zero_tokens(cuda):
    """The reference returns zeros of the right shape for an empty batch (linear_fp8.py:288-289, linear_awq.py:98)."""
    from llmqrt_amd.linear import FP8DynamicLinear, FP8StaticLinear, WQLinear_GEMM
    x = torch.empty((0, 512), dtype=torch.bfloat16, device=cuda)
    for m in (FP8DynamicLinear(512, 264, True, dev=cuda), FP8StaticLinear(512, 264, True, dev=cuda)):
        y = m(x)
        assert y.shape == (0, 264)
    y = WQLinear_GEMM(4, 128, 512, 264, False, cuda)(x.half())
    assert y.shape == (0, 264)
