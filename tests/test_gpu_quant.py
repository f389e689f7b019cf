"""GPU parity: activation quantizers vs the CPU oracle, bit-exact (integer/byte outputs and scales)."""
import pytest
import torch

from oracle import ref_math as R

pytestmark = pytest.mark.gpu


def _acts(M, K, seed, dtype):
    from llmqrt_amd import workloads as W
    return W.activations(M, K, seed, dtype=dtype)


# (258, 896) .. (257, 520) take the wavefront-per-row kernels (256 rows or more of at most 1024 elements): ragged row
# counts, one and two chunks per lane, rows shorter than a wavefront; the last three the half-size blocks with four
# chunks per thread (256 rows or more of 2056 .. 4096 elements): the shortest and longest such rows and K = 3584
SHAPES = [(1, 896), (16, 896), (7, 3584), (128, 3584), (33, 18944), (3, 8), (5, 24576), (2, 40960),
          (258, 896), (1027, 1024), (300, 8), (257, 520), (300, 3584), (257, 2056), (256, 4096)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,K", SHAPES)
def test_int8_per_token(cuda, M, K, dtype):
    from llmqrt_amd.quantize import quantize_activation_per_token_absmax, quantize_activation_per_token_absmax_f32
    x = _acts(M, K, 11 * M + K, dtype)
    x[0, : min(K, 64)] = 0  # exercise exact zeros
    if M > 2:
        x[2] = 0            # an all-zero row: scale = round(round(1e-5)/127)
    q_ref, s_ref = R.quantize_activation_per_token_absmax(x)
    q, s = quantize_activation_per_token_absmax(x.to(cuda))
    assert q.dtype == torch.int8 and s.dtype == dtype and s.shape == (M, 1)
    assert torch.equal(s.cpu().view(torch.int16), s_ref.view(torch.int16))
    assert torch.equal(q.cpu(), q_ref)
    q2, s2 = quantize_activation_per_token_absmax_f32(x.to(cuda))
    assert torch.equal(q2.cpu(), q_ref) and torch.equal(s2.cpu(), s_ref.float())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,K", SHAPES)
def test_fp8_per_token(cuda, M, K, dtype):
    from llmqrt_amd.quantize import per_token_quantize
    x = _acts(M, K, 13 * M + K, dtype)
    if M > 2 and dtype == torch.bfloat16:
        x[2] = 0  # fp16 zero rows give scale 0 -> NaN in the reference; covered separately
    q_ref, s_ref = R.fp8_per_token_quantize(x)
    q, s = per_token_quantize(x.to(cuda))
    assert q.dtype == torch.float8_e4m3fn and s.dtype == torch.float32 and s.shape == (M, 1)
    assert torch.equal(s.cpu(), s_ref)
    assert torch.equal(q.cpu().view(torch.uint8), q_ref.view(torch.uint8))


def test_fp16_zero_row_fp8_is_nan_like_reference(cuda):
    from llmqrt_amd.quantize import per_token_quantize
    x = torch.zeros(2, 64, dtype=torch.float16)
    x[1] = 1.0
    q_ref, s_ref = R.fp8_per_token_quantize(x)
    q, s = per_token_quantize(x.to(cuda))
    assert torch.equal(s.cpu(), s_ref)
    assert torch.equal(q.cpu().view(torch.uint8), q_ref.view(torch.uint8))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_all_16bit_patterns(cuda, dtype):
    """Every finite 16-bit pattern as an input element, against several row maxima."""
    from llmqrt_amd.quantize import per_token_quantize, quantize_activation_per_token_absmax
    bits = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16).view(dtype)
    finite = bits[torch.isfinite(bits.float())]
    n = (finite.numel() // 8) * 8
    rows = []
    for amax in (0.75, 3.1415, 37.5, 1000.0, 6.1e-5, 65000.0 if dtype == torch.float16 else 3.0e38):
        r = finite[:n].clone().float()
        r[r.abs() > amax] = 0
        r[0] = amax
        rows.append(r.to(dtype))
    x = torch.stack(rows)
    q_ref, s_ref = R.quantize_activation_per_token_absmax(x)
    q, s = quantize_activation_per_token_absmax(x.to(cuda))
    assert torch.equal(s.cpu().view(torch.int16), s_ref.view(torch.int16))
    assert torch.equal(q.cpu(), q_ref)
    f_ref, fs_ref = R.fp8_per_token_quantize(x)
    f, fs = per_token_quantize(x.to(cuda))
    assert torch.equal(fs.cpu(), fs_ref)
    assert torch.equal(f.cpu().view(torch.uint8), f_ref.view(torch.uint8))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,K", [(16, 896), (130, 3584), (1, 8)])
def test_per_tensor(cuda, M, K, dtype):
    from llmqrt_amd.quantize import per_tensor_quantize, quantize_activation_per_tensor_absmax
    x = _acts(M, K, 17 * M + K, dtype)
    q_ref, s_ref = R.quantize_activation_per_tensor_absmax(x)
    q, s = quantize_activation_per_tensor_absmax(x.to(cuda))
    assert s.dim() == 0 and s.dtype == dtype
    assert s.cpu().view(torch.int16).item() == s_ref.view(torch.int16).item()
    assert torch.equal(q.cpu(), q_ref)
    f_ref, fs_ref = R.fp8_per_tensor_quantize(x)
    f, fs = per_tensor_quantize(x.to(cuda))
    assert fs.dim() == 0 and fs.cpu().item() == fs_ref.item()
    assert torch.equal(f.cpu().view(torch.uint8), f_ref.view(torch.uint8))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_static_fp8(cuda, dtype):
    from llmqrt_amd.quantize import static_per_tensor_quantize
    x = _acts(64, 896, 5, dtype)
    for scale in (0.0123456, 0.25, 1.7):
        st = torch.tensor([scale], dtype=torch.float32)
        ref_t = R.fp8_static_per_tensor_quantize(x, st)          # fp32 tensor scale: fp32 quotient
        got_t = static_per_tensor_quantize(x.to(cuda), st.to(cuda))
        assert torch.equal(got_t.cpu().view(torch.uint8), ref_t.view(torch.uint8))
        ref_f = R.fp8_static_per_tensor_quantize(x, scale)       # Python float: quotient in x.dtype
        got_f = static_per_tensor_quantize(x.to(cuda), scale)
        assert torch.equal(got_f.cpu().view(torch.uint8), ref_f.view(torch.uint8))


def test_strided_input_and_3d(cuda):
    from llmqrt_amd.quantize import quantize_activation_per_token_absmax
    x = _acts(8, 1024, 3, torch.bfloat16)
    xs = x.to(cuda)[:, :512]                                     # row stride 1024, K 512
    q_ref, s_ref = R.quantize_activation_per_token_absmax(x[:, :512].contiguous())
    q, s = quantize_activation_per_token_absmax(xs)
    assert torch.equal(q.cpu(), q_ref) and torch.equal(s.cpu(), s_ref)
    x3 = x.view(2, 4, 1024)
    q3, s3 = quantize_activation_per_token_absmax(x3.to(cuda))
    assert q3.shape == (2, 4, 1024) and s3.shape == (2, 4, 1)
    assert torch.equal(q3.cpu().view(8, 1024), R.quantize_activation_per_token_absmax(x)[0])


def test_empty_rows(cuda):
    from llmqrt_amd.quantize import per_token_quantize, quantize_activation_per_token_absmax
    x = torch.empty(0, 64, dtype=torch.bfloat16, device=cuda)
    q, s = quantize_activation_per_token_absmax(x)
    assert q.shape == (0, 64) and s.shape == (0, 1)
    q, s = per_token_quantize(x)
    assert q.shape == (0, 64) and s.shape == (0, 1)


def test_full_size_scaling_property(cuda):
    """Largest quantizer launch of the benchmark (M = 8192, K = 18944), checked through a size-independent
    property instead of the CPU oracle: multiplying the input by 2 is exact in bf16, leaves every code
    unchanged and doubles every scale; a sample of rows is also compared with the oracle bit for bit."""
    from llmqrt_amd import workloads as W
    from llmqrt_amd.quantize import per_token_quantize, quantize_activation_per_token_absmax
    M, K = 8192, 18944
    x = W.activations(M, K, 4321).to(cuda)
    for quant in (quantize_activation_per_token_absmax, per_token_quantize):
        q1, s1 = quant(x)
        q2, s2 = quant(x * 2)
        assert torch.equal(q1.view(torch.uint8), q2.view(torch.uint8))
        assert torch.equal(s2.float(), 2 * s1.float())
    rows = torch.arange(3, M, M // 32)
    xr = x[rows.to(cuda)].cpu()
    q_ref, s_ref = R.quantize_activation_per_token_absmax(xr)
    q, s = quantize_activation_per_token_absmax(x)
    assert torch.equal(q[rows.to(cuda)].cpu(), q_ref) and torch.equal(s[rows.to(cuda)].cpu().view(torch.int16), s_ref.view(torch.int16))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("N,K", [(64, 264), (3, 7), (1, 3584), (300, 1000)])
def test_weight_per_channel(cuda, N, K, dtype):
    """Per-output-channel weight quantizer (utils/quantization_utils.py:27-38) in the dtype of w: codes and scales
    bit-exact against the oracle, for any K, a strided view, a row far below the activation quantizer's floor and an
    all-zero row (NaN scale, zero codes)."""
    from llmqrt_amd.quantize import quantize_weight_per_channel_absmax
    g = torch.Generator().manual_seed(N * 1000 + K)
    w = (torch.randn(N, 2 * K, generator=g) * 0.05).to(dtype)
    w[0] *= 1e-6
    if N > 2:
        w[2] = 0
    wv = w[:, :K]
    q_ref, s_ref = R.quantize_weight_per_channel_absmax(wv.contiguous(), native_dtype=True)
    q, s = quantize_weight_per_channel_absmax(w.to(cuda)[:, :K])
    assert q.dtype == torch.int8 and s.dtype == dtype and s.shape == (N, 1)
    assert torch.equal(q.cpu(), q_ref)
    sc, sr = s.cpu().view(-1), s_ref.view(-1)
    assert torch.equal(torch.isnan(sc), torch.isnan(sr))
    ok = ~torch.isnan(sr)
    assert torch.equal(sc[ok], sr[ok])


def test_sq_per_channel_module_quantizes_its_weight_on_the_gpu(cuda):
    """SqW8A8BBF16OBF16PerChannel.from_linear on a GPU module runs the HIP weight quantizer (fp32 arithmetic on the
    fp32 copy of the weight): buffers equal the oracle's."""
    from llmqrt_amd.linear import SqW8A8BBF16OBF16PerChannel
    torch.manual_seed(3)
    lin = torch.nn.Linear(264, 72, bias=True).to(cuda)
    mod = SqW8A8BBF16OBF16PerChannel.from_linear(lin, 8, 0, init_only=False, dtype=torch.bfloat16)
    q_ref, s_ref = R.quantize_weight_per_channel_absmax(lin.weight.data.cpu())
    assert torch.equal(mod.qweight.cpu(), q_ref) and torch.equal(mod.weight_scale.cpu(), s_ref.view(-1))


# ---- NaN inputs: torch's max / amax propagate a NaN into the scale, so the whole row (per token) or the whole tensor
# (per tensor) comes out as NaN scale with zero int8 codes / NaN fp8 codes.  (7, 3584): a block per row with the row
# in registers; (300, 512): a wavefront per row; (3, 24576): a block per row, second pass re-reading the row;
# (260, 3584): half-size blocks with four chunks per thread.
NAN_SHAPES = [(7, 3584), (300, 512), (3, 24576), (260, 3584)]


def _with_nans(M, K, seed, dtype):
    x = _acts(M, K, seed, dtype)
    x[0, K // 3] = float("nan")   # one NaN in an otherwise finite row
    x[1] = float("nan")           # an all-NaN row
    x[2, 0] = float("nan")
    x[2, K - 1] = float("-inf")   # NaN beside an infinity
    return x


def _same_with_nans(a, b):
    a, b = a.float(), b.float()
    return torch.equal(torch.isnan(a), torch.isnan(b)) and torch.equal(torch.nan_to_num(a, nan=0.0), torch.nan_to_num(b, nan=0.0))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,K", NAN_SHAPES)
def test_nan_elements_make_the_row_nan_like_the_reference(cuda, M, K, dtype):
    from llmqrt_amd.quantize import per_token_quantize, quantize_activation_per_token_absmax
    x = _with_nans(M, K, 5 * M + K, dtype)
    q_ref, s_ref = R.quantize_activation_per_token_absmax(x)
    assert torch.isnan(s_ref[:3]).all() and not torch.isnan(s_ref[3:]).any() and (q_ref[:3] == 0).all()
    q, s = quantize_activation_per_token_absmax(x.to(cuda))
    assert _same_with_nans(s.cpu(), s_ref)
    assert torch.equal(q.cpu(), q_ref)
    q8_ref, s8_ref = R.fp8_per_token_quantize(x)
    assert torch.isnan(q8_ref[:3].float()).all()
    q8, s8 = per_token_quantize(x.to(cuda))
    assert _same_with_nans(s8.cpu(), s8_ref)
    assert _same_with_nans(q8.cpu(), q8_ref)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_nan_element_per_tensor_like_the_reference(cuda, dtype):
    from llmqrt_amd.quantize import per_tensor_quantize, quantize_activation_per_tensor_absmax
    x = _acts(40, 1024, 77, dtype)
    x[17, 300] = float("nan")
    q_ref, s_ref = R.quantize_activation_per_tensor_absmax(x)
    q, s = quantize_activation_per_tensor_absmax(x.to(cuda))
    assert torch.isnan(s_ref).all() and _same_with_nans(s.cpu(), s_ref) and torch.equal(q.cpu(), q_ref)
    q8_ref, s8_ref = R.fp8_per_tensor_quantize(x)
    q8, s8 = per_tensor_quantize(x.to(cuda))
    assert _same_with_nans(s8.cpu(), s8_ref) and _same_with_nans(q8.cpu(), q8_ref)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,K", [(5, 3584), (260, 1024)])
def test_nan_element_through_rmsnorm_quant(cuda, M, K, dtype):
    """A NaN in a row makes its mean square, hence every normalised element, NaN: NaN scale, zero codes."""
    from llmqrt_amd.norm import rmsnorm_quantize_activation_per_token_absmax
    x = _acts(M, K, 3 * M + K, dtype)
    x[1, 5] = float("nan")
    w = (1.0 + 0.1 * torch.randn(K, generator=torch.Generator().manual_seed(1))).to(dtype)
    q, s = rmsnorm_quantize_activation_per_token_absmax(x.to(cuda), w.to(cuda), 1e-6)
    assert torch.isnan(s.cpu().float()[1]).all() and (q.cpu()[1] == 0).all()
    assert not torch.isnan(s.cpu().float()[0]).any() and not torch.isnan(s.cpu().float()[2:]).any()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,K", [(7, 3584), (300, 512), (3, 24576)])
def test_dynamic_quantizers_with_the_1e8_floor(cuda, M, K, dtype):
    """The twins of utils/quantization_utils.py:57-71 (clamp at 1e-8).  Rows whose absmax lies between the two
    floors tell them apart: with 1e-5 they quantize to 0 / +-1, with 1e-8 they use the full int8 range.  (In fp16
    1e-8 rounds to 0, so an all-zero row divides 0 by 0: NaN scale, zero codes, as in the reference.)"""
    from llmqrt_amd.quantize import (dynamic_quantize_activation_per_tensor_absmax,
                                     dynamic_quantize_activation_per_token_absmax, quantize_activation_per_token_absmax)
    x = _acts(M, K, 17 * M + K, dtype)
    x[1] = (x[1].float() * 1e-7).to(dtype)   # absmax ~4e-7 (fp16: subnormals)
    x[2] = 0
    q_ref, s_ref = R.dynamic_quantize_activation_per_token_absmax(x)
    keep = x.clone()
    q, s = dynamic_quantize_activation_per_token_absmax(x.to(cuda))
    assert _same_with_nans(s.cpu(), s_ref) and torch.equal(q.cpu(), q_ref)
    assert torch.equal(x.view(torch.int16), keep.view(torch.int16))
    if dtype == torch.bfloat16:   # (fp16 has no values between the two floors' scales: both round to its smallest steps)
        q5, _ = quantize_activation_per_token_absmax(x.to(cuda))
        assert not torch.equal(q5.cpu()[1], q_ref[1]), "the tiny row must tell the two floors apart"
    tiny = (x.float() * 1e-7).to(dtype)
    qt_ref, st_ref = R.dynamic_quantize_activation_per_tensor_absmax(tiny)
    qt, st = dynamic_quantize_activation_per_tensor_absmax(tiny.to(cuda))
    assert _same_with_nans(st.cpu(), st_ref) and torch.equal(qt.cpu(), qt_ref)
