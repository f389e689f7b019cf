"""Pins of the CPU oracle (oracle/ref_math.py, oracle/llmq_oracle.c): golden vectors, closed forms,
brute force and the agreement of two independent implementations.  No GPU involved."""
import json
import math
import pathlib

import numpy as np
import pytest
import torch

from oracle import c_oracle as C
from oracle import ref_math as R

GOLDEN = pathlib.Path(__file__).resolve().parent / "golden"


def _acts(M, K, seed, dtype):
    from llmqrt_amd import workloads as W
    return W.activations(M, K, seed, dtype=dtype)


# ---- int8 quantizers ------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,K", [(16, 896), (4, 3584), (3, 8)])
def test_int8_per_token_torch_vs_scalar_c(M, K, dtype):
    x = _acts(M, K, 1 + M + K, dtype)
    q1, s1 = R.quantize_activation_per_token_absmax(x)
    q2, s2 = C.quant_i8_per_token(x)
    assert torch.equal(q1, q2) and torch.equal(s1.view(torch.int16), s2.view(torch.int16))
    qt, st = R.quantize_activation_per_tensor_absmax(x)
    qc, sc = C.quant_i8_per_tensor(x)
    assert torch.equal(qt, qc) and st.view(torch.int16).item() == sc.view(torch.int16).item()


def test_int8_known_answers():
    for case in json.loads((GOLDEN / "int8_quant_kat.json").read_text()):
        dt = getattr(torch, case["dtype"])
        x = torch.tensor([case["x"]], dtype=dt)
        for fn in (R.quantize_activation_per_token_absmax, C.quant_i8_per_token):
            q, s = fn(x)
            assert s.float().item() == case["scale"]
            assert q[0].tolist() == case["q"]


def test_int8_zero_row_scale_and_bf16_semantics():
    x = torch.zeros(1, 8, dtype=torch.bfloat16)
    q, s = R.quantize_activation_per_token_absmax(x)
    # clamp bound 1e-5 rounds to bf16 1.00136e-05 (0x3728); /127 rounds to bf16 again
    bound = torch.tensor(1e-5).bfloat16()
    assert bound.view(torch.int16).item() == 0x3728
    assert s.item() == (bound.float() / 127).bfloat16().item()
    assert torch.count_nonzero(q) == 0
    # the reference's bf16 double rounding is visible: an fp32 evaluation differs on some codes
    x = _acts(16, 896, 0, torch.bfloat16)
    q, s = R.quantize_activation_per_token_absmax(x)
    s32 = x.float().abs().amax(-1, keepdim=True).clamp(min=1e-5) / 127
    q32 = (x.float() / s32).round().clamp(-128, 127).to(torch.int8)
    frac = (q != q32).float().mean().item()
    assert 0 < frac < 0.05
    assert (q.int() - q32.int()).abs().max().item() == 1


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_int8_all_16bit_patterns(dtype):
    bits = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16).view(dtype)
    finite = bits[torch.isfinite(bits.float())]
    n = (finite.numel() // 8) * 8
    for amax in (0.75, 37.5, 6.1e-5):
        r = finite[:n].clone().float()
        r[r.abs() > amax] = 0
        r[0] = amax
        x = r.to(dtype).view(1, -1)
        q1, s1 = R.quantize_activation_per_token_absmax(x)
        q2, s2 = C.quant_i8_per_token(x)
        assert torch.equal(q1, q2) and torch.equal(s1.view(torch.int16), s2.view(torch.int16))
        f1, fs1 = R.fp8_per_token_quantize(x)
        f2, fs2 = C.quant_fp8_per_token(x)
        assert torch.equal(f1.view(torch.uint8), f2.view(torch.uint8)) and torch.equal(fs1, fs2)


def test_weight_quantizer_argmax_maps_to_127():
    w = 0.02 * torch.randn(64, 256, generator=torch.Generator().manual_seed(0))
    q, s = R.quantize_weight_per_channel_absmax(w)
    assert q.abs().amax(dim=1).eq(127).all()          # fp32 semantics: the arg-max element is exactly +-127
    assert ((q.float() * s) - w).abs().max() <= s.max() / 2 + 1e-9


# ---- e4m3fn ----------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_weight_quantizer_native_dtype_is_the_per_token_quantizer_without_floor(dtype):
    """In the dtype of w the per-channel weight quantizer is the per-token activation quantizer (pinned above by known
    answers, the scalar C restatement and every 16-bit pattern) for every row whose absmax reaches the activation
    quantizer's floor of 1e-5; below it only the weight quantizer keeps dividing by absmax / 127."""
    g = torch.Generator().manual_seed(11)
    w = (torch.randn(64, 264, generator=g) * 0.05).to(dtype)
    w[3] *= 1e-3
    w[5, 7] = 3.0
    q, s = R.quantize_weight_per_channel_absmax(w, native_dtype=True)
    qt, st = R.quantize_activation_per_token_absmax(w)
    assert s.dtype == dtype and torch.equal(s.view(-1), st.view(-1)) and torch.equal(q, qt)
    tiny = (torch.randn(4, 64, generator=g) * 1e-7).to(dtype)
    q2, s2 = R.quantize_weight_per_channel_absmax(tiny, native_dtype=True)
    for r in range(4):
        if tiny[r].abs().max() > 0:
            assert q2[r].abs().max() >= 126  # the row maximum still maps to the top of the range (the scale is itself rounded)
    assert R.quantize_activation_per_token_absmax(tiny)[0].abs().max() < 16  # with the floor they stay near zero


def test_e4m3_decode_table_matches_format_definition():
    table = json.loads((GOLDEN / "e4m3fn_table.json").read_text())
    c_tab = C.e4m3_decode_table()
    t_tab = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float()
    for code, v in enumerate(table):
        if v == "nan":
            assert math.isnan(c_tab[code]) and math.isnan(t_tab[code].item())
        else:
            assert c_tab[code] == v and t_tab[code].item() == v
    assert table[0x7E] == 448.0 and table[0x01] == 2.0 ** -9


def test_e4m3_encode_roundtrip_ties_and_saturation():
    codes = [c for c in range(256) if (c & 0x7F) != 0x7F]
    vals = C.e4m3_decode_table()[codes]
    assert C.e4m3_encode(vals).tolist() == codes                      # decode -> encode is the identity
    # ties go to the even mantissa: 17 is halfway between 16 (m=0) and 18 (m=1); 19 between 18 and 20
    assert C.e4m3_encode([17.0, 19.0, 464.0, 448.0]).tolist() == [0x58, 0x5A, 0x7E, 0x7E]
    # torch's own cast agrees on every bf16 value in range, and maps > 464 to NaN (hence the clamp)
    bits = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    enc_t = bits.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    enc_c = C.e4m3_encode(bits.float().numpy())
    assert np.array_equal(enc_t, enc_c)
    assert torch.tensor([465.0]).to(torch.float8_e4m3fn).float().isnan().all()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fp8_quantizers_torch_vs_scalar_c(dtype):
    x = _acts(16, 896, 5, dtype)
    q1, s1 = R.fp8_per_token_quantize(x)
    q2, s2 = C.quant_fp8_per_token(x)
    assert torch.equal(q1.view(torch.uint8), q2.view(torch.uint8)) and torch.equal(s1, s2)
    # the arg-max element of each row lands on +-448 up to the bf16/fp16 rounding of the quotient
    assert (q1.float().abs().amax(-1) >= 416).all()
    q1, s1 = R.fp8_per_tensor_quantize(x)
    q2, s2 = C.quant_fp8_per_tensor(x)
    assert torch.equal(q1.view(torch.uint8), q2.view(torch.uint8)) and s1.item() == s2.item()
    q, s = R.fp8_per_token_quantize(torch.empty(0, 8, dtype=dtype))
    assert q.shape == (0, 8) and s.shape == (0, 1)


# ---- int8 GEMM + epilogues -------------------------------------------------------------------
def test_int_gemm_exact_vs_int64_loops_and_known_answer():
    g = torch.Generator().manual_seed(0)
    a = torch.randint(-128, 128, (9, 80), dtype=torch.int8, generator=g)
    b = torch.randint(-128, 128, (21, 80), dtype=torch.int8, generator=g)
    assert torch.equal(R.int8_gemm_exact(a, b), C.gemm_i8(a, b))
    assert torch.equal(R.int8_gemm_exact(a, b), (a.long() @ b.long().t()).int())
    a = torch.tensor([[1, -2, 3, -128]], dtype=torch.int8)
    b = torch.tensor([[4, 5, -6, -128], [0, 0, 0, 1]], dtype=torch.int8)
    assert R.int8_gemm_exact(a, b).tolist() == [[4 - 10 - 18 + 16384, -128]]
    # worst case of the workload stays inside int32 and exact in fp64
    a = torch.full((1, 18944), -128, dtype=torch.int8)
    assert R.int8_gemm_exact(a, a).item() == 18944 * 16384


def test_epilogue_invariants():
    g = torch.Generator().manual_seed(1)
    acc = torch.randint(-50000, 50000, (8, 12), generator=g).int()
    sa, sw = torch.rand(8, generator=g) + 0.1, torch.rand(12, generator=g) + 0.1
    bias = torch.randn(12, generator=g).bfloat16()
    ones_a, ones_w = torch.ones(8), torch.ones(12)
    # all-ones scales reduce to the int -> float cast (+ bias)
    assert torch.equal(R.w8a8_epilogue_per_token_per_channel(acc, ones_a, ones_w, None, torch.float32), acc.float())
    # scaling a row / column scale by 2 scales that row / column of the bias-free output by exactly 2
    y = R.w8a8_epilogue_per_token_per_channel(acc, sa, sw, None, torch.float32)
    sa2 = sa.clone(); sa2[3] *= 2
    y2 = R.w8a8_epilogue_per_token_per_channel(acc, sa2, sw, None, torch.float32)
    assert torch.equal(y2[3], 2 * y[3]) and torch.equal(y2[:3], y[:3])
    # per-tensor form equals the per-channel form with constant scales
    yt = R.w8a8_epilogue_per_tensor(acc, bias, 0.5, 1.0, torch.float32)
    yc = R.w8a8_epilogue_per_token_per_channel(acc, 0.5 * ones_a, ones_w, bias, torch.float32)
    assert torch.equal(yt, yc)
    # and the dequantize-then-matmul baseline agrees within fp32 rounding
    qx = torch.randint(-128, 128, (8, 64), dtype=torch.int8, generator=g)
    qw = torch.randint(-128, 128, (12, 64), dtype=torch.int8, generator=g)
    a = R.w8a8_epilogue_per_token_per_channel(R.int8_gemm_exact(qx, qw), sa, sw, bias, torch.float32)
    b = R.w8a8_linear_naive(qx, sa, qw, sw, bias, torch.float32)
    assert torch.allclose(a, b, rtol=1e-5, atol=1e-3)


def test_epilogue_multiplication_order():
    """The reference's torch helper multiplies (acc * w_scale) * a_scale (utils/quantization_utils.py:89-97), the
    op's epilogue (acc * a_scale) * w_scale (the row-wise fp8 op's tree).  Both round each fp32 product once:
    they agree to 2 fp32 ulps, are identical for power-of-two scales, and after narrowing to bf16 differ in
    at most a vanishing fraction of elements by one bf16 step."""
    g = torch.Generator().manual_seed(4)
    acc = torch.randint(-2000000, 2000000, (64, 96), generator=g).int()
    sa, sw = torch.rand(64, generator=g) * 0.05 + 1e-3, torch.rand(96, generator=g) * 0.01 + 1e-4
    a = R.w8a8_epilogue_per_token_per_channel(acc, sa, sw, None, torch.float32)
    b = R.dequantize_activation_w_per_channel_a_per_token(acc, sw, sa.view(-1, 1))
    assert b.dtype == torch.float32 and ((a - b).abs() <= 2.5e-7 * a.abs()).all()
    p2a, p2w = 2.0 ** torch.randint(-8, 0, (64,), generator=g), 2.0 ** torch.randint(-10, -2, (96,), generator=g)
    assert torch.equal(R.w8a8_epilogue_per_token_per_channel(acc, p2a, p2w, None, torch.float32),
                       R.dequantize_activation_w_per_channel_a_per_token(acc, p2w, p2a.view(-1, 1)))
    a16 = R.w8a8_epilogue_per_token_per_channel(acc, sa, sw, None, torch.bfloat16)
    b16 = R.dequantize_activation_w_per_channel_a_per_token(acc, sw, sa.view(-1, 1).bfloat16().float()).bfloat16()
    # (a_scales given in bf16 selects a bf16 result in the helper; compared on the same fp32 scale values)
    a16b = R.w8a8_epilogue_per_token_per_channel(acc, sa.bfloat16().float(), sw, None, torch.bfloat16)
    assert (a16b != b16).float().mean() < 1e-3
    assert ((a16b.float() - b16.float()).abs() <= 2.0 ** -7 * b16.float().abs()).all()
    assert a16.dtype == torch.bfloat16


def test_reference_recipe_tolerance_sq():
    """unittest/test_sq_linear.py:8-34: the per-tensor op is within atol 0.1 of an fp16 Linear."""
    g = torch.Generator().manual_seed(0)
    weight = torch.randint(-128, 127, (1024, 512), dtype=torch.int8, generator=g)
    bias = torch.randn(1024, generator=g).half()
    x = torch.randint(-128, 127, (128, 512), dtype=torch.int8, generator=g)
    y_gt = torch.nn.functional.linear(x.float() * 0.002, weight.float() * 0.00334, bias.float())
    y = R.w8a8_epilogue_per_tensor(R.int8_gemm_exact(x, weight), bias, 0.00334 * 0.002, 1.0, torch.float16)
    assert torch.allclose(y_gt, y.float(), atol=0.1)


# ---- AWQ --------------------------------------------------------------------------------------
def test_awq_orders_are_inverse_permutations():
    O, Rv = R.AWQ_ORDER, R.AWQ_REVERSE_ORDER
    assert sorted(O) == list(range(8)) and all(Rv[O[i]] == i for i in range(8))
    assert [((j & 1) << 2) | (j >> 1) for j in range(8)] == list(Rv)   # closed form used by the kernels


def test_awq_known_words():
    for case in json.loads((GOLDEN / "awq_kat.json").read_text()):
        word = torch.tensor([[case["word"]]], dtype=torch.int32)
        assert R.awq_unpack(word)[0].tolist() == case["columns"]
        assert R.awq_pack(torch.tensor([case["columns"]], dtype=torch.int32)).item() == case["word"]


def test_awq_pack_unpack_identity_all_slots():
    for slot in range(8):
        for v in range(16):
            cols = torch.zeros(1, 16, dtype=torch.int32)
            cols[0, slot] = v
            cols[0, 8 + slot] = 15 - v
            assert torch.equal(R.awq_unpack(R.awq_pack(cols)), cols)
    g = torch.Generator().manual_seed(0)
    cols = torch.randint(0, 16, (7, 64), generator=g, dtype=torch.int32)
    assert torch.equal(R.awq_unpack(R.awq_pack(cols)), cols)


def test_awq_dequant_torch_vs_scalar_c_and_closed_form():
    from llmqrt_amd import workloads as W
    w = W.dense_weights(72, 256, 3)
    qw, qz, s = R.awq_quantize_weight(w, 64)
    d1, d2 = R.awq_dequantize(qw, qz, s, 64), C.awq_dequant(qw, qz, s, 64)
    assert torch.equal(d1.view(torch.int16), d2.view(torch.int16))
    # quantization error: half a step from q, half a step from the rounded zero point (+ fp16 rounding)
    step = s.float().repeat_interleave(64, dim=0)
    assert ((d1.float() - w.t()).abs() <= 1.0 * step + 1e-3 * step + 1e-6).all()
    # the product package's packer produces the same words as the oracle's
    a, b, c = W.awq_weights(72, 256, 3, group=64)
    assert torch.equal(a, qw) and torch.equal(b, qz) and torch.equal(c, s)
    x = W.activations(3, 256, 4, dtype=torch.float16, outliers=False)
    y1, y2 = R.awq_gemm(x, qw, qz, s, 64), C.awq_gemm(x, qw, qz, s, 64)
    assert (y1.float() - y2.float()).abs().max() <= 2e-3 * y1.float().abs().max()


# ---- RMSNorm ----------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_rmsnorm_closed_forms(dtype):
    eps = 1e-6
    # a constant row c has RMS |c|: inv = 1/sqrt(c^2 + eps), y = w * round(c * inv)
    c = 3.0
    x = torch.full((2, 64), c, dtype=dtype)
    w = torch.linspace(-2, 2, 64).to(dtype)
    y, inv = R.rmsnorm(x, w, eps)
    assert torch.allclose(inv, torch.full((2, 1), 1.0 / math.sqrt(c * c + eps)), rtol=3e-7, atol=0)
    n = torch.tensor(c * (1.0 / math.sqrt(c * c + eps))).to(dtype)      # rounds to exactly 1.0
    assert float(n) == 1.0
    assert torch.equal(y, w.expand(2, 64))
    # a single spike of height a in K zeros: mean = a^2 / K
    x = torch.zeros(1, 256, dtype=dtype)
    x[0, 17] = -8.0
    y, inv = R.rmsnorm(x, torch.ones(256, dtype=dtype), 0.0)
    assert float(inv) == pytest.approx(math.sqrt(256) / 8.0, rel=3e-7)
    assert float(y[0, 17]) == -16.0 and float(y.abs().sum()) == 16.0
    # an all-zero row: inv = 1/sqrt(eps), output exactly zero
    y, inv = R.rmsnorm(torch.zeros(1, 64, dtype=dtype), w, eps)
    assert float(inv) == pytest.approx(1000.0, rel=3e-7) and not y.any()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,K", [(5, 896), (3, 3584), (2, 8)])
def test_rmsnorm_torch_vs_scalar_c_and_f64(M, K, dtype):
    eps = 1e-6
    x = _acts(M, K, 900 + M + K, dtype)
    g = torch.Generator().manual_seed(K)
    w = (1.0 + 0.1 * torch.randn(K, generator=g)).to(dtype)
    y, inv = R.rmsnorm(x, w, eps)
    # the reciprocal RMS agrees with a double-precision evaluation to a few fp32 ulps ...
    inv64 = C.inv_rms_f64(x, eps)
    assert torch.allclose(inv.view(-1).double(), inv64, rtol=5e-7, atol=0)
    # ... and everything after it is pinned bit for bit by the independent scalar implementation
    assert torch.equal(R.rmsnorm_given_inv(x, w, inv).view(torch.int16), y.view(torch.int16))
    assert torch.equal(C.rmsnorm_given_inv(x, w, inv).view(torch.int16), y.view(torch.int16))
    # against exact arithmetic the result is within the two roundings of the formula
    exact = w.double() * (x.double() * inv64.view(M, 1))
    ulp = 2.0 ** (-8 if dtype == torch.bfloat16 else -11)
    assert ((y.double() - exact).abs() <= 2.5 * ulp * exact.abs() + 1e-30).all()
    # scale invariance: normalising 2x gives the same result up to eps
    y2, _ = R.rmsnorm((x.float() * 2).to(dtype), w, 0.0)
    y0, _ = R.rmsnorm(x, w, 0.0)
    assert (y2.float() - y0.float()).abs().max() <= 2 * ulp * y0.float().abs().max()
