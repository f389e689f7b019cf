"""CPU-only checks of the boundary: the shared library loads, exports every symbol that
include/llmq.h declares, its argument validation returns the documented codes before any HIP
call, and the Python wrappers mirror the reference's interface and error behaviour."""
import ctypes
import pathlib
import re

import pytest
import torch

ROOT = pathlib.Path(__file__).resolve().parent.parent


def _declared_symbols():
    text = (ROOT / "include" / "llmq.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(llmq_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from llmqrt_amd import _abi
    lib = _abi.lib()
    declared = _declared_symbols()
    assert len(declared) >= 14
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in llmq.h but not exported"
    assert sorted(_abi.SIGNATURES) == declared, "ctypes table and header disagree"
    assert lib.llmq_abi_version() == 1
    assert lib.llmq_status_string(0) == b"ok"
    assert b"workspace" in lib.llmq_status_string(-4)


def test_argument_validation_needs_no_gpu():
    from llmqrt_amd import _abi
    L = _abi.lib()
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.addressof(buf)
    p16 = (p + 15) & ~15
    # negative sizes / misaligned K / strides
    assert L.llmq_gemm_w8a8(p16, 64, p16, 64, None, None, 1.0, None, None, 0, 0.0, p16, 0, 8, -1, 8, 64, None, None, 0, None) == -3
    assert L.llmq_gemm_w8a8(p16, 24, p16, 24, None, None, 1.0, None, None, 0, 0.0, p16, 0, 8, 4, 8, 24, None, None, 0, None) == -3
    assert L.llmq_gemm_w8a8(None, 64, p16, 64, None, None, 1.0, None, None, 0, 0.0, p16, 0, 8, 4, 8, 64, None, None, 0, None) == -1
    assert L.llmq_gemm_w8a8(p16, 64, p16, 64, None, None, 1.0, None, None, 0, 0.0, p16, 2, 8, 4, 8, 64, None, None, 0, None) == -2
    assert L.llmq_gemm_w8a8(p16 + 1, 64, p16, 64, None, None, 1.0, None, None, 0, 0.0, p16, 0, 8, 4, 8, 64, None, None, 0, None) == -6
    assert L.llmq_gemm_w8a8(p16, 64, p16, 64, None, None, 1.0, None, None, 0, 0.0, p16, 0, 8, 0, 8, 64, None, None, 0, None) == 0  # M == 0
    assert L.llmq_gemm_fp8(p16, 7, 64, p16, 64, None, None, 1.0, None, None, 0, 0.0, p16, 0, 8, 4, 8, 64, None, None, 0, None) == -2
    assert L.llmq_quant_i8_per_token(p16, 2, 4, 64, 64, p16, p16, 2, None) == -2      # fp32 activations unsupported
    assert L.llmq_quant_i8_per_token(p16, 0, 4, 60, 64, p16, p16, 0, None) == -3      # K % 8
    assert L.llmq_quant_i8_per_token(p16, 0, 0, 64, 64, p16, p16, 0, None) == 0       # M == 0
    assert L.llmq_quant_i8_per_tensor(p16, 0, 4, 64, 64, p16, p16, 0, None, 0, None) == -4
    assert L.llmq_awq_gemm(p16, 100, p16, p16, p16, None, p16, 2, 64, 100, 128, None, 0, None) == -3   # K % 32
    assert L.llmq_awq_gemm(p16, 128, p16, p16, p16, None, p16, 2, 60, 128, 128, None, 0, None) == -3   # N % 8
    assert L.llmq_awq_dequant(p16, p16, p16, p16, 128, 64, 48, None) == -3                              # K % G
    assert L.llmq_gemm_force_plan(99, 1) == -3 and L.llmq_gemm_force_plan(106, 1) == -3 and L.llmq_gemm_force_plan(-1, 1) == 0
    assert L.llmq_quant_workspace_bytes() >= 4096
    # split-K plans ask for a workspace, plain ones do not
    assert L.llmq_gemm_workspace_bytes(8192, 37888, 3584) == 0
    assert L.llmq_awq_gemm_workspace_bytes(1, 4608, 3584) > 0


def test_wrappers_fail_loudly_off_gpu():
    from llmqrt_amd import sq_fp8_kernels as ops
    from llmqrt_amd.quantize import quantize_activation_per_token_absmax
    x = torch.zeros(4, 64, dtype=torch.int8)
    w = torch.zeros(8, 64, dtype=torch.int8)
    with pytest.raises(RuntimeError, match="GPU"):
        ops.w8a8_int8_linear_bbf16_obf16_per_tensor(x, w.t(), torch.zeros(8, dtype=torch.bfloat16), 1.0, 1.0)
    with pytest.raises(RuntimeError, match="GPU"):
        quantize_activation_per_token_absmax(torch.zeros(2, 8, dtype=torch.bfloat16))


def test_missing_library_is_an_error(monkeypatch, tmp_path):
    from llmqrt_amd import _abi
    monkeypatch.setattr(_abi, "_lib", None)
    monkeypatch.setattr(_abi, "_LIB_PATH", tmp_path / "libllmq_gfx950.so")
    with pytest.raises(RuntimeError, match="no CPU or PyTorch fallback"):
        _abi.lib()


def test_product_package_never_touches_the_oracle():
    for path in (ROOT / "llmqrt_amd").rglob("*.py"):
        text = path.read_text()
        assert "oracle" not in text, f"{path} mentions the oracle"


def test_registry_and_module_interfaces():
    from llmqrt_amd.linear import (FP8DynamicLinear, FP8StaticLinear, SqW8A8BBF16OBF16PerTensor, WQLinear_GEMM,
                                   get_concrete_linear_module, method_to_linear)
    assert set(method_to_linear) == {"awq", "sq", "fp8_static_quant", "fp8_dynamic_quant"}
    assert get_concrete_linear_module("awq") is WQLinear_GEMM
    lin = torch.nn.Linear(128, 64, bias=True)
    sq = SqW8A8BBF16OBF16PerTensor.from_linear(lin, 8, 0, True, dtype=torch.bfloat16)
    assert sq.qweight.shape == (64, 128) and sq.qweight.dtype == torch.int8
    assert sq.bias.dtype == torch.bfloat16 and sq.weight_scale.dim() == 0 and sq.input_scale.dim() == 0
    assert set(sq.state_dict()) == {"qweight", "bias", "weight_scale", "input_scale"}
    f8 = FP8DynamicLinear.from_linear(lin, 8, 0, True, dtype=torch.bfloat16, per_tensor=False)
    assert f8.weight.dtype == torch.bfloat16 and f8.weight_scale.shape == (64, 1)
    assert FP8DynamicLinear.from_linear(lin, 8, 0, True, per_tensor=True).weight_scale.shape == (1,)
    st = FP8StaticLinear.from_linear(lin, 8, 0, True)
    assert set(st.state_dict()) == {"weight", "weight_scale", "bias", "input_scale", "output_scale"}
    awq = WQLinear_GEMM.from_linear(lin, 4, 64, True)
    assert awq.qweight.shape == (128, 8) and awq.qzeros.shape == (2, 8) and awq.scales.shape == (2, 64)
    assert awq.scales.dtype == torch.float16 and awq.bias.dtype == torch.float16
    with pytest.raises(AssertionError):
        FP8DynamicLinear.from_linear(lin, 8, 128, True)
    with pytest.raises(NotImplementedError):
        WQLinear_GEMM(8, 64, 128, 64, False, "cpu")


def test_awq_module_packer_matches_oracle():
    """from_linear takes scales / zeros as [K/G, N], the orientation the reference indexes
    (linear_awq.py:165-186, 203-219); N != K/G here so a transposed argument cannot pass unnoticed."""
    from llmqrt_amd.linear import WQLinear_GEMM
    from oracle import ref_math as R
    g = torch.Generator().manual_seed(0)
    lin = torch.nn.Linear(128, 64, bias=False)
    lin.weight.data = 0.02 * torch.randn(64, 128, generator=g)
    G = 64
    wg = lin.weight.data.t().contiguous().view(2, G, 64)      # [K/G, G, N]
    mx, mn = wg.amax(1), wg.amin(1)
    scales = ((mx - mn) / 15).clamp(min=1e-5)                 # [K/G, N]
    zeros = (-mn / scales).round().clamp(0, 15)               # [K/G, N]
    m = WQLinear_GEMM.from_linear(lin, 4, G, False, scales=scales, zeros=zeros)
    assert m.scales.shape == (2, 64) and torch.equal(m.scales, scales.half())
    iw = R.awq_unpack(m.qweight)
    assert iw.min() >= 0 and iw.max() <= 15
    assert torch.equal(R.awq_unpack(m.qzeros), zeros.int())
    # element by element against the reference's loop: intw[k, n] = round((W[n, k] + z s) / s)
    for k, n in [(0, 0), (5, 63), (64, 1), (127, 40)]:
        want = torch.round((lin.weight.data[n, k] + zeros[k // G, n] * scales[k // G, n]) / scales.half()[k // G, n])
        assert iw[k, n] == int(want)
    deq = R.awq_dequantize(m.qweight, m.qzeros, m.scales, G)
    assert (deq.float() - lin.weight.data.t()).abs().max() <= 0.51 * scales.max()
    with pytest.raises(RuntimeError, match="scales and zeros must be"):
        WQLinear_GEMM.from_linear(lin, 4, G, False, scales=scales.t().contiguous(), zeros=zeros.t().contiguous())


def test_workload_shapes_and_byte_counts():
    from llmqrt_amd import workloads as W
    assert W.QWEN2_7B_PROJ["gate_up"] == (3584, 37888) and W.CONFIG0_SHAPE == (16, 896, 4864)
    x = W.activations(16, 896, 0)
    assert x.dtype == torch.bfloat16 and x.shape == (16, 896)
    assert torch.equal(x, W.activations(16, 896, 0))                     # seeded
    assert 15 < x.float().abs().amax(-1).min() < 100                     # outlier channels set the row max
    q, s = W.int8_weights(64, 128, 1)
    assert q.dtype == torch.int8 and s.shape == (64,) and q.abs().amax(1).eq(127).all()
    f, fs = W.fp8_weights(64, 128, 1)
    assert f.dtype == torch.float8_e4m3fn and f.float().abs().amax(1).eq(448).all()
    assert W.gemm_ops(2048, 4608, 3584) == 67645734912
    assert W.awq_gemm_bytes(1, 4608, 3584) == 8596480                    # 8.60 MB
    assert W.w8a8_gemm_bytes(16, 4864, 896) == 4547648                   # 4.55 MB


def test_rmsnorm_argument_validation_needs_no_gpu():
    from llmqrt_amd import _abi
    L = _abi.lib()
    ok_ptr = 0x1000
    # null weight / output, bad dtype, K not a multiple of 8, misaligned input
    assert L.llmq_rmsnorm(ok_ptr, 0, 4, 64, 64, None, 1e-6, ok_ptr, None, None) == -1
    assert L.llmq_rmsnorm(ok_ptr, 0, 4, 64, 64, ok_ptr, 1e-6, None, None, None) == -1
    assert L.llmq_rmsnorm(ok_ptr, 2, 4, 64, 64, ok_ptr, 1e-6, ok_ptr, None, None) == -2
    assert L.llmq_rmsnorm(ok_ptr, 0, 4, 60, 64, ok_ptr, 1e-6, ok_ptr, None, None) == -3
    assert L.llmq_rmsnorm(ok_ptr + 2, 0, 4, 64, 64, ok_ptr, 1e-6, ok_ptr, None, None) == -6
    assert L.llmq_rmsnorm(ok_ptr, 0, 0, 64, 64, ok_ptr, 1e-6, ok_ptr, None, None) == 0
    assert L.llmq_rmsnorm_quant_i8_per_token(ok_ptr, 0, 4, 64, 64, ok_ptr, 1e-6, None, None, ok_ptr, 0, None, None) == -1
    assert L.llmq_rmsnorm_quant_i8_per_token(ok_ptr, 0, 4, 64, 64, ok_ptr, 1e-6, None, ok_ptr, ok_ptr, 1, None, None) == -2
    assert L.llmq_rmsnorm_quant_fp8_per_token(ok_ptr, 1, 4, 64, 32, ok_ptr, 1e-6, None, ok_ptr, ok_ptr, None, None) == -3


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; asking for more exits with a message instead of running."""
    import subprocess
    import sys
    root = pathlib.Path(__file__).resolve().parent.parent
    r = subprocess.run([sys.executable, str(root / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=300)
    assert r.returncode != 0
    assert "one GPU" in r.stderr and r.stdout.strip() == ""
