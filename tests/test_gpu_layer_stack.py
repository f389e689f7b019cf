"""GPU parity of the decoder-layer linear stack (qkv, o, gate_up, down at Qwen2-7B shapes) in SmoothQuant W8A8
with the smoothing factors (alpha = 0.5) folded into the preceding RMSNorm weight.

qkv and gate_up read the residual stream through the fused RMSNorm + per-token quantizer kernel with the
folded norm weight g / s; o and down read their producer's output (already divided by s) through the plain
per-token quantizer.  Every stage is compared with the oracle composition
  RMSNorm (nn_models/modules/nonlinear/norm.py:4-16, callers block.py:68,76)
  -> quantize_activation_per_token_absmax (linear_sq.py:55-65)
  -> exact integer GEMM -> per-token x per-channel dequantization (utils/quantization_utils.py:89-97):
the reciprocal RMS within a few fp32 ulps, codes / scales / int32 accumulators bit-exact, outputs within
1e-2 (max abs error over max abs reference).  32 tokens are checked in full, 2048 tokens on sampled rows.
"""
import pytest
import torch

from oracle import ref_math as R

pytestmark = pytest.mark.gpu

OUT_TOL = 1e-2
INV_RTOL = 5e-7


@pytest.fixture(scope="module")
def layer():
    from llmqrt_amd import workloads as W
    return W.smoothquant_layer(alpha=0.5)


def _run_projection(cuda, p, pname, M):
    """-> dict of CPU tensors produced by the HIP path for one projection."""
    from llmqrt_amd import _abi, workloads as W
    from llmqrt_amd.norm import rmsnorm_quantize_activation_per_token_absmax as norm_quant
    from llmqrt_amd.quantize import quantize_activation_per_token_absmax_f32
    K, N = p["K"], p["N"]
    x = W.layer_input(pname, M, p["s"])
    xd = x.to(cuda)
    got = {"x": x}
    if p["norm_weight_folded"] is not None:
        inv = torch.empty(M, dtype=torch.float32, device=cuda)
        q, sc = norm_quant(xd, p["norm_weight_folded"].to(cuda), W.LAYER_NORM_EPS, scale_dtype=torch.float32,
                           _inv_dump=inv)
        got["inv"] = inv.cpu()
    else:
        q, sc = quantize_activation_per_token_absmax_f32(xd)
    qw, ws = p["qweight"].to(cuda), p["w_scale"].to(cuda)
    out = torch.empty((M, N), dtype=torch.bfloat16, device=cuda)
    acc = torch.empty((M, N), dtype=torch.int32, device=cuda)
    L = _abi.lib()
    wsb = L.llmq_gemm_workspace_bytes(M, N, K)
    wsp = torch.empty(max(wsb, 16), dtype=torch.uint8, device=cuda)
    _abi.check(L.llmq_gemm_w8a8(q.data_ptr(), K, qw.data_ptr(), K, sc.data_ptr(), ws.data_ptr(), 1.0, None, None, 0,
                                0.0, out.data_ptr(), _abi.BF16, N, M, N, K, acc.data_ptr(), wsp.data_ptr(),
                                wsp.numel(), _abi.stream_of(xd)), "llmq_gemm_w8a8")
    # the production launch (no accumulator dump: the fast epilogue) must give the same outputs
    out2 = torch.empty_like(out)
    _abi.check(L.llmq_gemm_w8a8(q.data_ptr(), K, qw.data_ptr(), K, sc.data_ptr(), ws.data_ptr(), 1.0, None, None, 0,
                                0.0, out2.data_ptr(), _abi.BF16, N, M, N, K, None, wsp.data_ptr(), wsp.numel(),
                                _abi.stream_of(xd)), "llmq_gemm_w8a8")
    torch.cuda.synchronize()
    assert torch.equal(out, out2)
    got.update(q=q.cpu(), scale=sc.cpu().view(-1), acc=acc.cpu(), out=out.cpu())
    return got


@pytest.mark.parametrize("M", [32, 2048])
@pytest.mark.parametrize("pname", ["qkv", "o", "gate_up", "down"])
def test_layer_stack_projection(cuda, layer, pname, M):
    from llmqrt_amd import workloads as W
    p = layer[pname]
    got = _run_projection(cuda, p, pname, M)
    rows = torch.arange(M) if M <= 64 else torch.arange(0, M, M // 32)
    x = got["x"][rows]
    if p["norm_weight_folded"] is not None:
        _, inv_ref = R.rmsnorm(x, p["norm_weight_folded"], W.LAYER_NORM_EPS)
        inv = got["inv"][rows]
        assert torch.allclose(inv, inv_ref.view(-1), rtol=INV_RTOL, atol=0)
        y = R.rmsnorm_given_inv(x, p["norm_weight_folded"], inv)
    else:
        y = x
    q_ref, s_ref = R.quantize_activation_per_token_absmax(y)
    assert torch.equal(got["q"][rows], q_ref)
    assert torch.equal(got["scale"][rows], s_ref.float().view(-1))
    acc_ref = R.int8_gemm_exact(q_ref, p["qweight"])
    assert torch.equal(got["acc"][rows], acc_ref)
    ref = R.w8a8_epilogue_per_token_per_channel(acc_ref, s_ref, p["w_scale"], None, torch.bfloat16).float()
    err = (got["out"][rows].float() - ref).abs().max() / ref.abs().max()
    assert err <= OUT_TOL
    # against the dequantize-then-matmul form the reference's forward uses (linear_sq.py:117-125)
    naive = R.w8a8_linear_naive(q_ref, s_ref, p["qweight"], p["w_scale"], None, torch.bfloat16).float()
    assert (got["out"][rows].float() - naive).abs().max() / naive.abs().max() <= OUT_TOL


def test_smoothing_preserves_the_dense_layer(cuda, layer):
    """End to end on 32 tokens of qkv: the W8A8 result with the folded norm stays close to the fp32 dense
    layer norm(x) @ W^T it replaces (the smoothing itself is an identity; what remains is quantization noise)."""
    from llmqrt_amd import workloads as W
    p = layer["qkv"]
    got = _run_projection(cuda, p, "qkv", 32)
    y, _ = R.rmsnorm(got["x"], p["norm_weight"], W.LAYER_NORM_EPS)
    dense = y.float() @ p["w"].t()
    rel = (got["out"].float() - dense).abs().max() / dense.abs().max()
    # the oracle's own W8A8 result on the folded form carries the same quantization noise
    yf, _ = R.rmsnorm(got["x"], p["norm_weight_folded"], W.LAYER_NORM_EPS)
    q_ref, s_ref = R.quantize_activation_per_token_absmax(yf)
    ref = R.w8a8_epilogue_per_token_per_channel(R.int8_gemm_exact(q_ref, p["qweight"]), s_ref, p["w_scale"], None,
                                                torch.bfloat16).float()
    rel_ref = (ref - dense).abs().max() / dense.abs().max()
    assert rel < 0.15 and rel <= rel_ref + OUT_TOL
