"""GPU: llmq_gemm_w8a8_static - the W8A8 GEMM entry point that takes no workspace and allocates nothing (its
split-K partial sums live in a static device array) - gives bit-identical outputs to llmq_gemm_w8a8 with a
caller workspace.  Two calls in a row share the array, the second with a smaller problem; both use a K split, so
the array is really written and read.  Collected last: it runs after every other GPU test has used the library
and also passes alone in a fresh process."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _problem(M, N, K, seed, cuda):
    g = torch.Generator().manual_seed(seed)
    qx = torch.randint(-128, 128, (M, K), dtype=torch.int8, generator=g).to(cuda)
    qw = torch.randint(-128, 128, (N, K), dtype=torch.int8, generator=g).to(cuda)
    sa = (torch.rand(M, generator=g) * 0.05 + 0.01).to(cuda)
    sw = (torch.rand(N, generator=g) * 0.01 + 0.001).to(cuda)
    bias = torch.randn(N, generator=g).bfloat16().to(cuda)
    return qx, qw, sa, sw, bias


def _run(L, abi, static, p, M, N, K, cuda):
    qx, qw, sa, sw, bias = p
    out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=cuda)
    stream = torch.cuda.current_stream().cuda_stream
    head = (qx.data_ptr(), K, qw.data_ptr(), K, sa.data_ptr(), sw.data_ptr(), 1.0, None, bias.data_ptr(), abi.BF16, 1.0,
            out.data_ptr(), abi.BF16, N, M, N, K)
    if static:
        rc = L.llmq_gemm_w8a8_static(*head, stream)
    else:
        nbytes = L.llmq_gemm_workspace_bytes(M, N, K)
        assert nbytes > 0, "the case must exercise the split-K scratch"
        ws = torch.empty(nbytes, dtype=torch.uint8, device=cuda)
        rc = L.llmq_gemm_w8a8(*head, None, ws.data_ptr(), nbytes, stream)
    abi.check(rc, "gemm")
    torch.cuda.synchronize()
    return out


def test_static_scratch_gemm_matches_workspace_gemm(cuda):
    from llmqrt_amd import _abi
    L = _abi.lib()
    assert L.llmq_gemm_static_scratch_bytes() == 32 << 20
    cases = [(128, 3584, 18944, 1), (96, 1024, 18944, 2)]  # 7 MiB of partials, then a smaller problem (above 64 tokens: below,
    # the few-token kernel needs no scratch at all)
    problems = [_problem(M, N, K, seed, cuda) for M, N, K, seed in cases]
    want = [_run(L, _abi, False, p, M, N, K, cuda) for p, (M, N, K, _) in zip(problems, cases)]
    # back to back on one stream, no synchronisation in between other than the stream order
    got = [_run(L, _abi, True, p, M, N, K, cuda) for p, (M, N, K, _) in zip(problems, cases)]
    for g, w in zip(got, want):
        assert not torch.isnan(g.float()).any()
        assert torch.equal(g.view(torch.int16), w.view(torch.int16))
    # and once more in the opposite order (small, then large): stale contents of the array are harmless
    for idx in (1, 0):
        M, N, K, _ = cases[idx]
        assert torch.equal(_run(L, _abi, True, problems[idx], M, N, K, cuda).view(torch.int16), want[idx].view(torch.int16))


def test_static_scratch_gemm_rejects_oversized_problems(cuda):
    from llmqrt_amd import _abi
    L = _abi.lib()
    M, N, K = 1536, 4096, 65536
    assert L.llmq_gemm_workspace_bytes(M, N, K) > L.llmq_gemm_static_scratch_bytes()
    rc = L.llmq_gemm_w8a8_static(0x1000, K, 0x1000, K, None, None, 1.0, None, None, 0, 0.0, 0x1000, 0, N, M, N, K, None)
    assert rc == -7 and b"scratch" in L.llmq_status_string(rc)
