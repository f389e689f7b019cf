"""GPU parity: AWQ W4A16 kernels vs the CPU oracle.

Dequantized weights: bit-exact.  GEMM: max |y - y_ref| / max |y_ref| <= 1e-2 against
dequantize-then-matmul with fp32 accumulation (the reference's own fallback math; its Triton kernel
accumulates in fp16 with atomics and is not a bit-level oracle).
"""
import pytest
import torch

from oracle import ref_math as R

pytestmark = pytest.mark.gpu
REL_TOL = 1e-2


def rel_err(y, ref):
    y, ref = y.float().cpu(), ref.float()
    return ((y - ref).abs().max() / ref.abs().max().clamp(min=1e-30)).item()


@pytest.mark.parametrize("K,N,G", [(3584, 4608, 128), (896, 4864, 128), (256, 264, 64), (128, 8, 32), (512, 1000, 512),
                                   (8, 520, 8), (12, 1000, 12), (20, 8, 20)])  # the last two: one group that is not a multiple of 8
def test_dequant_bit_exact(cuda, K, N, G):
    from llmqrt_amd import workloads as W
    from llmqrt_amd.awq_kernels import awq_dequantize_triton
    qw, qz, s = W.awq_weights(N, K, K + N, group=G)
    ref = R.awq_dequantize(qw, qz, s, G)
    out = awq_dequantize_triton(qw.to(cuda), s.to(cuda), qz.to(cuda))
    assert out.dtype == torch.float16 and out.shape == (K, N)
    assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16))


def test_dequant_all_nibble_values(cuda):
    """Every (q, z) pair in every nibble slot, with scales that exercise fp16 rounding and subnormals."""
    from llmqrt_amd.awq_kernels import awq_dequantize_triton
    K, N = 256, 16
    g = torch.Generator().manual_seed(1)
    q = torch.arange(K, dtype=torch.int32).view(K, 1).expand(K, N) % 16
    q = (q + torch.arange(N, dtype=torch.int32).view(1, N)) % 16
    z = torch.randint(0, 16, (K // 32, N), generator=g, dtype=torch.int32)
    s = torch.rand(K // 32, N, generator=g).half() * 0.01
    s[0, :4] = torch.tensor([6.0e-8, 1.0e-5, 0.333, 1000.0]).half()
    qw, qz = R.awq_pack(q), R.awq_pack(z)
    ref = R.awq_dequantize(qw, qz, s, 32)
    out = awq_dequantize_triton(qw.to(cuda), s.to(cuda), qz.to(cuda))
    assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16))


_DECODE_WEIGHTS = {}


def _decode_weights(K, N):
    """One seeded weight set per shape, with the oracle's dequantized copy (shared by the token counts)."""
    from llmqrt_amd import workloads as W
    if (K, N) not in _DECODE_WEIGHTS:
        qw, qz, s = W.awq_weights(N, K, 3000 + K % 1000 + N % 1000, group=128)
        _DECODE_WEIGHTS[(K, N)] = (qw, qz, s, R.awq_dequantize(qw, qz, s, 128).float())
    return _DECODE_WEIGHTS[(K, N)]


# every cell of the decode workload: qkv, o, gate_up, down of Qwen2-7B (and the Qwen2-0.5B up-projection) x 1, 4, 16, 64
# tokens, on the plan the library picks by itself
@pytest.mark.parametrize("M", [1, 4, 16, 64])
@pytest.mark.parametrize("K,N", [(3584, 4608), (3584, 3584), (3584, 37888), (18944, 3584), (896, 4864)])
def test_gemm_decode_shapes(cuda, M, K, N):
    from llmqrt_amd import workloads as W
    from llmqrt_amd.awq_kernels import awq_gemm_triton
    qw, qz, s, wdeq = _decode_weights(K, N)
    x = W.activations(M, K, 3100 + M, dtype=torch.float16, outliers=False)
    ref = (x.float() @ wdeq).half()   # dequantize-then-matmul with fp32 accumulation (R.awq_gemm on the shared copy)
    out = awq_gemm_triton(x.to(cuda), qw.to(cuda), s.to(cuda), qz.to(cuda), split_k_iters=8)
    assert out.dtype == torch.float16 and out.shape == (M, N)
    assert rel_err(out, ref) <= REL_TOL
    out2 = awq_gemm_triton(x.to(cuda), qw.to(cuda), s.to(cuda), qz.to(cuda), split_k_iters=8)
    assert torch.equal(out, out2), "the kernel must be deterministic"


@pytest.mark.parametrize("M,K,N,G", [(3, 256, 264, 64), (17, 128, 8, 32), (5, 512, 1000, 512), (65, 1024, 136, 128),
                                     (130, 256, 2048, 128), (2, 18944, 3584, 128), (16, 3584, 37888, 128)])
def test_gemm_ragged_and_wide(cuda, M, K, N, G):
    from llmqrt_amd import workloads as W
    from llmqrt_amd.awq_kernels import awq_gemm_triton
    qw, qz, s = W.awq_weights(N, K, 5 * M + N, group=G)
    x = W.activations(M, K, 6 * M + K, dtype=torch.float16, outliers=False)
    ref = R.awq_gemm(x, qw, qz, s, G)
    out = awq_gemm_triton(x.to(cuda), qw.to(cuda), s.to(cuda), qz.to(cuda), split_k_iters=8)
    assert rel_err(out, ref) <= REL_TOL


def test_gemm_asserts_like_reference(cuda):
    from llmqrt_amd.awq_kernels import awq_gemm_triton
    qw = torch.zeros(128, 16, dtype=torch.int32, device=cuda)
    qz = torch.zeros(1, 16, dtype=torch.int32, device=cuda)
    s = torch.ones(1, 128, dtype=torch.float16, device=cuda)
    x = torch.ones(2, 128, dtype=torch.float16, device=cuda)
    with pytest.raises(AssertionError):
        awq_gemm_triton(x, qw, s, qz, split_k_iters=3)     # not a power of two
    with pytest.raises(AssertionError):
        awq_gemm_triton(x, qw, s, qz, split_k_iters=64)    # > 32
    with pytest.raises(AssertionError):
        awq_gemm_triton(x[:, :64], qw, s, qz, split_k_iters=8)
    out = awq_gemm_triton(x, qw, s, qz, split_k_iters=8)    # all-zero q and z -> zeros
    assert torch.count_nonzero(out).item() == 0


def test_gemm_random_shapes(cuda):
    """Seeded random sizes: any M up to 70, N a multiple of 8, K a multiple of the group, groups 32 / 64 / 128."""
    from llmqrt_amd import workloads as W
    from llmqrt_amd.awq_kernels import awq_gemm_triton
    g = torch.Generator().manual_seed(777)
    for case in range(24):
        G = (32, 64, 128)[case % 3]
        M = int(torch.randint(1, 71, (1,), generator=g))
        N = 8 * int(torch.randint(1, 200, (1,), generator=g))
        K = G * int(torch.randint(1, 1 + 2048 // G, (1,), generator=g))
        qw, qz, sc = W.awq_weights(N, K, 9000 + case, group=G)
        x = W.activations(M, K, 9100 + case, dtype=torch.float16, outliers=False)
        bias = torch.randn(N, generator=g).half() if case % 2 else None
        y = awq_gemm_triton(x.to(cuda), qw.to(cuda), sc.to(cuda), qz.to(cuda), split_k_iters=8,
                            bias=None if bias is None else bias.to(cuda))
        ref = R.awq_gemm(x, qw, qz, sc, G)
        if bias is not None:
            ref = (ref.float() + bias.float()).half()
        rel = ((y.float().cpu() - ref.float()).abs().max() / ref.float().abs().max().clamp(min=1e-30)).item()
        assert rel <= 1e-2, (case, M, N, K, G, rel)


@pytest.mark.parametrize("M", [1, 16, 64, 200])
def test_gemm_at_a_vocabulary_size_n(cuda, M):
    """N = 152064 (594 column tiles of the few-token kernel, more blocks than any projection of the benchmark) on every
    path by token count, against the library's own dequantizer + fp32 matmul."""
    from llmqrt_amd.awq_kernels import awq_dequantize_triton, awq_gemm_triton
    K, N, G = 3584, 152064, 128
    g = torch.Generator(device=cuda).manual_seed(M)
    qw = torch.randint(-2**31, 2**31 - 1, (K, N // 8), dtype=torch.int32, device=cuda, generator=g)
    qz = torch.randint(-2**31, 2**31 - 1, (K // G, N // 8), dtype=torch.int32, device=cuda, generator=g)
    sc = (torch.rand(K // G, N, device=cuda, generator=g) * 0.02 + 0.001).half()
    x = torch.randn(M, K, device=cuda, generator=g).half()
    y = awq_gemm_triton(x, qw, sc, qz, 8)
    ref = x.float() @ awq_dequantize_triton(qw, sc, qz).float()
    assert ((y.float() - ref).abs().max() / ref.abs().max()).item() <= REL_TOL


def test_gemm_wide_random_sweep_equals_dequantize_then_matmul(cuda):
    """400 seeded shapes over every path behind awq_gemm_triton (few-token kernel with 1-4 token slabs, streaming kernels,
    tile kernel, dequantize + fp16 GEMM; groups 32 / 64 / 128; N from 32 to 8000; random 32-bit words, i.e. every nibble
    value everywhere): the product against the library's own dequantizer (bit-exact against the oracle, above) followed
    by an fp32 matmul - the equivalence the reference's module relies on when it switches paths at 1024 tokens
    (nn_models/modules/linear/linear_awq.py:64-65)."""
    import random
    from llmqrt_amd.awq_kernels import awq_dequantize_triton, awq_gemm_triton
    rnd = random.Random(4242)
    for case in range(400):
        M = rnd.choice([1, 2, 3, 4, 5, 7, 8, 9, 15, 16, 17, 31, 32, 33, 48, 63, 64, 65, 100, 256, 300, 1024, 1500])
        G = rnd.choice([128, 128, 128, 64, 32])
        K = G * rnd.randint(1, 40 if G == 128 else 20)
        N = 8 * rnd.choice([4, 8, 12, 16, 20, 32, 33, 64, 100, 128, 448, 576, 1000])
        g = torch.Generator(device=cuda).manual_seed(case)
        qw = torch.randint(-2**31, 2**31 - 1, (K, N // 8), dtype=torch.int32, device=cuda, generator=g)
        qz = torch.randint(-2**31, 2**31 - 1, (K // G, N // 8), dtype=torch.int32, device=cuda, generator=g)
        sc = (torch.rand(K // G, N, device=cuda, generator=g) * 0.02 + 0.001).half()
        x = torch.randn(M, K, device=cuda, generator=g).half()
        y = awq_gemm_triton(x, qw, sc, qz, 8)
        ref = x.float() @ awq_dequantize_triton(qw, sc, qz).float()
        err = ((y.float() - ref).abs().max() / ref.abs().max().clamp_min(1e-30)).item()
        assert err <= REL_TOL, (case, M, N, K, G, err)


@pytest.mark.parametrize("K", [512, 8320])
def test_module_paths_agree_around_the_token_threshold(cuda, K):
    """WQLinear_GEMM switches from the fused kernel to dequantize + matmul at a measured token count; one token
    below and at the threshold both paths must meet the same bound against the oracle."""
    from llmqrt_amd import workloads as W
    from llmqrt_amd.linear import WQLinear_GEMM
    from llmqrt_amd.linear.linear_awq import dequant_matmul_token_threshold
    N = 264
    qw, qz, sc = W.awq_weights(N, K, 4242)
    m = WQLinear_GEMM(4, 128, K, N, False, cuda)
    m.qweight, m.qzeros, m.scales = qw.to(cuda), qz.to(cuda), sc.to(cuda)
    t = dequant_matmul_token_threshold(K, N)
    assert t < 1024
    for M in (t - 1, t):
        x = W.activations(M, K, 4300 + M, dtype=torch.float16, outliers=False)
        y = m(x.to(cuda).view(1, M, K))
        assert y.shape == (1, M, N) and y.dtype == torch.float16
        assert rel_err(y.view(M, N), R.awq_gemm(x, qw, qz, sc, 128)) <= REL_TOL
    # with the switch off the same token count stays on the fused kernels
    from llmqrt_amd.linear import linear_awq
    linear_awq.USE_DEQUANT_MATMUL = False
    try:
        y2 = m(x.to(cuda).view(1, t, K))
    finally:
        linear_awq.USE_DEQUANT_MATMUL = True
    assert rel_err(y2.view(t, N), R.awq_gemm(x, qw, qz, sc, 128)) <= REL_TOL


@pytest.fixture
def force_awq_plan():
    from llmqrt_amd import _abi
    yield lambda v, splits, k_waves=0: _abi.check(_abi.lib().llmq_awq_force_plan(v, splits, k_waves), "llmq_awq_force_plan")
    _abi.lib().llmq_awq_force_plan(0, 0, 0)


# (M, K, N, G): ragged token / channel edges, K with a half tile at the end (K % 64 == 32), one K tile,
# groups of 32 (two per K tile) / 64 / 128 / K, more than one token tile and more than one channel tile
TILE_SHAPES = [(300, 1056, 520, 32), (65, 64, 8, 64), (1, 96, 136, 32), (257, 512, 264, 512), (130, 3584, 4608, 128),
               (64, 1024, 1000, 128)]


@pytest.mark.parametrize("tile", [3, 4, 7])
@pytest.mark.parametrize("splits", [0, 1, 3])
@pytest.mark.parametrize("M,K,N,G", TILE_SHAPES)
def test_tile_kernel_every_shape_and_split(cuda, force_awq_plan, tile, splits, M, K, N, G):
    """The many-token tile kernel (all three tile shapes, fused and split-K) against the oracle.  Its weights are
    fp16((q - z) * s) as in the reference dequantizer, accumulated in fp32."""
    from llmqrt_amd import workloads as W
    from llmqrt_amd.awq_kernels import awq_gemm_triton
    qw, qz, s = W.awq_weights(N, K, 7 * M + N, group=G)
    x = W.activations(M, K, 8 * M + K, dtype=torch.float16, outliers=False)
    bias = (0.1 * torch.randn(N, generator=torch.Generator().manual_seed(M))).half() if splits != 1 else None
    ref = R.awq_gemm(x, qw, qz, s, G)
    if bias is not None:
        ref = (ref.float() + bias.float()).half()
    force_awq_plan(tile, splits)
    out = awq_gemm_triton(x.to(cuda), qw.to(cuda), s.to(cuda), qz.to(cuda), split_k_iters=8,
                          bias=None if bias is None else bias.to(cuda))
    assert out.shape == (M, N) and out.dtype == torch.float16
    assert rel_err(out, ref) <= REL_TOL, (tile, splits, M, K, N, G)
    out2 = awq_gemm_triton(x.to(cuda), qw.to(cuda), s.to(cuda), qz.to(cuda), split_k_iters=8,
                           bias=None if bias is None else bias.to(cuda))
    assert torch.equal(out, out2), "deterministic"


@pytest.mark.parametrize("tile", [3, 4, 7])
@pytest.mark.parametrize("M,K,N,G,xstride", [(65, 64, 8, 64, 64), (257, 512, 264, 512, 1024), (130, 3584, 4608, 128, 3584),
                                            (300, 1088, 520, 32, 1096), (600, 1024, 1000, 128, 1024)])
def test_tile_kernel_direct_loads_equal_register_staging(cuda, force_awq_plan, tile, M, K, N, G, xstride):
    """With K a multiple of 64 the tile kernel fetches its activation tiles straight into LDS; variant + 32 keeps the
    register-staged loop.  Same products, same order: equal on every element, for every tile shape, ragged token /
    channel edges, several token tiles, and a row stride larger than K."""
    from llmqrt_amd import workloads as W
    from llmqrt_amd.awq_kernels import awq_gemm_triton
    qw, qz, s = W.awq_weights(N, K, 9 * M + N, group=G)
    x = W.activations(M, xstride, 10 * M + K, dtype=torch.float16, outliers=False).to(cuda)[:, :K]
    args = (x, qw.to(cuda), s.to(cuda), qz.to(cuda))
    force_awq_plan(tile, 0)
    direct = awq_gemm_triton(*args, split_k_iters=8)
    force_awq_plan(tile + 32, 0)
    staged = awq_gemm_triton(*args, split_k_iters=8)
    assert torch.equal(direct.view(torch.int16), staged.view(torch.int16))
    assert rel_err(direct, R.awq_gemm(x.cpu(), qw, qz, s, G)) <= REL_TOL


def test_tile_kernel_prefill_size(cuda):
    """1024 tokens of the Qwen2-7B qkv projection through the default plan (256x256 tiles)."""
    from llmqrt_amd import workloads as W
    from llmqrt_amd.awq_kernels import awq_gemm_triton
    M, K, N = 1024, 3584, 4608
    qw, qz, s = W.awq_weights(N, K, 515)
    x = W.activations(M, K, 516, dtype=torch.float16, outliers=False)
    out = awq_gemm_triton(x.to(cuda), qw.to(cuda), s.to(cuda), qz.to(cuda), split_k_iters=8)
    assert rel_err(out, R.awq_gemm(x, qw, qz, s, 128)) <= REL_TOL


@pytest.mark.parametrize("variant", [5, 6])
@pytest.mark.parametrize("splits", [0, 2])
@pytest.mark.parametrize("M,K,N", [(17, 1024, 264), (33, 512, 4608), (50, 3584, 1000), (64, 896, 4864), (3, 256, 136)])
def test_streaming_kernel_with_shared_unpack(cuda, force_awq_plan, variant, splits, M, K, N):
    """The streaming kernel with 2 (variant 5) or 4 (variant 6) token tiles per wavefront: every unpacked weight
    operand feeds all tiles; weights are dequantized to fp16((q - z) * s) like the reference's."""
    from llmqrt_amd import workloads as W
    from llmqrt_amd.awq_kernels import awq_gemm_triton
    qw, qz, s = W.awq_weights(N, K, 11 * M + N)
    x = W.activations(M, K, 12 * M + K, dtype=torch.float16, outliers=False)
    bias = (0.1 * torch.randn(N, generator=torch.Generator().manual_seed(M))).half() if splits else None
    ref = R.awq_gemm(x, qw, qz, s, 128)
    if bias is not None:
        ref = (ref.float() + bias.float()).half()
    force_awq_plan(variant, splits)
    out = awq_gemm_triton(x.to(cuda), qw.to(cuda), s.to(cuda), qz.to(cuda), split_k_iters=8,
                          bias=None if bias is None else bias.to(cuda))
    assert rel_err(out, ref) <= REL_TOL, (variant, splits, M, K, N)


# (M, K, N): one partial tile (N = 32), tiles that end inside a block's column range (N = 96, 4864 with 256-byte
# tiles), one group / one stage pair, several groups per block and per split, a strided activation matrix
DECODE_SHAPES = [(1, 128, 32), (3, 256, 96), (16, 896, 4864), (4, 3584, 4608), (13, 1024, 1056), (2, 2048, 512)]


@pytest.mark.parametrize("variant", [8, 9, 10, 11])
@pytest.mark.parametrize("splits", [0, 1, 3])
@pytest.mark.parametrize("M,K,N", DECODE_SHAPES)
def test_decode_kernel_every_variant_and_split(cuda, force_awq_plan, variant, splits, M, K, N):
    """The LDS-staged decode kernel (up to 16 tokens, group 128): both tile widths (128 / 256 bytes per row,
    variants 8, 10 / 9, 11), both prefetch depths (variants 10, 11: two stages in flight), fused and split along K,
    against the oracle; deterministic; a row stride larger than K."""
    from llmqrt_amd import workloads as W
    from llmqrt_amd.awq_kernels import awq_gemm_triton
    qw, qz, s = W.awq_weights(N, K, 13 * M + N)
    x = W.activations(M, 2 * K, 14 * M + K, dtype=torch.float16, outliers=False)[:, :K]  # row stride 2K
    bias = (0.1 * torch.randn(N, generator=torch.Generator().manual_seed(M))).half() if splits != 1 else None
    ref = R.awq_gemm(x, qw, qz, s, 128)
    if bias is not None:
        ref = (ref.float() + bias.float()).half()
    force_awq_plan(variant, splits)
    xd = W.activations(M, 2 * K, 14 * M + K, dtype=torch.float16, outliers=False).to(cuda)[:, :K]
    assert xd.stride(0) == 2 * K
    args = (xd, qw.to(cuda), s.to(cuda), qz.to(cuda))
    out = awq_gemm_triton(*args, split_k_iters=8, bias=None if bias is None else bias.to(cuda))
    assert out.shape == (M, N) and out.dtype == torch.float16
    assert rel_err(out, ref) <= REL_TOL, (variant, splits, M, K, N)
    out2 = awq_gemm_triton(*args, split_k_iters=8, bias=None if bias is None else bias.to(cuda))
    assert torch.equal(out, out2), "deterministic"


@pytest.mark.parametrize("slices", [2, 4])
@pytest.mark.parametrize("splits", [0, 1, 3])
@pytest.mark.parametrize("M,K,N", DECODE_SHAPES + [(8, 18944, 3584), (5, 640, 288)])
def test_decode_kernel_k_slices_inside_the_block(cuda, force_awq_plan, slices, splits, M, K, N):
    """K slices inside a block (2 or 4 sets of wavefronts with their own LDS stages, added in slice order): against
    the oracle and deterministic, fused and split along K, with bias; covers blocks with fewer groups than slices
    (K = 128: one group for four slices; K = 640 in 3 splits: 2 + 2 + 1 groups) and the long K of `down`."""
    from llmqrt_amd import workloads as W
    from llmqrt_amd.awq_kernels import awq_gemm_triton
    qw, qz, s = W.awq_weights(N, K, 17 * M + N)
    x = W.activations(M, K, 19 * M + K, dtype=torch.float16, outliers=False)
    bias = (0.1 * torch.randn(N, generator=torch.Generator().manual_seed(M))).half() if splits != 1 else None
    ref = R.awq_gemm(x, qw, qz, s, 128)
    if bias is not None:
        ref = (ref.float() + bias.float()).half()
    force_awq_plan(8, splits, slices)
    args = (x.to(cuda), qw.to(cuda), s.to(cuda), qz.to(cuda))
    out = awq_gemm_triton(*args, split_k_iters=8, bias=None if bias is None else bias.to(cuda))
    assert rel_err(out, ref) <= REL_TOL, (slices, splits, M, K, N)
    out2 = awq_gemm_triton(*args, split_k_iters=8, bias=None if bias is None else bias.to(cuda))
    assert torch.equal(out, out2), "deterministic"


@pytest.mark.parametrize("plan", [(0, 0, 0), (8, 0, 2), (8, 3, 4), (8, 1, 1), (8, 5, 2)])
@pytest.mark.parametrize("M,K,N", [(17, 1024, 288), (33, 512, 4608), (50, 3584, 1024), (64, 896, 4864), (40, 18944, 3584),
                                   (64, 3584, 37888), (31, 128, 32)])
def test_decode_kernel_token_slabs(cuda, force_awq_plan, plan, M, K, N):
    """17-64 tokens through the few-token kernel as slabs of 16 tokens (a ragged last slab; column-tile x split counts
    that are not multiples of 8, so that padded blocks exit; more blocks than fit at once): the automatic plan and
    forced slices / splits, against the oracle, with bias and a row stride larger than K; deterministic."""
    from llmqrt_amd import workloads as W
    from llmqrt_amd.awq_kernels import awq_gemm_triton
    qw, qz, s = W.awq_weights(N, K, 23 * M + N)
    x = W.activations(M, 2 * K, 29 * M + K, dtype=torch.float16, outliers=False)
    bias = (0.1 * torch.randn(N, generator=torch.Generator().manual_seed(M))).half()
    ref = (R.awq_gemm(x[:, :K], qw, qz, s, 128).float() + bias.float()).half()
    force_awq_plan(*plan)
    xd = x.to(cuda)[:, :K]
    assert xd.stride(0) == 2 * K
    args = (xd, qw.to(cuda), s.to(cuda), qz.to(cuda))
    out = awq_gemm_triton(*args, split_k_iters=8, bias=bias.to(cuda))
    assert out.shape == (M, N) and out.dtype == torch.float16
    assert rel_err(out, ref) <= REL_TOL, (plan, M, K, N)
    out2 = awq_gemm_triton(*args, split_k_iters=8, bias=bias.to(cuda))
    assert torch.equal(out, out2), "deterministic"


@pytest.mark.parametrize("M,K,N", [(4, 3584, 4608), (16, 18944, 3584), (48, 3584, 4608)])
def test_decode_kernel_in_a_hip_graph(cuda, M, K, N):
    """The few-token kernel ends its K split inside the launch with arrival tickets that return to zero; a captured
    launch replays on the counters of the workspace it was captured with.  Every replay, with fresh activations and
    eager calls on the same workspace in between (never at the same time), must reproduce the eager result bit for bit."""
    from llmqrt_amd import _abi, workloads as W
    L = _abi.lib()
    qw, qz, s = (t.to(cuda) for t in W.awq_weights(N, K, 77 + M))
    x = W.activations(M, K, 700, dtype=torch.float16, outliers=False).to(cuda)
    out = torch.empty((M, N), dtype=torch.float16, device=cuda)
    nws = L.llmq_awq_gemm_workspace_bytes(M, N, K)
    assert nws > 0, "the shapes are meant to exercise the K split"
    wsp = torch.zeros(nws, dtype=torch.uint8, device=cuda)   # the counters at its start are cleared once
    tb = L.llmq_awq_workspace_ticket_bytes()

    def run(stream):
        rc = L.llmq_awq_gemm(x.data_ptr(), K, qw.data_ptr(), s.data_ptr(), qz.data_ptr(), None, out.data_ptr(), M, N, K,
                             128, wsp.data_ptr(), nws, stream)
        assert rc == 0

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        run(side.cuda_stream)
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            run(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    main = torch.cuda.current_stream().cuda_stream
    for rep in range(4):
        x.copy_(W.activations(M, K, 710 + rep, dtype=torch.float16, outliers=False).to(cuda))
        run(main)
        torch.cuda.synchronize()
        eager = out.clone()
        out.zero_()
        wsp[tb:].fill_(0xFF)     # the contents behind the counters must not matter
        assert int(wsp[:tb].max()) == 0, "every call leaves the counters at zero"
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {rep}"
    ref = R.awq_gemm(x.cpu(), qw.cpu(), qz.cpu(), s.cpu(), 128)
    assert rel_err(out, ref) <= REL_TOL


def test_decode_kernel_on_two_streams_at_once(cuda):
    """Calls on different streams overlap on the GPU; each stream has its own workspace, hence its own arrival
    counters, so every result must equal the one computed alone however long the two streams run side by side."""
    from llmqrt_amd import _abi, workloads as W
    L = _abi.lib()
    K, N = 3584, 4608
    qw, qz, s = (t.to(cuda) for t in W.awq_weights(N, K, 91))
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    Ms = (4, 48)
    xs = [W.activations(M, K, 900 + i, dtype=torch.float16, outliers=False).to(cuda) for i, M in enumerate(Ms)]
    nws = [L.llmq_awq_gemm_workspace_bytes(M, N, K) for M in Ms]
    assert all(n > 0 for n in nws), "both shapes are meant to split K across blocks"
    wsp = [torch.zeros(n, dtype=torch.uint8, device=cuda) for n in nws]
    alone = []
    for i, M in enumerate(Ms):
        out = torch.empty((M, N), dtype=torch.float16, device=cuda)
        rc = L.llmq_awq_gemm(xs[i].data_ptr(), K, qw.data_ptr(), s.data_ptr(), qz.data_ptr(), None, out.data_ptr(), M, N, K,
                             128, wsp[i].data_ptr(), nws[i], torch.cuda.current_stream().cuda_stream)
        assert rc == 0
        torch.cuda.synchronize()
        alone.append(out)
    reps = 300
    outs = [[torch.empty((M, N), dtype=torch.float16, device=cuda) for _ in range(4)] for M in Ms]
    torch.cuda.synchronize()
    for r in range(reps):
        for i, M in enumerate(Ms):
            rc = L.llmq_awq_gemm(xs[i].data_ptr(), K, qw.data_ptr(), s.data_ptr(), qz.data_ptr(), None,
                                 outs[i][r % 4].data_ptr(), M, N, K, 128, wsp[i].data_ptr(), nws[i], streams[i].cuda_stream)
            assert rc == 0
        if r % 4 == 3:
            for st in streams:
                st.synchronize()
            for i in range(2):
                for o in outs[i]:
                    assert torch.equal(o, alone[i]), (r, i)
                    o.zero_()
    torch.cuda.synchronize()


def test_decode_kernel_extreme_nibbles_and_zero_tokens(cuda, force_awq_plan):
    """All-15 weights against zero points 0 and all-0 weights against zero points 15 (the largest |q - z|), and a
    token block whose rows past M must not leak into the result."""
    from llmqrt_amd.awq_kernels import awq_gemm_triton
    K, N, M = 256, 64, 5
    g = torch.Generator().manual_seed(5)
    x = torch.randn(M, K, generator=g).half()
    s = (torch.rand(K // 128, N, generator=g) * 0.02 + 0.001).half()
    for qv, zv in ((15, 0), (0, 15)):
        qw = R.awq_pack(torch.full((K, N), qv, dtype=torch.int32))
        qz = R.awq_pack(torch.full((K // 128, N), zv, dtype=torch.int32))
        ref = R.awq_gemm(x, qw, qz, s, 128)
        for variant in (8, 9):
            force_awq_plan(variant, 0)
            out = awq_gemm_triton(x.to(cuda), qw.to(cuda), s.to(cuda), qz.to(cuda), split_k_iters=8)
            assert rel_err(out, ref) <= REL_TOL, (qv, zv, variant)


@pytest.mark.parametrize("K,N,G", [(3584, 4608, 128), (896, 4864, 128), (256, 264, 64), (128, 8, 32), (512, 1000, 512),
                                   (8, 520, 8), (72, 40, 72)])
def test_dequant_transposed_bit_exact(cuda, K, N, G):
    """The transposed dequantizer (fp16 [N, K], the GEMM's weight operand): the oracle's dequantized matrix, transposed,
    bit for bit; K that is not a multiple of its 64-row tiles, N / 8 that is not a multiple of its 32-word tiles."""
    from llmqrt_amd import workloads as W
    from llmqrt_amd.awq_kernels import awq_dequantize_transposed
    qw, qz, s = W.awq_weights(N, K, K + N, group=G)
    ref = R.awq_dequantize(qw, qz, s, G)
    out = awq_dequantize_transposed(qw.to(cuda), s.to(cuda), qz.to(cuda))
    assert out.dtype == torch.float16 and out.shape == (N, K)
    assert torch.equal(out.cpu().view(torch.int16), ref.t().contiguous().view(torch.int16))


@pytest.mark.parametrize("M,K,N", [(1024, 3584, 4608), (300, 520, 1000), (65, 72, 40), (2048, 1024, 512), (1, 128, 8)])
def test_gemm_f16_against_fp64(cuda, M, K, N):
    """The fp16 MFMA GEMM (fp32 accumulation): raw accumulators against an fp64 product of the same fp16 operands, the
    fp16 output with and without bias; ragged M / N, K that is not a multiple of the K tile."""
    from llmqrt_amd.awq_kernels import gemm_f16
    g = torch.Generator().manual_seed(M + K + N)
    x = torch.randn(M, K, generator=g).half()
    w = (torch.randn(N, K, generator=g) * 0.05).half()
    bias = torch.randn(N, generator=g).half()
    ref = x.double() @ w.double().t()
    dump = torch.empty((M, N), dtype=torch.float32, device=cuda)
    y = gemm_f16(x.to(cuda), w.to(cuda), _acc_dump=dump)
    assert rel_err(dump, ref) <= 1e-5
    assert rel_err(y, ref) <= 1e-3
    yb = gemm_f16(x.to(cuda), w.to(cuda), bias.to(cuda))
    assert rel_err(yb, ref + bias.double()) <= 1e-3


def test_module_many_token_path_is_own_kernels(cuda):
    """Above its token threshold WQLinear_GEMM runs the transposed dequantizer and the fp16 MFMA GEMM of this library
    (no torch.matmul): output within tolerance of the oracle, with bias, 3-D input."""
    from llmqrt_amd import workloads as W
    from llmqrt_amd.linear import WQLinear_GEMM
    from llmqrt_amd.linear.linear_awq import dequant_matmul_token_threshold
    K, N = 1024, 1056
    qw, qz, s = W.awq_weights(N, K, 77)
    mod = WQLinear_GEMM(4, 128, K, N, True, cuda)
    mod.qweight.copy_(qw); mod.qzeros.copy_(qz); mod.scales.copy_(s)
    mod.bias.copy_((0.1 * torch.randn(N, generator=torch.Generator().manual_seed(3))).half())
    T = dequant_matmul_token_threshold(K, N) + 64
    x = W.activations(T, K, 78, dtype=torch.float16, outliers=False)
    ref = (R.awq_gemm(x, qw, qz, s, 128).float() + mod.bias.float().cpu()).half()
    real_matmul = torch.matmul
    try:
        def no_matmul(*a, **k):
            raise AssertionError("torch.matmul must not run on this path")
        torch.matmul = no_matmul
        y = mod(x.to(cuda).view(2, T // 2, K))
    finally:
        torch.matmul = real_matmul
    assert y.shape == (2, T // 2, N)
    assert rel_err(y.reshape(T, N), ref) <= REL_TOL
