"""Seeded random-shape sweeps over the dispatch of the GEMM entry points (GEMV, chunked GEMV, split
reduction with both tile heights, staged and weights-direct kernels, the int8 kernels): every shape
is checked against an fp32 product of the dequantised matrix on the GPU (lq_a16w4_dequant is itself
checked bit for bit against the CPU oracle elsewhere) and, for int8, against an exact integer product.
A hang in any configuration shows as a time-out of the case that names the shape."""
import random

import pytest
import torch

from tests.util import make_w4

pytestmark = pytest.mark.gpu

TOL = 5e-3  # bf16 output rounding gives ~1.7e-3


@pytest.fixture(scope="module")
def ops(hip_lib):
    assert torch.cuda.is_available()
    from latentq_llm_amd import ops
    return ops


def _shapes(seed, n, token_counts, n_choices, k_max):
    rng = random.Random(seed)
    out = []
    for _ in range(n):
        M = rng.choice(token_counts)
        N = rng.choice(n_choices) if rng.random() < 0.5 else 64 * rng.randint(1, 160)
        K = 128 * rng.randint(1, k_max)
        if N * K > 48e6:
            K = 128 * max(1, int(48e6 // N) // 128)
        out.append((M, N, K))
    return out


GEMM_SHAPES = _shapes(1, 40, [17, 33, 100, 128, 129, 250, 384, 511, 640, 777, 1024, 1500, 2050], [4096, 8192, 11008], 40)
GEMV_SHAPES = _shapes(2, 40, list(range(1, 17)), [64, 512, 4096, 8192, 8224, 11008], 96)


@pytest.mark.parametrize("M,N,K", GEMM_SHAPES + GEMV_SHAPES)
def test_forward_and_dx_random_shapes(ops, M, N, K):
    _, packed, scales, zeros = make_w4(N, K, M + N + K)
    w = (packed.cuda(), scales.cuda(), zeros.cuda())
    W = ops.a16w4_dequant(*w, (N, K)).float()
    g = torch.Generator(device="cuda").manual_seed(M * 7 + 1)
    x = torch.randn(M, K, device="cuda", generator=g).to(torch.bfloat16)
    bias = torch.randn(N, device="cuda", generator=g).to(torch.bfloat16) if (M + N) % 3 == 0 else None
    y = ops.a16w4_forward(x, *w, (N, K), bias=bias).float()
    ref = x.float() @ W.t() + (bias.float() if bias is not None else 0)
    assert ((y - ref).norm() / ref.norm()).item() < TOL
    if N % 64:
        return  # dX needs N % 64 == 0 (the forward pass N % 16)
    dy = torch.randn(M, N, device="cuda", generator=g).to(torch.bfloat16)
    dx = ops.a16w4_dx(dy, *w, (N, K)).float()
    ref = dy.float() @ W
    assert ((dx - ref).norm() / ref.norm()).item() < TOL


@pytest.mark.parametrize("M,N,K", _shapes(3, 24, [17, 100, 256, 300, 1024, 2048, 3000], [2048, 4096, 8192], 24))
def test_a8w8_random_shapes(ops, M, N, K):
    g = torch.Generator(device="cuda").manual_seed(M + N + K)
    x8 = torch.randint(-127, 128, (M, K), device="cuda", generator=g, dtype=torch.int8)
    w8 = torch.randint(-127, 128, (N, K), device="cuda", generator=g, dtype=torch.int8)
    sx = torch.rand(M, device="cuda", generator=g) + 0.1
    sw = torch.rand(N, device="cuda", generator=g) + 0.1
    y, acc = ops.a8w8_forward(x8, w8, sx, sw, want_acc=True)
    want = x8.double() @ w8.double().t()  # exact: |acc| < 2^31 << 2^53
    assert torch.equal(acc.double(), want)
    assert torch.equal(y, ((want.float() * sx[:, None]) * sw[None, :]).to(torch.bfloat16))


@pytest.mark.parametrize("M,N,K,bias", [(300, 11008, 256, False), (1000, 11024, 512, True), (768, 5504, 1024, False),
                                        (3072, 4096, 2048, True), (1536, 11008, 4096, False), (384, 11024, 4096, True)])
def test_forward_weights_direct_kernel_with_128x128_tiles(ops, M, N, K, bias):
    """Shapes the planner gives to the weights-direct kernel with 128 x 128 tiles (between one and two rounds of
    its 128 x 256 tiles): ragged token counts, a last tile of 16 columns (N = 11024), 4 to 64 reduction steps,
    with and without bias, against the fp32 product of the dequantised matrix."""
    assert ops.a16w4_plan(M, (N, K))[0] == "direct_128x128"
    _, packed, scales, zeros = make_w4(N, K, M + N + K)
    w = (packed.cuda(), scales.cuda(), zeros.cuda())
    W = ops.a16w4_dequant(*w, (N, K)).float()
    g = torch.Generator(device="cuda").manual_seed(M + 3)
    x = torch.randn(M, K, device="cuda", generator=g).to(torch.bfloat16)
    b = torch.randn(N, device="cuda", generator=g).to(torch.bfloat16) if bias else None
    y = ops.a16w4_forward(x, *w, (N, K), bias=b).float()
    ref = x.float() @ W.t() + (b.float() if bias else 0)
    assert ((y - ref).norm() / ref.norm()).item() < TOL


def test_forward_128x128_direct_kernel_identity_is_exact_dequant(ops):
    """X = identity through the 128 x 128 weights-direct kernel: every output is one dequantised weight, bit for bit."""
    N, K = 11008, 1024
    M = K
    assert ops.a16w4_plan(M, (N, K))[0] == "direct_128x128"
    _, packed, scales, zeros = make_w4(N, K, 31)
    w = (packed.cuda(), scales.cuda(), zeros.cuda())
    x = torch.eye(K, device="cuda", dtype=torch.bfloat16)
    y = ops.a16w4_forward(x, *w, (N, K))
    assert torch.equal(y, ops.a16w4_dequant(*w, (N, K)).t().contiguous())


def _dw_shapes(seed, n):
    rng = random.Random(seed)
    out = []
    for _ in range(n):
        M = 64 * rng.randint(1, 40)
        N = 8 * rng.randint(1, 700) if rng.random() < 0.6 else rng.choice([256, 4096, 11008])
        K = 16 * rng.randint(1, 300) if rng.random() < 0.6 else rng.choice([256, 4096, 11008])
        if N * K > 24e6:
            K = 16 * max(1, int(24e6 // N) // 16)
        out.append((M, N, K))
    return out


@pytest.mark.parametrize("M,N,K", _dw_shapes(5, 24))
def test_weight_grad_random_shapes(ops, M, N, K):
    """dW = dY^T X over random shapes (partial tiles along both output dimensions, 1 to 40 reduction steps) against
    the fp32 product on the GPU; the int8 accumulate epilogue against the stand-alone pass on the stored product."""
    g = torch.Generator(device="cuda").manual_seed(M + N + K)
    dy = (torch.randn(M, N, device="cuda", generator=g) * 0.05).to(torch.bfloat16)
    x = torch.randn(M, K, device="cuda", generator=g).to(torch.bfloat16)
    dw = ops.weight_grad(dy, x)
    ref = dy.float().t() @ x.float()
    assert ((dw.float() - ref).norm() / ref.norm()).item() < TOL
    q = torch.randint(-100, 100, (N, K), device="cuda", generator=g, dtype=torch.int8)
    s = (torch.rand(N, 1, device="cuda", generator=g) * 0.01 + 1e-3).to(torch.bfloat16)
    q2 = q.clone()
    ops.weight_grad_acc8(dy, x, q, s, seed=3, offset=M)
    ops.gradq8_quant(dw, q2, s, True, seed=3, offset=M)
    assert torch.equal(q, q2)


@pytest.mark.parametrize("M,N,K", _shapes(7, 16, [17, 100, 256, 300, 1024, 2050], [4096, 8192, 11008], 24))
def test_dx_epilogues_and_int8_dx_random_shapes(ops, M, N, K):
    """The accumulate and SiLU-backward epilogues of the dX kernel, two products in one reduction, and the dX from int8
    codes over random shapes."""
    if N % 64:
        N = (N // 64 + 1) * 64
    _, packed, scales, zeros = make_w4(N, K, M + N + K)
    w = (packed.cuda(), scales.cuda(), zeros.cuda())
    g = torch.Generator(device="cuda").manual_seed(M * 3 + 2)
    dy = torch.randn(M, N, device="cuda", generator=g).to(torch.bfloat16)
    base = torch.randn(M, K, device="cuda", generator=g).to(torch.bfloat16)
    W = ops.a16w4_dequant(*w, (N, K)).float()
    ref = dy.float() @ W
    acc = base.clone()
    ops.a16w4_dx(dy, *w, (N, K), out=acc, accumulate=True)
    want = base.float() + ref
    assert ((acc.float() - want).norm() / want.norm()).item() < TOL
    gg = torch.randn(M, K, device="cuda", generator=g).to(torch.bfloat16)
    uu = torch.randn(M, K, device="cuda", generator=g).to(torch.bfloat16)
    dg, du = ops.a16w4_dx_silu_bwd(dy, *w, (N, K), gg, uu)
    sg = torch.sigmoid(gg.float())
    for got, wnt in ((dg, ref * uu.float() * sg * (1 + gg.float() * (1 - sg))), (du, ref * gg.float() * sg)):
        assert ((got.float() - wnt).norm() / wnt.norm()).item() < 2 * TOL
    _, packed2, scales2, zeros2 = make_w4(N, K, M + N + K + 1)
    w2 = (packed2.cuda(), scales2.cuda(), zeros2.cuda())
    dy2 = torch.randn(M, N, device="cuda", generator=g).to(torch.bfloat16)
    pair = ops.a16w4_dx_pair(dy, w, dy2, w2, (N, K))
    want = ref + dy2.float() @ ops.a16w4_dequant(*w2, (N, K)).float()
    assert ((pair.float() - want).norm() / want.norm()).item() < TOL
    w8 = torch.randint(-128, 128, (N, K), device="cuda", generator=g, dtype=torch.int8)
    qs = (torch.rand(N, device="cuda", generator=g) * 0.01 + 1e-3).to(torch.bfloat16)
    dx8 = ops.a8w8_dx(dy, w8, qs)
    ref8 = dy.float() @ (w8.to(torch.bfloat16) * qs[:, None]).to(torch.bfloat16).float()
    assert ((dx8.float() - ref8).norm() / ref8.norm()).item() < TOL
