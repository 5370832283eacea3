"""GPU parity tests: every kernel is called through the C ABI (latentq_llm_amd.ops -> ctypes ->
liblatentq_hip.so) and compared with the CPU oracle on the same seeded inputs.

Bars: bit-exact for codes, int32 accumulators, Philox draws, int8 activations and layout
converters; rel-L2 <= 1e-2 (max-abs printed) for bf16 GEMM/GEMV outputs.
"""
import numpy as np
import pytest
import torch

from tests import util
from tests.util import bits, from_bits, make_w4, randn_bf16, rel_l2

pytestmark = pytest.mark.gpu

REL_L2_TOL = 1e-2


@pytest.fixture(scope="module")
def ops(hip_lib):
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from latentq_llm_amd import ops as _ops
    return _ops


@pytest.fixture(scope="module")
def co():
    from oracle import c_oracle
    return c_oracle


def bits_t(t):
    return t.detach().cpu().contiguous().view(torch.int16)


def dev(t):
    return t.cuda()


# ------------------------------------------------------------------ Philox --
@pytest.mark.parametrize("n,seed,offset", [(1, 0, 0), (7, 1, 0), (4096, 0xDEADBEEFCAFEF00D, 12345),
                                           (1000003, 42, 2**32 - 5), (64, 7, 2**64 - 3)])
def test_philox_uniform_bit_exact(ops, co, n, seed, offset):
    got = ops.philox_uniform(n, seed, offset).cpu().numpy()
    want = co.philox_uniform(n, seed, offset)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert got.min() >= 0.0 and got.max() < 1.0


# ----------------------------------------------------------------- requant --
def _requant_case(ops, co, N, K, seed, lr, gstd, mode, tweak=None):
    codes, packed, scales, zeros = make_w4(N, K, seed)
    grad = randn_bf16((N, K), seed + 1, gstd)
    if tweak:
        scales, zeros, grad = tweak(scales, zeros, grad)
    pseed, poff = 0x1234567 + seed, 1000 * seed
    if mode == "inject":
        g = torch.Generator().manual_seed(seed + 2)
        u = torch.rand((N, K), generator=g, dtype=torch.float32)
        want = co.requant(packed.numpy(), bits(scales), bits(zeros), bits(grad), lr, N, K, u=u.numpy())
        got = ops.requant_sr(dev(packed), dev(scales), dev(zeros), dev(grad), lr, (N, K), u=dev(u))
    else:
        want = co.requant(packed.numpy(), bits(scales), bits(zeros), bits(grad), lr, N, K, seed=pseed, offset=poff)
        got = ops.requant_sr(dev(packed), dev(scales), dev(zeros), dev(grad), lr, (N, K), seed=pseed, offset=poff)
    got = got.cpu().numpy().view(np.uint8)
    mism = int((got != want).sum())
    assert mism == 0, f"{mism} of {want.size} bytes differ"
    return got, packed.numpy().view(np.uint8)


@pytest.mark.parametrize("mode", ["inject", "philox"])
@pytest.mark.parametrize("N,K", [(1, 128), (3, 384), (64, 256), (257, 1024), (1000, 128)])
def test_requant_bit_exact_small(ops, co, N, K, mode):
    _requant_case(ops, co, N, K, seed=N + K, lr=1e-4, gstd=1e-3, mode=mode)


@pytest.mark.parametrize("mode", ["inject", "philox"])
def test_requant_bit_exact_large_update(ops, co, mode):
    # updates of the order of a code step, so that many codes actually move
    got, old = _requant_case(ops, co, 128, 512, seed=5, lr=1.0, gstd=2e-3, mode=mode)
    assert (got != old).mean() > 0.2


@pytest.mark.parametrize("mode", ["inject", "philox"])
def test_requant_edge_parameters(ops, co, mode):
    """Non-integer / large zeros, zero, negative, tiny and huge scales, inf/nan/huge gradients."""
    def tweak(scales, zeros, grad):
        s = scales.clone().reshape(-1)
        z = zeros.clone().reshape(-1)
        g = grad.clone()
        special_s = [0.0, -0.003, 2.0 ** -60, 2.0 ** 60, 2.0 ** -120, 3e38, float("inf"), 1.0]
        special_z = [7.5, 6.28125, 300.0, -3.0, 0.0, 15.0, 241.0, 1e6]
        for i, v in enumerate(special_s):
            s[i::17][: 4] = v
        for i, v in enumerate(special_z):
            z[3 + i::13][: 4] = v
        flat = g.reshape(-1)
        flat[5::97] = float("inf")
        flat[11::89] = float("-inf")
        flat[17::83] = float("nan")
        flat[23::79] = 3e38
        flat[29::73] = -3e38
        flat[31::71] = 0.0
        return s.reshape(scales.shape), z.reshape(zeros.shape), g
    _requant_case(ops, co, 96, 512, seed=9, lr=0.5, gstd=1e-2, mode=mode, tweak=tweak)


def test_requant_in_place_and_properties(ops, co):
    """codes_out may alias codes_in; g = 0, u = 0.5 leaves codes unchanged; huge |g| saturates."""
    N, K = 64, 512
    codes, packed, scales, zeros = make_w4(N, K, 3)
    d = [dev(t) for t in (packed, scales, zeros)]
    zero_g = torch.zeros((N, K), dtype=torch.bfloat16, device="cuda")
    half = torch.full((N, K), 0.5, dtype=torch.float32, device="cuda")
    buf = d[0].clone()
    ops.requant_sr(buf, d[1], d[2], zero_g, 1e-4, (N, K), u=half, out=buf)
    assert torch.equal(buf, d[0])
    big = torch.full((N, K), 1e30, dtype=torch.bfloat16, device="cuda")
    lo = ops.requant_sr(d[0], d[1], d[2], big, 1.0, (N, K), u=half)
    hi = ops.requant_sr(d[0], d[1], d[2], -big, 1.0, (N, K), u=half)
    assert torch.all(lo.view(torch.uint8) == 0) and torch.all(hi.view(torch.uint8) == 0xFF)


def test_requant_full_size_properties(ops, co):
    """Benchmark size (8192 x 2048): Philox mode equals injected mode fed with the materialised
    stream, idempotence at g = 0 / u = 0.5, and a sampled bit-exact comparison with the oracle."""
    N, K = 8192, 2048
    codes, packed, scales, zeros = make_w4(N, K, 11)
    grad = randn_bf16((N, K), 12, 1e-3)
    dp, ds, dz, dg = dev(packed), dev(scales), dev(zeros), dev(grad)
    seed, off = 2024, 77
    a = ops.requant_sr(dp, ds, dz, dg, 1e-4, (N, K), seed=seed, offset=off)
    u = ops.philox_uniform(N * K, seed, off)
    b = ops.requant_sr(dp, ds, dz, dg, 1e-4, (N, K), u=u)
    assert torch.equal(a, b)
    rows = 64  # oracle on a slice of rows (the update is row-local)
    want = co.requant(packed[: rows * K // 2].numpy(), bits(scales[: rows * K // 128]), bits(zeros[: rows * K // 128]),
                      bits(grad[:rows]), 1e-4, rows, K, seed=seed, offset=off)
    assert np.array_equal(a[: rows * K // 2].cpu().numpy().view(np.uint8), want)
    half = torch.full((N, K), 0.5, dtype=torch.float32, device="cuda")
    same = ops.requant_sr(dp, ds, dz, torch.zeros_like(dg), 1e-4, (N, K), u=half)
    assert torch.equal(same, dp)


# ----------------------------------------------------------------- dequant --
@pytest.mark.parametrize("N,K", [(16, 128), (48, 384), (300, 1024)])
def test_dequant_bit_exact(ops, co, N, K):
    codes, packed, scales, zeros = make_w4(N, K, N)
    zeros.view(-1)[::5] = 7.5  # exercise the bf16 rounding of (q - z)
    want = co.dequant(packed.numpy(), bits(scales), bits(zeros), N, K)
    got = bits(ops.a16w4_dequant(dev(packed), dev(scales), dev(zeros), (N, K)))
    assert np.array_equal(got, want)


# --------------------------------------------------------------- A16W4 fwd --
def _fwd_case(ops, co, M, N, K, seed, with_bias):
    codes, packed, scales, zeros = make_w4(N, K, seed)
    x = randn_bf16((M, K), seed + 1)
    bias = randn_bf16((N,), seed + 2) if with_bias else None
    _, want64 = co.a16w4_fwd(bits(x), packed.numpy(), bits(scales), bits(zeros), None if bias is None else bits(bias),
                             M, N, K, want_f64=True)
    got = ops.a16w4_forward(dev(x), dev(packed), dev(scales), dev(zeros), (N, K), None if bias is None else dev(bias))
    torch.cuda.synchronize()
    got = got.float().cpu()
    want = torch.from_numpy(want64)
    err = rel_l2(got, want)
    print(f"fwd M={M} N={N} K={K} rel_l2={err:.3e} max_abs={float((got.double() - want).abs().max()):.3e}")
    assert err <= REL_L2_TOL
    return err


@pytest.mark.parametrize("M,N,K,bias", [(17, 16, 128, False), (33, 48, 256, True), (128, 128, 128, False),
                                        (129, 256, 384, True), (300, 272, 512, False), (1024, 3072, 768, True),
                                        # ragged in M and N on large grids: odd group counts (staged kernel) ...
                                        (4100, 4112, 128, True), (3000, 6160, 384, False),
                                        # ... and even ones (weights-direct kernel): 4, 12 and 20 steps, i.e. one
                                        # partial quad of scales, one and a half, and two and a half
                                        (4100, 4112, 256, True), (3000, 6160, 768, False), (2100, 4112, 1280, True)])
def test_a16w4_fwd_gemm(ops, co, M, N, K, bias):
    _fwd_case(ops, co, M, N, K, seed=M + N + K, with_bias=bias)


@pytest.mark.parametrize("M,N,K,bias", [(17, 4096, 4096, True), (32, 11008, 4096, False), (37, 1024, 11008, True)])
def test_a16w4_fwd_a_few_more_tokens_than_one_gemv(ops, co, M, N, K, bias):
    """17..64 tokens on matrices large enough that chunks of 16 through the GEMV beat the GEMM."""
    _fwd_case(ops, co, M, N, K, seed=M + N + K, with_bias=bias)


@pytest.mark.parametrize("M", [1, 2, 4, 5, 16])
@pytest.mark.parametrize("N,K,bias", [(16, 128, False), (64, 640, True), (4096, 4096, False), (256, 11008, True)])
def test_a16w4_fwd_gemv(ops, co, M, N, K, bias):
    _fwd_case(ops, co, M, N, K, seed=M + N + K, with_bias=bias)


@pytest.mark.parametrize("M,N,K", [(16, 8192, 1536), (9, 8224, 1152), (16, 8192, 2560), (12, 512, 5120), (16, 8192, 640)])
def test_a16w4_fwd_gemv_many_tokens_staged_scales(ops, co, M, N, K):
    """5..16 tokens with the scales and zeros of a workgroup's rows staged through LDS: 32-row workgroups
    on tall matrices (also with a wave that has no batch of its own: 3 and 5 batches on 4 waves), several
    batches per wave on 8 waves, padded (K = 2560, 5120: 80- and 160-byte rows) and unpadded rows."""
    _fwd_case(ops, co, M, N, K, seed=M + N + K, with_bias=(M % 2 == 0))


def test_gemv_and_gemm_agree_on_the_same_tokens_within_the_documented_bound(ops, co):
    """Up to 16 tokens take the GEMV, which multiplies s * sum((q - z) x) in fp32; more tokens take kernels that
    round the dequantised weight to bf16 first, as the reference does. The same token therefore gets slightly
    different outputs depending on how many tokens ride along: at most 2^-9 relative per weight, i.e. well
    inside the parity bar. Measured here between M = 16 (GEMV), M = 17 (GEMV chunks or GEMM) and M = 256 (GEMM)."""
    N, K = 4096, 4096
    codes, packed, scales, zeros = make_w4(N, K, 77)
    x = randn_bf16((256, K), 78)
    w = (dev(packed), dev(scales), dev(zeros))
    xd = dev(x)
    y16 = ops.a16w4_forward(xd[:16].contiguous(), *w, (N, K)).float()
    y17 = ops.a16w4_forward(xd[:17].contiguous(), *w, (N, K)).float()[:16]
    y256 = ops.a16w4_forward(xd, *w, (N, K)).float()[:16]
    _, want64 = co.a16w4_fwd(bits(x[:16]), packed.numpy(), bits(scales), bits(zeros), None, 16, N, K, want_f64=True)
    want = torch.from_numpy(want64)
    for name, y in (("M=16", y16), ("M=17", y17), ("M=256", y256)):
        print(f"{name}: rel_l2 vs float64 {rel_l2(y.cpu(), want):.3e}")
    d = rel_l2(y16, y256)
    print(f"GEMV(16) vs GEMM(256) on the same 16 tokens: rel_l2 {d:.3e}, max abs {float((y16 - y256).abs().max()):.3e}; "
          f"M=17 vs M=256: {rel_l2(y17, y256):.3e}")
    assert 0 < d <= 5e-3 and rel_l2(y17, y256) <= 5e-3
    # the output scale is |y| ~ sqrt(K) * |w| ~ 0.1: no element moves by more than a few bf16 ulps of that
    assert float((y16 - y256).abs().max()) <= 2.0 ** -7 * float(y256.abs().max())


@pytest.mark.parametrize("M,N,K", [(1, 64, 640), (4, 4096, 4096), (16, 8192, 1536), (17, 16, 128), (300, 272, 512),
                                   (2048, 512, 512)])
def test_scales_and_zeros_need_only_2_byte_alignment(ops, co, M, N, K):
    """Scales and zeros handed over at an address that is 2 bytes past a 256-byte boundary (a view into a larger
    checkpoint tensor): forward (GEMV, staged and weights-direct GEMM), dX, dequant and the requantizer give
    the same bits as with aligned copies."""
    codes, packed, scales, zeros = make_w4(N, K, M + N + K)
    x = dev(randn_bf16((M, K), 5))
    dy = dev(randn_bf16((M, N), 6))
    grad = dev(randn_bf16((N, K), 7, 1e-2))
    G = N * K // 128
    hold_s = torch.zeros(G + 1, 1, dtype=torch.bfloat16, device="cuda")
    hold_z = torch.zeros(G + 1, 1, dtype=torch.bfloat16, device="cuda")
    s_off, z_off = hold_s[1:], hold_z[1:]
    s_off.copy_(scales)
    z_off.copy_(zeros)
    assert s_off.data_ptr() % 4 == 2 and z_off.data_ptr() % 4 == 2
    p, s_al, z_al = dev(packed), dev(scales), dev(zeros)
    assert torch.equal(ops.a16w4_forward(x, p, s_off, z_off, (N, K)), ops.a16w4_forward(x, p, s_al, z_al, (N, K)))
    assert torch.equal(ops.a16w4_dequant(p, s_off, z_off, (N, K)), ops.a16w4_dequant(p, s_al, z_al, (N, K)))
    if N % 64 == 0:
        assert torch.equal(ops.a16w4_dx(dy, p, s_off, z_off, (N, K)), ops.a16w4_dx(dy, p, s_al, z_al, (N, K)))
    a = ops.requant_sr(p, s_off, z_off, grad, 1e-2, (N, K), seed=3, offset=9)
    b = ops.requant_sr(p, s_al, z_al, grad, 1e-2, (N, K), seed=3, offset=9)
    assert torch.equal(a, b)


def test_a16w4_fwd_identity_is_exact_dequant(ops, co):
    """X = identity: every output is a single dequantised weight, so the GEMM result must equal
    the reference dequantisation bit for bit (checks unpack + bf16 rounding through the kernel)."""
    N, K = 384, 256
    codes, packed, scales, zeros = make_w4(N, K, 21)
    x = torch.eye(K, dtype=torch.bfloat16)
    got = ops.a16w4_forward(dev(x), dev(packed), dev(scales), dev(zeros), (N, K))
    want = co.dequant(packed.numpy(), bits(scales), bits(zeros), N, K)  # [N, K]
    assert np.array_equal(bits(got).T, want)


def test_a16w4_fwd_identity_is_exact_dequant_direct_kernel(ops, co):
    """The same on a grid of 16 x 16 tiles, which runs the weights-direct kernel (half-integer zeros
    included: q - z stays exact in bf16, so the reference's two roundings and the kernel's one agree)."""
    N, K = 4096, 2048
    codes, packed, scales, zeros = make_w4(N, K, 22)
    zeros.view(-1)[::7] = 7.5
    x = torch.eye(K, dtype=torch.bfloat16)
    got = ops.a16w4_forward(dev(x), dev(packed), dev(scales), dev(zeros), (N, K))
    want = co.dequant(packed.numpy(), bits(scales), bits(zeros), N, K)  # [N, K]
    assert int((bits(got).T != want).sum()) == 0


def test_a16w4_fwd_integer_exact(ops, co):
    """scales = 1, zeros = 0, small-integer X: the result is an exact small integer... in fp32;
    checks the full contraction (every k reaches the right accumulator) without tolerance
    as long as the sums stay below 2^8 (bf16-exact)."""
    M, N, K = 64, 32, 128
    g = torch.Generator().manual_seed(5)
    codes = torch.randint(0, 2, (N, K), generator=g, dtype=torch.uint8)
    packed = util.pack_codes(codes)
    scales = torch.ones(N * K // 128, 1, dtype=torch.bfloat16)
    zeros = torch.zeros(N * K // 128, 1, dtype=torch.bfloat16)
    x = torch.randint(-1, 2, (M, K), generator=g).to(torch.bfloat16)
    got = ops.a16w4_forward(dev(x), dev(packed), dev(scales), dev(zeros), (N, K)).float().cpu()
    want = x.float() @ codes.float().t()
    assert want.abs().max() < 256
    assert torch.equal(got, want)


@pytest.mark.parametrize("N,K", [(64, 256), (256, 4096), (8224, 1024), (512, 11008), (11008, 512)])
@pytest.mark.parametrize("M", [1, 3, 4, 7, 8, 13, 16])
def test_gemv_one_hot_tokens_give_the_exact_dequantised_weights(ops, co, N, K, M):
    """Decode path at bit level: token m is one-hot at a column k_m, so y[m, n] = s (P - (128 + z) S) with
    P = 128 + q and S = 1, i.e. s (q - z) formed exactly in fp32 and rounded once: the reference's dequantised weight
    W[n, k_m] bit for bit (integer zeros). Shapes and token counts walk through every GEMV configuration (2 to 16
    waves, 4 / 8 / 16 staged rows, one and two row tiles, scales through LDS, tail batches of fewer than 4 groups)."""
    codes, packed, scales, zeros = make_w4(N, K, N + K + M)
    ks = [(37 * m + 5) * 131 % K for m in range(M)]
    ks[0], ks[-1] = (0, K - 1) if M > 1 else (K - 1, K - 1)
    x = torch.zeros((M, K), dtype=torch.bfloat16)
    for m, k in enumerate(ks):
        x[m, k] = 1.0
    got = ops.a16w4_forward(dev(x), dev(packed), dev(scales), dev(zeros), (N, K))
    want = co.dequant(packed.numpy(), bits(scales), bits(zeros), N, K)  # [N, K] bf16 bits
    for m, k in enumerate(ks):
        assert np.array_equal(bits(got[m]), want[:, k]), (m, k)


@pytest.mark.parametrize("M,N,K", [(1, 256, 4096), (4, 512, 1024), (8, 8224, 512), (16, 256, 11008), (16, 8224, 384)])
def test_gemv_integer_exact(ops, M, N, K):
    """Power-of-two scales, integer zeros and small-integer activations: every partial sum of the decode kernel is
    exact in fp32, so the output equals the exact product (which bf16 holds) whatever the order of summation."""
    g = torch.Generator().manual_seed(M + N + K)
    codes = torch.randint(0, 16, (N, K), generator=g, dtype=torch.uint8)
    packed = util.pack_codes(codes)
    G = N * K // 128
    scales = torch.tensor([2.0 ** -(i % 2) for i in range(G)], dtype=torch.bfloat16).reshape(G, 1)
    zeros = torch.randint(6, 10, (G, 1), generator=g).to(torch.bfloat16)
    x = torch.zeros((M, K), dtype=torch.bfloat16)
    nz = torch.randint(0, K, (M, 12), generator=g)
    for m in range(M):
        x[m, nz[m]] = (2 * torch.randint(0, 2, (12,), generator=g) - 1).to(torch.bfloat16)  # |sum| <= 12 * 9, steps of 1/2
    got = ops.a16w4_forward(dev(x), dev(packed), dev(scales), dev(zeros), (N, K)).cpu()
    W = (codes.double().reshape(G, 128) - zeros.double()) * scales.double()
    want = x.double() @ W.reshape(N, K).t()
    assert float(want.abs().max()) < 128 and torch.equal(want, want.to(torch.bfloat16).double())
    assert torch.equal(got.double(), want)


# ---------------------------------------------------------------- A16W4 dX --
@pytest.mark.parametrize("M,N,K", [(17, 64, 128), (64, 128, 256), (130, 192, 384), (300, 320, 512), (1024, 3072, 768),
                                   (4, 128, 256)])
def test_a16w4_dx(ops, co, M, N, K):
    codes, packed, scales, zeros = make_w4(N, K, M + N)
    dy = randn_bf16((M, N), 7)
    _, want64 = co.a16w4_dx(bits(dy), packed.numpy(), bits(scales), bits(zeros), M, N, K, want_f64=True)
    got = ops.a16w4_dx(dev(dy), dev(packed), dev(scales), dev(zeros), (N, K)).float().cpu()
    want = torch.from_numpy(want64)
    err = rel_l2(got, want)
    print(f"dx M={M} N={N} K={K} rel_l2={err:.3e} max_abs={float((got.double() - want).abs().max()):.3e}")
    assert err <= REL_L2_TOL


def test_a16w4_dx_identity_is_exact_dequant(ops, co):
    N, K = 256, 384
    codes, packed, scales, zeros = make_w4(N, K, 22)
    dy = torch.eye(N, dtype=torch.bfloat16)
    got = ops.a16w4_dx(dev(dy), dev(packed), dev(scales), dev(zeros), (N, K))
    want = co.dequant(packed.numpy(), bits(scales), bits(zeros), N, K)
    assert np.array_equal(bits(got), want)


def test_a16w4_adjoint_identity(ops):
    """<X W^T, dY> == <X, dY W> up to bf16 output rounding, at the OPT-125m fc1 shape."""
    M, N, K = 1024, 3072, 768
    codes, packed, scales, zeros = make_w4(N, K, 31)
    x, dy = randn_bf16((M, K), 32), randn_bf16((M, N), 33)
    dp, ds, dz = dev(packed), dev(scales), dev(zeros)
    y = ops.a16w4_forward(dev(x), dp, ds, dz, (N, K)).double().cpu()
    dx = ops.a16w4_dx(dev(dy), dp, ds, dz, (N, K)).double().cpu()
    lhs = float((y * dy.double()).sum())
    rhs = float((x.double() * dx).sum())
    scale = float(y.norm() * dy.double().norm())
    assert abs(lhs - rhs) <= 1e-3 * scale


# -------------------------------------------------------------------- A8W8 --
@pytest.mark.parametrize("M,N,K,bias", [(17, 16, 128, False), (64, 128, 256, True), (130, 272, 384, False),
                                        (300, 512, 1024, True), (2048, 2048, 2048, False),
                                        # ragged and large enough for the weights-direct kernel; odd number of K steps
                                        (4100, 4112, 384, True),
                                        # one and two K steps through the 256 x 256 tile kernel
                                        (3600, 3648, 128, False), (3330, 3840, 256, True),
                                        # long reductions on small outputs: four stages, 49 / 50 / 51 / 52 steps
                                        (300, 512, 6272, True), (129, 256, 6400, False), (520, 1040, 6528, True),
                                        (64, 128, 6656, False)])
def test_a8w8(ops, co, M, N, K, bias):
    g = torch.Generator().manual_seed(M + N + K)
    x8 = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int8)
    w8 = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8)
    sx = (torch.randn(M, generator=g) * 0.05).abs() + 1e-4
    sw = (torch.randn(N, generator=g) * 0.01).abs() + 1e-5
    b = randn_bf16((N,), 3) if bias else None
    want_y, want_acc = co.a8w8(x8.numpy(), w8.numpy(), sx.numpy(), sw.numpy(), None if b is None else bits(b), M, N, K)
    y, acc = ops.a8w8_forward(dev(x8), dev(w8), dev(sx), dev(sw), None if b is None else dev(b), want_acc=True)
    assert np.array_equal(acc.cpu().numpy(), want_acc), "int32 accumulators must be bit-exact"
    err = rel_l2(y.float().cpu(), from_bits(want_y).float())
    print(f"a8w8 M={M} N={N} K={K} rel_l2={err:.3e}")
    assert err <= REL_L2_TOL
    # the fused epilogue is deterministic fp32 arithmetic: it matches the oracle bit for bit as well
    assert np.array_equal(bits(y), want_y)


def test_a8w8_extreme_accumulators(ops, co):
    """All +-127 over K = 8192: |acc| = 127*127*8192 = 132 128 768 < 2^31."""
    M, N, K = 32, 32, 8192
    x8 = torch.full((M, K), 127, dtype=torch.int8)
    w8 = torch.full((N, K), -127, dtype=torch.int8)
    w8[::2] = 127
    one = torch.ones(M), torch.ones(N)
    _, acc = ops.a8w8_forward(dev(x8), dev(w8), dev(one[0]), dev(one[1]), want_acc=True)
    acc = acc.cpu()
    assert int(acc[0, 0]) == 127 * 127 * 8192 and int(acc[0, 1]) == -127 * 127 * 8192


@pytest.mark.parametrize("shape,clamp", [((333, 77), None), ((2048, 1024), None), ((64, 128), 3.14159), ((64, 128), 1e-30),
                                         ((64, 128), -2.0), ((40, 8), 0.0)])
def test_act_quant_bit_exact(ops, co, shape, clamp):
    """The tensor's own maximum as clamp value (a bf16 number: the reciprocal-product form), clamp values that are not
    bf16 numbers, tiny, negative or zero (the division form), with NaN and infinities among the inputs."""
    x = randn_bf16(shape, 1, 2.0)
    clampv = float(x.max()) if clamp is None else clamp
    x.view(-1)[5] = float("nan")
    x.view(-1)[17] = float("inf")
    x.view(-1)[18] = float("-inf")
    x.view(-1)[19] = 3e38
    got = ops.act_quant_i8(dev(x), torch.tensor([clampv], device="cuda")).cpu().numpy()
    want = co.act_quant_i8(bits(x), clampv).reshape(got.shape)
    assert np.array_equal(got, want), np.nonzero(got != want)[0][:10]


@pytest.mark.parametrize("shape", [(333, 77), (2048, 1024), (1, 8), (7, 3), (2048, 8192)])
@pytest.mark.parametrize("alpha_bf16", [False, True])
def test_act_quant_dynamic_bit_exact(ops, co, shape, alpha_bf16):
    """clampv = the tensor's own maximum found on the device: int8 values, clamp value, alpha and the per-row
    scale vector against the oracle, bit for bit."""
    M, K = shape
    x = randn_bf16(shape, 21 + M, 2.0)
    got8, gsx, work = ops.act_quant_i8_dynamic(dev(x), alpha_bf16)
    want8, wsx, cv, alpha = co.act_quant_i8_dynamic(bits(x), M, K, alpha_bf16)
    assert np.array_equal(got8.cpu().numpy().reshape(-1), want8)
    w = work.cpu().numpy()
    assert w[0] == cv == float(x.max()) and w[1] == alpha
    assert np.array_equal(gsx.cpu().numpy().view(np.uint32), wsx.view(np.uint32))


def test_act_quant_dynamic_edge_values(ops, co):
    """All-negative tensors (max is the element nearest zero), infinities, and a NaN (NaN clamp, all zeros)."""
    M, K = 64, 136
    x = -randn_bf16((M, K), 5).abs() - 0.5
    for tweak in (None, ("inf", float("inf")), ("ninf", float("-inf")), ("nan", float("nan"))):
        xx = x.clone()
        if tweak:
            xx.view(-1)[1234] = tweak[1]
        got8, gsx, work = ops.act_quant_i8_dynamic(dev(xx), True)
        want8, wsx, cv, alpha = co.act_quant_i8_dynamic(bits(xx), M, K, True)
        assert np.array_equal(got8.cpu().numpy().reshape(-1), want8), tweak
        w = work.cpu().numpy()[:2]
        assert np.array_equal(w.view(np.uint32) & 0x7FFFFFFF, np.array([cv, alpha], np.float32).view(np.uint32) & 0x7FFFFFFF) \
            or (np.isnan(w).all() and np.isnan(cv) and np.isnan(alpha)), tweak
        assert np.array_equal(np.isnan(gsx.cpu().numpy()), np.isnan(wsx))


@pytest.mark.parametrize("shape", [(5, 8), (333, 72), (2048, 2048), (2048, 8192), (64, 8200), (3, 16392)])
def test_act_quant_per_token_bit_exact(ops, co, shape):
    """One scale per token row: int8 values and scales against the oracle bit for bit, with an all-zero row, a NaN,
    an infinity, a tiny row and rows of rounding ties among the inputs; row lengths on both sides of what a wave
    keeps in registers."""
    M, K = shape
    x = randn_bf16(shape, 31 + M, 3.0)
    x[0] = 0
    if M > 4:
        x[1, 5] = float("nan")
        x[2, 1] = float("inf")
        x[3] *= 1e-30
        x[4, :] = 127.0
        x[4, 3] = -63.5
        x[4, K - 1] = 0.5
    got8, gsx = ops.act_quant_i8_per_token(dev(x))
    want8, wsx = co.act_quant_i8_per_token(bits(x), M, K)
    assert np.array_equal(gsx.cpu().numpy().view(np.uint32) , wsx.view(np.uint32))
    g = got8.cpu().numpy().reshape(-1)
    assert np.array_equal(g, want8), np.nonzero(g != want8)[0][:10]


@pytest.mark.parametrize("shape", [(1, 16), (333, 80), (2048, 2048), (64, 8208)])
def test_act_dequant_equals_the_two_tensor_operations(ops, shape):
    """lq_act_dequant_i8 = x8.to(bf16) * scale.to(bf16), bit for bit, per token and per tensor (scales that are no
    bf16 numbers, a zero, an infinity and a NaN among them)."""
    M, K = shape
    g = torch.Generator().manual_seed(M + K)
    x8c = torch.randint(-128, 128, shape, generator=g, dtype=torch.int8)
    sxc = (torch.rand(M, generator=g) * 0.1 + 1e-3)
    if M > 4:
        sxc[0], sxc[1], sxc[2] = 0.0, float("inf"), float("nan")
    x8, sx = dev(x8c), dev(sxc)
    want = x8c.to(torch.bfloat16) * sxc.view(-1, 1).to(torch.bfloat16)   # the two operations, on the CPU
    got = ops.act_dequant_i8(x8, sx, True).cpu()
    # NaNs (0 * inf, x * NaN) in the same places, whatever their payload bits; everything else bit for bit
    nan = torch.isnan(want)
    assert torch.equal(torch.isnan(got), nan)
    diff = (got.view(torch.int16) != want.view(torch.int16)) & ~nan
    assert int(diff.sum()) == 0, (int(diff.sum()), diff.nonzero()[:5].tolist())
    s1c = torch.tensor([3.0, 0.0123456, 7.0])
    s1 = dev(s1c)[1:2]   # an element inside a larger buffer
    want = x8c.to(torch.bfloat16) * s1c[1].to(torch.bfloat16)
    got = ops.act_dequant_i8(x8, s1, False).cpu()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    with pytest.raises(ValueError):
        ops.act_dequant_i8(x8, sx[:-1] if M > 1 else dev(torch.zeros(2)), True)


@pytest.mark.parametrize("clampv", [3.984375, 0.0123, 250.0, 2.0 ** -45, 0.0])
@pytest.mark.parametrize("n", [5, 4096 * 33 + 3])
def test_act_fake_quant_equals_the_tensor_chain(ops, n, clampv):
    """lq_act_fake_quant = (x * s).round_().clamp_(-128, 127).div_(s) with s = 127 / clampv in bf16, bit for bit: values
    on rounding ties, beyond the clamp, infinities and a NaN among the inputs; scales inside and outside the range
    of the reciprocal product (and the infinite scale of a zero clamp value)."""
    c = torch.tensor([clampv], dtype=torch.bfloat16)
    s = 127. / c
    x = randn_bf16((n,), n, 2.0) * float(c.float().abs().clamp(min=1e-30))
    x = x.to(torch.bfloat16)
    sf = float(s.float())
    if n > 16 and 0 < abs(sf) < float("inf"):
        x[:8] = (torch.tensor([0.5, 1.5, 2.5, -0.5, -1.5, 126.5, 127.5, -128.5]) / sf).to(torch.bfloat16)
        x[8], x[9], x[10], x[11] = float("inf"), float("-inf"), float("nan"), 0.0
    want = (x * s).round_().clamp_(-128, 127).div_(s)   # the chain, on the CPU
    assert torch.equal(bits_t(127. / dev(c)), bits_t(s))  # the scalar the module computes on the device is the same number
    got = ops.act_fake_quant(dev(x), dev(s).reshape(1)).cpu()
    nan = torch.isnan(want)
    assert torch.equal(torch.isnan(got), nan)
    diff = (got.view(torch.int16) != want.view(torch.int16)) & ~nan
    assert int(diff.sum()) == 0, (int(diff.sum()), diff.nonzero()[:5].tolist())


def test_a8w8_per_token_forward_matches_float64(ops):
    """Per-token x per-channel scaled output of the int8 GEMM (bf16 scales read in the epilogue) against the float64
    product of the dequantised operands."""
    M, N, K = 300, 256, 1024
    x = randn_bf16((M, K), 3, 1.0)
    x[7] *= 40.0  # an outlier token: per-token scales keep the others' resolution
    g = torch.Generator().manual_seed(5)
    w8 = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8)
    qs = (torch.rand(N, generator=g) * 0.01 + 1e-3).to(torch.bfloat16)
    x8, sx = ops.act_quant_i8_per_token(dev(x))
    y = ops.a8w8_forward(x8, dev(w8), sx, dev(qs)).cpu()
    want = (x8.cpu().double() * sx.cpu().double()[:, None]) @ (w8.double() * qs.double()[:, None]).t()
    err = rel_l2(y, want)
    print(f"a8w8 per-token rel_l2={err:.3e}")
    assert err < 4e-3
    # and against the unquantised product: the quantisation error of per-token int8 activations
    full = x.double() @ (w8.double() * qs.double()[:, None]).t()
    assert rel_l2(y, full) < 2e-2
    y32 = ops.a8w8_forward(x8, dev(w8), sx, dev(qs.float())).cpu()
    assert torch.equal(y, y32)  # bf16 scales widened in the epilogue = the fp32 copy of them


@pytest.mark.parametrize("M,N,K", [(2048, 2048, 2048), (300, 64, 128), (2048, 8192, 2048), (100, 2048, 8192), (520, 192, 384)])
def test_a8w8_dx_from_int8_codes(ops, M, N, K):
    """dX = dY . bf16(W8 * qs): the weight tile is formed inside the GEMM. Against the float64 product with that
    bf16 weight (rel-L2, printed), and exactly for integer-valued operands with power-of-two scales."""
    g = torch.Generator().manual_seed(N + K)
    w8 = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int8)
    qs = ((torch.randn(N, generator=g) * 0.01).abs() + 1e-3).to(torch.bfloat16)
    dy = randn_bf16((M, N), 3)
    dx = ops.a8w8_dx(dev(dy), dev(w8), dev(qs)).cpu()
    wf = (w8.to(torch.bfloat16) * qs[:, None]).to(torch.bfloat16)  # what the reference's backward materialises
    want = dy.double() @ wf.double()
    err = rel_l2(dx, want)
    print(f"a8w8_dx {M}x{N}x{K}: rel_l2={err:.3e} max_abs={float((dx.double() - want).abs().max()):.3e}")
    assert err < 4e-3
    # exact case: a few rows of dY one-hot with power-of-two values, scales powers of two: dX rows are scaled weight rows
    dy1 = torch.zeros((M, N), dtype=torch.bfloat16)
    rows = [0, M // 2, M - 1]
    cols = [0, N // 3, N - 1]
    for r_, c_ in zip(rows, cols):
        dy1[r_, c_] = 2.0
    qs2 = torch.tensor([2.0 ** ((i % 5) - 7) for i in range(N)], dtype=torch.bfloat16)
    dx1 = ops.a8w8_dx(dev(dy1), dev(w8), dev(qs2)).cpu()
    for r_, c_ in zip(rows, cols):
        assert torch.equal(dx1[r_].float(), 2.0 * w8[c_].float() * qs2[c_].float())
    assert not dx1[1].any()


# ------------------------------------------------------------------ repack --
@pytest.mark.parametrize("N,K", [(16, 128), (100, 384), (4096, 1024)])
def test_repack_round_trip(ops, co, N, K):
    codes, packed, _, _ = make_w4(N, K, N + 1)
    gptq = co.native_to_gptq(packed.numpy(), N, K)
    got = ops.repack_native_to_gptq(dev(packed), (N, K)).cpu().numpy()
    assert np.array_equal(got, gptq)
    back = ops.repack_gptq_to_native(dev(torch.from_numpy(gptq)), (N, K)).cpu()
    assert torch.equal(back, packed)


# ------------------------------------------------------------- error paths --
def test_error_reporting(ops):
    from latentq_llm_amd._C import LatentQError
    N, K = 16, 128
    codes, packed, scales, zeros = make_w4(N, K, 1)
    x = randn_bf16((32, K), 2)
    with pytest.raises(LatentQError, match="CPU"):
        ops.a16w4_forward(x, packed, scales, zeros, (N, K))
    with pytest.raises(ValueError):
        ops.a16w4_forward(dev(x)[:, :64].contiguous(), dev(packed), dev(scales), dev(zeros), (N, K))


# ------------------------------------------------------------- transpose / dW --
@pytest.mark.parametrize("R,C", [(8, 8), (64, 64), (72, 136), (2048, 4096), (1000, 11008)])
def test_transpose_bf16(ops, R, C):
    x = randn_bf16((R, C), R + C)
    got = ops.transpose_bf16(dev(x))
    assert got.shape == (C, R) and got.is_contiguous()
    assert torch.equal(got.cpu(), x.t().contiguous())


def test_weight_grad_matches_the_strided_gemm(ops):
    dy, x = randn_bf16((512, 384), 1), randn_bf16((512, 256), 2)
    got = ops.weight_grad(dev(dy), dev(x))
    want = dy.float().t().mm(x.float())
    assert got.shape == (384, 256)
    assert util.rel_l2(got.float().cpu(), want) < 5e-3


# ------------------------------------------------------- split reduction (skinny grids) --
@pytest.mark.parametrize("M,N,K,bias", [(512, 1024, 4096, True), (200, 2048, 1280, False), (130, 4096, 11008, True)])
def test_a16w4_fwd_split_reduction(ops, co, M, N, K, bias):
    """Grids of a few dozen tiles with a long reduction: the forward product runs as slices of K with
    fp32 partial tiles in the scratch buffer (slice lengths 16+16+16+16, 8+8+4 and 44+44+44+40 steps)."""
    _fwd_case(ops, co, M, N, K, seed=M + N + K, with_bias=bias)


@pytest.mark.parametrize("M,N,K", [(512, 4096, 1024), (200, 1280, 2048), (64, 11008, 4096)])
def test_a16w4_dx_split_reduction(ops, co, M, N, K):
    codes, packed, scales, zeros = make_w4(N, K, M + N)
    dy = randn_bf16((M, N), 7)
    _, want64 = co.a16w4_dx(bits(dy), packed.numpy(), bits(scales), bits(zeros), M, N, K, want_f64=True)
    got = ops.a16w4_dx(dev(dy), dev(packed), dev(scales), dev(zeros), (N, K)).float().cpu()
    assert rel_l2(got, torch.from_numpy(want64)) <= REL_L2_TOL


def test_split_reduction_identity_is_exact_and_deterministic(ops, co):
    """X = identity through the split path: every output is one dequantised weight plus exact zeros
    from the other slices, so the result equals the reference dequantisation bit for bit; and two
    runs give the same bits (the slices are added in a fixed order)."""
    N, K = 256, 1024
    codes, packed, scales, zeros = make_w4(N, K, 23)
    x = dev(torch.eye(K, dtype=torch.bfloat16))
    got = ops.a16w4_forward(x, dev(packed), dev(scales), dev(zeros), (N, K))
    want = co.dequant(packed.numpy(), bits(scales), bits(zeros), N, K)
    assert np.array_equal(bits(got).T, want)
    xr = dev(randn_bf16((K, K), 3))
    a = ops.a16w4_forward(xr, dev(packed), dev(scales), dev(zeros), (N, K))
    b = ops.a16w4_forward(xr, dev(packed), dev(scales), dev(zeros), (N, K))
    assert torch.equal(a, b)


def test_workspace_entry_points_without_a_workspace_match_the_plain_ones(ops):
    """lq_a16w4_fwd (no scratch) and lq_a16w4_fwd_ws agree within the bf16 output rounding."""
    from latentq_llm_amd import _C
    M, N, K = 256, 1024, 2048
    codes, packed, scales, zeros = make_w4(N, K, 41)
    x, p, s, z = dev(randn_bf16((M, K), 42)), dev(packed), dev(scales), dev(zeros)
    y0 = torch.empty(M, N, dtype=torch.bfloat16, device=x.device)
    st = torch.cuda.current_stream().cuda_stream
    _C.call("lq_a16w4_fwd", x.data_ptr(), p.data_ptr(), s.data_ptr(), z.data_ptr(), None, y0.data_ptr(), M, N, K, 128, st)
    y1 = ops.a16w4_forward(x, p, s, z, (N, K))
    assert rel_l2(y1.float().cpu(), y0.float().cpu()) < 4e-3


@pytest.mark.parametrize("slices", [0, 1, 2, 3, 8])
def test_workspace_smaller_than_wanted_is_used_as_far_as_it_goes(ops, slices):
    """A scratch buffer that holds fewer slices than the planner would like (or none) only changes the
    split, never the validity: results stay within the output rounding of the plain entry point."""
    from latentq_llm_amd import _C
    M, N, K = 128, 2048, 1024  # dX: 16 tiles of 128 x 128, 32 reduction steps: up to 4 slices of 8 steps
    codes, packed, scales, zeros = make_w4(N, K, 77)
    dy, p, s, z = dev(randn_bf16((M, N), 78)), dev(packed), dev(scales), dev(zeros)
    st = torch.cuda.current_stream().cuda_stream
    ref = torch.empty(M, K, dtype=torch.bfloat16, device="cuda")
    _C.call("lq_a16w4_dx", dy.data_ptr(), p.data_ptr(), s.data_ptr(), z.data_ptr(), ref.data_ptr(), M, N, K, 128, st)
    nbytes = slices * M * K * 4 + 64
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    out = torch.empty_like(ref)
    _C.call("lq_a16w4_dx_ws", dy.data_ptr(), p.data_ptr(), s.data_ptr(), z.data_ptr(), out.data_ptr(), M, N, K, 128,
            ws.data_ptr(), nbytes, st)
    assert rel_l2(out.float().cpu(), ref.float().cpu()) < 4e-3
    if slices < 2:
        assert torch.equal(out, ref)  # no room for a split: the same kernel as the plain entry point


# ------------------------------------------------------ fused gate / up / SiLU product --
def _gate_up_case(ops, co, M, N, K, seed):
    _, pg, sg, zg = make_w4(N, K, seed)
    _, pu, su, zu = make_w4(N, K, seed + 1)
    x = randn_bf16((M, K), seed + 2)
    _, g64 = co.a16w4_fwd(bits(x), pg.numpy(), bits(sg), bits(zg), None, M, N, K, want_f64=True)
    _, u64 = co.a16w4_fwd(bits(x), pu.numpy(), bits(su), bits(zu), None, M, N, K, want_f64=True)
    g64, u64 = torch.from_numpy(g64), torch.from_numpy(u64)
    want = g64 / (1 + torch.exp(-g64)) * u64
    gate, up = (dev(pg), dev(sg), dev(zg)), (dev(pu), dev(su), dev(zu))
    xd = dev(x)
    got = ops.a16w4_gate_up_silu(xd, gate, up, (N, K))
    torch.cuda.synchronize()
    err = rel_l2(got.float().cpu(), want)
    # the same product from two ordinary forwards and bf16 tensor operations (two more roundings)
    unfused = torch.nn.functional.silu(ops.a16w4_forward(xd, *gate, (N, K))) * ops.a16w4_forward(xd, *up, (N, K))
    err_unfused = rel_l2(unfused.float().cpu(), want)
    print(f"gate/up M={M} N={N} K={K}: fused rel_l2={err:.3e}, two forwards + bf16 silu*mul rel_l2={err_unfused:.3e}")
    assert err <= REL_L2_TOL
    if M * N >= 1 << 16:  # enough outputs for the comparison to mean something: one rounding instead of three
        assert err <= err_unfused * 1.05
    assert rel_l2(got.float(), unfused.float()) <= REL_L2_TOL
    return got


@pytest.mark.parametrize("M,N,K", [(17, 16, 256), (128, 128, 256), (130, 272, 512), (300, 400, 768), (1000, 1040, 1280),
                                   (2048, 11008, 4096)])
def test_a16w4_gate_up_silu(ops, co, M, N, K):
    """silu(X Wg^T) * (X Wu^T) in one launch against float64, ragged in M and N (N = 16: one partial tile; 272,
    400, 1040: a partial last tile of 16 columns), 4..20 reduction steps, and the benchmark's shape."""
    if N * K > 2 ** 24:
        # the float64 oracle on the full matrix takes minutes: check a band of tokens against it instead
        _, pg, sg, zg = make_w4(N, K, 5)
        _, pu, su, zu = make_w4(N, K, 6)
        x = randn_bf16((M, K), 7)
        got = ops.a16w4_gate_up_silu(dev(x), (dev(pg), dev(sg), dev(zg)), (dev(pu), dev(su), dev(zu)), (N, K))
        rows = [0, 127, 128, 1000, 2047]
        xs = x[rows]
        _, g64 = co.a16w4_fwd(bits(xs), pg.numpy(), bits(sg), bits(zg), None, len(rows), N, K, want_f64=True)
        _, u64 = co.a16w4_fwd(bits(xs), pu.numpy(), bits(su), bits(zu), None, len(rows), N, K, want_f64=True)
        g64, u64 = torch.from_numpy(g64), torch.from_numpy(u64)
        want = g64 / (1 + torch.exp(-g64)) * u64
        err = rel_l2(got[rows].float().cpu(), want)
        print(f"gate/up full size: rel_l2={err:.3e} on {len(rows)} token rows")
        assert err <= REL_L2_TOL
        return
    _gate_up_case(ops, co, M, N, K, seed=M + N + K)


@pytest.mark.parametrize("M", [1, 3, 4, 5, 16])
@pytest.mark.parametrize("N,K", [(16, 128), (64, 640), (4096, 4096), (256, 11008)])
def test_a16w4_gate_up_silu_few_tokens(ops, co, M, N, K):
    """Up to 16 tokens: one GEMV pass over both matrices (2 to 16 waves, partial batches, K not a multiple of 256)."""
    _gate_up_case(ops, co, M, N, K, seed=M + N + K)


def test_a16w4_gate_up_silu_rejects_what_it_does_not_cover(ops):
    from latentq_llm_amd._C import LatentQError
    _, p, s, z = make_w4(64, 256, 1)
    w = (dev(p), dev(s), dev(z))
    _, p, s, z = make_w4(64, 384, 1)
    w = (dev(p), dev(s), dev(z))
    with pytest.raises(LatentQError, match="multiple of 256"):
        ops.a16w4_gate_up_silu(dev(randn_bf16((32, 384), 2)), w, w, (64, 384))


def test_fused_mlp_module_matches_the_three_layers(hip_lib):
    """QuantLlamaMLP / make_fused_mlp on QLinearA16W4 layers: the fused path (many tokens) and the composed path
    (few tokens) both agree with down(silu(gate(x)) * up(x)) run layer by layer."""
    import torch.nn as nn
    from latentq_llm_amd import quant as Q
    from latentq_llm_amd.fused_mlp import QuantLlamaMLP, make_fused_mlp

    hid, ffn = 256, 512

    def layer(n, k, seed):
        _, packed, scales, zeros = make_w4(n, k, seed)
        m = Q.QLinearA16W4(k, n, bias=False, lbit=0)
        m.zeros.data, m.scales.data, m.wshape = zeros.clone(), scales.clone(), [n, k]
        m.weight.set_value(packed, [m.scales, m.zeros, m.wshape])
        m = m.bfloat16().cuda()
        m.to("cuda")
        return m

    class MLP(nn.Module):
        def __init__(self):
            super().__init__()
            self.gate_proj, self.up_proj, self.down_proj = layer(ffn, hid, 1), layer(ffn, hid, 2), layer(hid, ffn, 3)

        def forward(self, x):
            return self.down_proj(torch.nn.functional.silu(self.gate_proj(x)) * self.up_proj(x))

    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.mlp = MLP()

    blk = Block()
    plain = blk.mlp
    fused = make_fused_mlp(blk).mlp
    assert isinstance(fused, QuantLlamaMLP) and fused.gate_proj is plain.gate_proj
    # 6 tokens: the fused GEMV pass; 40 tokens: the composed path (silu and product on the two forward results);
    # 512 tokens: the fused MFMA kernel
    for tokens in ((2, 3), (2, 20), (4, 128)):
        x = randn_bf16(tokens + (hid,), 9).cuda()
        with torch.no_grad():
            want, got = plain(x), fused(x)
        assert got.shape == want.shape == tokens + (hid,)
        err = rel_l2(got.float(), want.float())
        print(f"{tokens}: fused MLP vs layer by layer rel_l2={err:.3e}")
        assert err <= REL_L2_TOL


def _mlp_layers(Q, hid, ffn, train):
    def layer(n, k, seed):
        _, packed, scales, zeros = make_w4(n, k, seed)
        m = Q.QLinearA16W4(k, n, bias=False, lbit=16)
        m.zeros.data, m.scales.data, m.wshape = zeros.clone(), scales.clone(), [n, k]
        m.weight.set_value(packed, [m.scales, m.zeros, m.wshape])
        m = m.bfloat16().cuda()
        m.to("cuda")
        if train:
            m.weight.requires_grad = True
            m.add_hook()
        return m, (packed, scales, zeros)
    return layer(ffn, hid, 1), layer(ffn, hid, 2), layer(hid, ffn, 3)


def test_fused_mlp_composed_path_with_odd_hidden_size(hip_lib):
    """A hidden size that is no multiple of 256 takes the composed path at every token count above 16."""
    from latentq_llm_amd import quant as Q
    from latentq_llm_amd.fused_mlp import QuantLlamaMLP
    (g, _), (u, _), (d, _) = _mlp_layers(Q, 384, 512, train=False)
    fused = QuantLlamaMLP(g, d, u)
    for tokens in (20, 200):
        x = randn_bf16((tokens, 384), tokens).cuda()
        with torch.no_grad():
            want = d(torch.nn.functional.silu(g(x)) * u(x))
            got = fused(x)
        assert rel_l2(got.float(), want.float()) <= REL_L2_TOL


@pytest.mark.parametrize("tokens,hid,ffn", [(300, 256, 512), (12, 256, 512), (520, 512, 1408), (40, 384, 512)])
def test_fused_mlp_training_step(hip_lib, tokens, hid, ffn):
    """A QuantLlamaMLP whose layers are being trained: output, input gradient and the three weight gradients against
    the float64 composition, and against the same block run layer by layer through autograd; the hooks' dict_temp
    is drained; a second backward accumulates. (hid = 384 is not a multiple of 256: the layers' own forward.)"""
    from latentq_llm_amd import ops, quant as Q
    from latentq_llm_amd.fused_mlp import QuantLlamaMLP
    (g, gw), (u, uw), (d, dw_) = _mlp_layers(Q, hid, ffn, train=True)
    fused = QuantLlamaMLP(g, d, u)
    x_cpu = randn_bf16((tokens, hid), 5)
    dy_cpu = randn_bf16((tokens, hid), 6)
    x = x_cpu.cuda().requires_grad_(True)
    y = fused(x)
    y.backward(dy_cpu.cuda())
    assert len(Q.dict_temp) == 0
    # float64 composition on the dequantised weights
    Wg = ops.a16w4_dequant(gw[0].cuda(), gw[1].cuda(), gw[2].cuda(), (ffn, hid)).double().cpu()
    Wu = ops.a16w4_dequant(uw[0].cuda(), uw[1].cuda(), uw[2].cuda(), (ffn, hid)).double().cpu()
    Wd = ops.a16w4_dequant(dw_[0].cuda(), dw_[1].cuda(), dw_[2].cuda(), (hid, ffn)).double().cpu()
    xd = x_cpu.double().requires_grad_(True)
    gg, uu = xd @ Wg.t(), xd @ Wu.t()
    hh = torch.nn.functional.silu(gg) * uu
    yy = hh @ Wd.t()
    gg.retain_grad(); uu.retain_grad(); hh.retain_grad()
    yy.backward(dy_cpu.double())
    errs = {
        "y": rel_l2(y.detach().cpu(), yy.detach()),
        "dx": rel_l2(x.grad.cpu(), xd.grad),
        "dW_down": rel_l2(d.weight.grad.cpu(), dy_cpu.double().t() @ hh.detach()),
        "dW_up": rel_l2(u.weight.grad.cpu(), uu.grad.t() @ x_cpu.double()),
        "dW_gate": rel_l2(g.weight.grad.cpu(), gg.grad.t() @ x_cpu.double()),
    }
    print(f"fused MLP training ({tokens} tokens, {hid}/{ffn}) rel_l2 vs float64: " + " ".join(f"{k}={v:.2e}" for k, v in errs.items()))
    assert max(errs.values()) <= REL_L2_TOL
    # layer by layer through autograd on the same layers: same quantities within bf16 rounding
    grads = [m.weight.grad.clone() for m in (g, u, d)]
    for m in (g, u, d):
        m.weight.grad = None
    x2 = x_cpu.cuda().requires_grad_(True)
    y2 = d(torch.nn.functional.silu(g(x2)) * u(x2))
    y2.backward(dy_cpu.cuda())
    assert rel_l2(y.detach().float(), y2.detach().float()) <= 6e-3 and rel_l2(x.grad.float(), x2.grad.float()) <= 6e-3
    for a, m in zip(grads, (g, u, d)):
        assert rel_l2(a.float(), m.weight.grad.float()) <= 6e-3
    # accumulation over a second backward of the fused block
    for m, a in zip((g, u, d), grads):
        m.weight.grad = a.clone()
    fused(x).backward(dy_cpu.cuda())
    for a, m in zip(grads, (g, u, d)):
        assert rel_l2(m.weight.grad.float(), 2 * a.float()) <= 1e-2


def test_fused_mlp_inference_call_refuses_training_inputs(hip_lib):
    from latentq_llm_amd import quant as Q
    from latentq_llm_amd.fused_mlp import QuantLlamaMLP
    (g, _), (u, _), (d, _) = _mlp_layers(Q, 256, 512, train=True)
    fused = QuantLlamaMLP(g, d, u)
    with pytest.raises(RuntimeError, match="no backward"):
        fused.fused_gate_up(randn_bf16((20, 256), 1).cuda())


@pytest.mark.parametrize("M,N,K", [(2048, 1024, 512), (300, 272, 256), (7, 512, 384), (16, 256, 256)])
def test_gate_up_silu_save_stores_the_products(ops, M, N, K):
    """The training form of the fused gate / up launch: h equals the inference form bit for bit, and the stored
    products are X . deq(W)^T of the two matrices (float64 bar; above 16 tokens also the bf16 rounding of the very
    sums h was formed from: silu(g) * u recomputed from them stays within 2 bf16 ulps of h)."""
    _, pg, sg, zg = make_w4(N, K, 1)
    _, pu, su, zu = make_w4(N, K, 2)
    gate, up = (dev(pg), dev(sg), dev(zg)), (dev(pu), dev(su), dev(zu))
    x = dev(randn_bf16((M, K), 3))
    h0 = ops.a16w4_gate_up_silu(x, gate, up, (N, K))
    h, g, u = ops.a16w4_gate_up_silu(x, gate, up, (N, K), save=True)
    assert torch.equal(h, h0)
    Wg = ops.a16w4_dequant(*gate, (N, K)).double()
    Wu = ops.a16w4_dequant(*up, (N, K)).double()
    assert rel_l2(g, x.double() @ Wg.t()) < 3e-3 and rel_l2(u, x.double() @ Wu.t()) < 3e-3
    re = torch.nn.functional.silu(g.double()) * u.double()
    assert bool(((h.double() - re).abs() <= re.abs() * 2.0 ** -6 + 1e-6).all())


@pytest.mark.parametrize("M,N,K", [(2048, 1024, 512), (100, 256, 384), (520, 1408, 512)])
def test_dx_epilogue_forms(ops, M, N, K):
    """lq_a16w4_dx_acc = lq_a16w4_dx followed by a bf16 addition, bit for bit; lq_a16w4_dx_silu_bwd against the fp32
    formula on the bf16-rounded product (1 ulp: exp and reciprocal are the hardware's)."""
    codes, packed, scales, zeros = make_w4(N, K, 3)
    w = (dev(packed), dev(scales), dev(zeros))
    dy = dev(randn_bf16((M, N), 4))
    base = dev(randn_bf16((M, K), 5, 30.0))
    p = ops.a16w4_dx(dy, *w, (N, K))
    acc = base.clone()
    ops.a16w4_dx(dy, *w, (N, K), out=acc, accumulate=True)
    assert torch.equal(acc, base + p)
    g, u = dev(randn_bf16((M, K), 6, 2.0)), dev(randn_bf16((M, K), 7))
    dg, du = ops.a16w4_dx_silu_bwd(dy, *w, (N, K), g, u)
    pf, gf, uf = p.double(), g.double(), u.double()
    sg = torch.sigmoid(gf)
    want_dg = pf * uf * sg * (1 + gf * (1 - sg))
    want_du = pf * gf * sg
    assert rel_l2(dg, want_dg) < 3e-3 and rel_l2(du, want_du) < 3e-3
    # elementwise: within 2 bf16 ulps of the size of the factors (silu'(g) passes through zero near g = -1.28, so the
    # bound is relative to |P u| and |P g|, not to the result)
    for got, want, scale in ((dg, want_dg, (pf * uf).abs() * 1.1), (du, want_du, (pf * gf).abs())):
        diff = (got.double() - want).abs()
        # (the absolute term: P here comes from a launch that may cut the reduction differently, and where the sum
        # cancels the two fp32 sums differ by more than a bf16 ulp of the small result)
        assert bool((diff <= scale * 2.0 ** -7 + 2e-5 * (1 + uf.abs() + gf.abs())).all())


@pytest.mark.parametrize("M,N,K", [(2048, 1024, 512), (100, 256, 384), (520, 1408, 512), (17, 64, 128)])
def test_dx_pair(ops, M, N, K):
    """lq_a16w4_dx_pair = dY1 . deq(W1) + dY2 . deq(W2) in one reduction: against float64; with one of the two
    gradients zero it is the other product's unsplit kernel bit for bit (the reduction only gains exact zeros),
    which pins which operands go together and the order of the two halves."""
    _, p1, s1, z1 = make_w4(N, K, 3)
    _, p2, s2, z2 = make_w4(N, K, 13)
    w1, w2 = (dev(p1), dev(s1), dev(z1)), (dev(p2), dev(s2), dev(z2))
    dy1, dy2 = dev(randn_bf16((M, N), 4)), dev(randn_bf16((M, N), 14))
    got = ops.a16w4_dx_pair(dy1, w1, dy2, w2, (N, K))
    want = dy1.double() @ ops.a16w4_dequant(*w1, (N, K)).double() + dy2.double() @ ops.a16w4_dequant(*w2, (N, K)).double()
    assert rel_l2(got, want) < 3e-3
    assert bool(((got.double() - want).abs() <= want.abs() * 2.0 ** -8 + 1e-3 * N ** 0.5 * 2.0 ** -8).all())
    zero = torch.zeros_like(dy1)
    for a, b, single in ((dy1, zero, (dy1, w1)), (zero, dy2, (dy2, w2))):
        base = torch.zeros((M, K), dtype=torch.bfloat16, device=dy1.device)
        ops.a16w4_dx(single[0], *single[1], (N, K), out=base, accumulate=True)  # the unsplit kernel: 0 + P
        assert torch.equal(ops.a16w4_dx_pair(a, w1, b, w2, (N, K)), base)
    # the caller's buffer, and argument checks
    out = torch.empty((M, K), dtype=torch.bfloat16, device=dy1.device)
    assert ops.a16w4_dx_pair(dy1, w1, dy2, w2, (N, K), out=out) is out and torch.equal(out, got)
    with pytest.raises(ValueError):
        ops.a16w4_dx_pair(dy1, w1, dy2[:-1], w2, (N, K))


@pytest.mark.parametrize("N,K", [(1, 8), (12, 64), (100, 1032), (2048, 8192)])
def test_w8_requant_bit_exact(ops, co, N, K):
    """lq_w8_requant against the C restatement of Qfunc_8bit_res: random latents, ties, saturation, infinities, NaN
    (-> 0), scales of both signs and outside the range in which the kernel multiplies by the reciprocal."""
    lat = randn_bf16((N, K), N + K, 0.05)
    qs = (torch.rand(N, 1, generator=torch.Generator().manual_seed(N)) * 1e-3 + 1e-4).to(torch.bfloat16)
    if N >= 12:
        qs[3] = -qs[3]
        qs[4] = 2.0 ** -50
        qs[5] = 2.0 ** 50
        lat[5] *= 2.0 ** 55
        lat[1, 0], lat[1, 1], lat[2, 3] = float("inf"), float("-inf"), float("nan")
        lat[0, :8] = (torch.tensor([0.5, 1.5, 2.5, -0.5, -1.5, 127.5, -128.5, 300.0]) * qs[0].float()).to(torch.bfloat16)
    want = co.w8_requant(bits(lat), bits(qs), N, K)
    got = ops.w8_requant(dev(lat), dev(qs)).cpu().numpy().reshape(-1)
    assert np.array_equal(got, want), np.nonzero(got != want)[0][:10]
