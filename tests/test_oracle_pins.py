"""CPU tests that pin the oracle (oracle/lq_oracle.c, oracle/torch_ref.py) WITHOUT retyping it.

The reference ships no tests, golden vectors or fixtures for this path, so each oracle
function is pinned by what the mathematics fixes:

  pack / unpack          known answers worked out by hand from the two-line rule, exhaustive
                         round trip over all 256 bytes, little-endian word 0x67452301
  dequant                torch's own bf16 tensor arithmetic (the arithmetic the reference runs),
                         an exact rational model with explicit round-to-nearest-even,
                         the GPTQ identity (q - (z_stored + 1)) * s
  A16W4 fwd / dX         torch float64 matmul on the dequantised matrix, the adjoint identity,
                         identity activations, bf16 torch.mm (the reference's CPU path) to tolerance
  Philox4x32-10          the three Random123 known-answer vectors; draw mapping (block, word, half), range, grid
  requant                exact rational model (fractions.Fraction, own RNE rounding), invariants
                         (idempotence, floor / ceiling at the extreme draws, saturation, 16 bits of an
                         injected uniform), unbiasedness incl. a sub-grid drift check
  reciprocal divide      exhaustive sweep over every bf16 scale (lqo_markstein_check)
  A8W8 int32             numpy int64 matmul; extreme value 127*127*8192
  A8W8 bf16 epilogue     "parity unpinned": the reference's epilogue lives in the external,
                         un-vendored torch_int (FWkey/torch-int-bf16, no pinned version); only the
                         closed form bf16((acc*sx)*sw + bias) of this build is checked
  act quant              torch's bf16 tensor arithmetic (given clamp value, and clampv = input.max());
                         alpha and the per-token form against numpy float32 (IEEE) arithmetic, written
                         with numpy's own vector operations
  GPTQ <-> native        defining bit formula, brute force
"""
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from oracle import torch_ref as tr
from tests.util import bits, from_bits, make_w4, pack_codes, randn_bf16, rel_l2


# exact rounding helpers and models: shared with the generator of the committed vectors
from tests.golden.exact_model import bf16, f32  # noqa: E402


def frac_of_bits(b: int) -> Fraction:
    return Fraction(float(co.bf16_bits_to_f32(np.array([b], np.uint16))[0]))


def test_rn_helper_against_numpy():
    rng = np.random.default_rng(0)
    for v in rng.standard_normal(200) * 10.0 ** rng.integers(-20, 20, 200):
        assert float(f32(Fraction(float(v)))) == float(np.float32(v))
    ties = [Fraction(1) + Fraction(1, 2 ** 8), Fraction(1) + Fraction(3, 2 ** 8), Fraction(257, 2), Fraction(259, 2)]
    assert [bf16(t) for t in ties] == [Fraction(1), Fraction(1) + Fraction(1, 64), Fraction(128), Fraction(130)]


# -------------------------------------------------------------------- packing --
def test_pack_known_answers():
    assert list(co.pack(np.array([15, 3, 8, 0, 7, 15], np.uint8))) == [0xF3, 0x80, 0x7F]
    assert co.pack(np.arange(8, dtype=np.uint8)).view("<u4")[0] == 0x67452301
    t = tr.compress(torch.tensor([15, 3, 8, 0, 7, 15], dtype=torch.uint8))
    assert t.tolist() == [-13, -128, 127]


def test_pack_unpack_exhaustive():
    allb = np.arange(256, dtype=np.uint8)
    codes = co.unpack(allb)
    assert codes.max() == 15 and np.array_equal(codes[0::2], allb >> 4) and np.array_equal(codes[1::2], allb & 15)
    assert np.array_equal(co.pack(codes), allb)
    tcodes = tr.decompress(torch.from_numpy(allb.view(np.int8)))
    assert np.array_equal(tcodes.numpy().reshape(-1).astype(np.uint8), codes)
    assert np.array_equal(tr.compress(tcodes).numpy().view(np.uint8), allb)


# -------------------------------------------------------------------- dequant --
def test_dequant_matches_torch_bf16_arithmetic():
    N, K = 24, 384
    codes, packed, scales, zeros = make_w4(N, K, 0)
    zeros.view(-1)[::3] = 7.5
    zeros.view(-1)[1::7] = 6.28125
    zeros.view(-1)[2::11] = 300.0
    want = tr.dequant_4bit_g(packed, scales, zeros, (N, K))  # torch's own bf16 ops
    got = co.dequant(packed.numpy(), bits(scales), bits(zeros), N, K)
    assert np.array_equal(got, bits(want))


def test_dequant_exact_rational_model():
    rng = np.random.default_rng(1)
    for _ in range(300):
        q = int(rng.integers(0, 16))
        zb = int(co.f32_to_bf16_bits(np.array([rng.choice([6, 7, 8, 9, 7.5, 0.3, 100.25])], np.float32))[0])
        sb = int(co.f32_to_bf16_bits(np.array([abs(rng.standard_normal()) * 0.02 / 7 + 1e-6], np.float32))[0])
        z, s = frac_of_bits(zb), frac_of_bits(sb)
        want = bf16(f32(bf16(f32(q - z)) * s))
        packed = co.pack(np.array([q] * 128, np.uint8))
        got = co.dequant(packed, np.array([sb], np.uint16), np.array([zb], np.uint16), 1, 128)
        assert Fraction(float(co.bf16_bits_to_f32(got.reshape(-1)[:1])[0])) == want


def test_dequant_gptq_identity():
    """GPTQ stores zero - 1 and dequantises (q - (z_stored + 1)) * s (PTQ/quant/quant_linear.py:339)."""
    N, K = 8, 256
    codes, packed, scales, zeros = make_w4(N, K, 2)
    w = co.bf16_bits_to_f32(co.dequant(packed.numpy(), bits(scales), bits(zeros), N, K)).reshape(N, K)
    z_stored = zeros.float().reshape(N, K // 128) - 1
    s = scales.float().reshape(N, K // 128)
    full = (codes.float().reshape(N, K // 128, 128) - (z_stored[..., None] + 1)) * s[..., None]
    assert np.array_equal(w, full.to(torch.bfloat16).float().reshape(N, K).numpy())


# ------------------------------------------------------------------ A16W4 GEMM --
def test_fwd_and_dx_against_float64_matmul_and_adjoint():
    M, N, K = 40, 48, 256
    codes, packed, scales, zeros = make_w4(N, K, 3)
    x, dy, b = randn_bf16((M, K), 4), randn_bf16((M, N), 5), randn_bf16((N,), 6)
    w = from_bits(co.dequant(packed.numpy(), bits(scales), bits(zeros), N, K)).double()
    y, y64 = co.a16w4_fwd(bits(x), packed.numpy(), bits(scales), bits(zeros), bits(b), M, N, K, want_f64=True)
    assert np.allclose(y64, (x.double() @ w.t() + b.double()).numpy(), rtol=1e-12, atol=1e-12)
    assert np.array_equal(y, bits(torch.from_numpy(y64).to(torch.float32).to(torch.bfloat16)))
    dx, d64 = co.a16w4_dx(bits(dy), packed.numpy(), bits(scales), bits(zeros), M, N, K, want_f64=True)
    assert np.allclose(d64, (dy.double() @ w).numpy(), rtol=1e-12, atol=1e-12)
    _, y64nb = co.a16w4_fwd(bits(x), packed.numpy(), bits(scales), bits(zeros), None, M, N, K, want_f64=True)
    lhs = float((torch.from_numpy(y64nb) * dy.double()).sum())
    rhs = float((x.double() * torch.from_numpy(d64)).sum())
    assert abs(lhs - rhs) <= 1e-9 * max(1.0, abs(lhs))


def test_fwd_identity_and_reference_cpu_path():
    N, K = 32, 128
    codes, packed, scales, zeros = make_w4(N, K, 7)
    eye = torch.eye(K, dtype=torch.bfloat16)
    y = co.a16w4_fwd(bits(eye), packed.numpy(), bits(scales), bits(zeros), None, K, N, K)
    assert np.array_equal(y.T, co.dequant(packed.numpy(), bits(scales), bits(zeros), N, K))
    x = randn_bf16((64, K), 8)
    ref = tr.w4_forward(x, packed, scales, zeros, (N, K))  # reference CPU path: bf16 torch.mm
    _, y64 = co.a16w4_fwd(bits(x), packed.numpy(), bits(scales), bits(zeros), None, 64, N, K, want_f64=True)
    assert rel_l2(ref.float(), torch.from_numpy(y64)) < 5e-3


# --------------------------------------------------------------------- Philox --
def test_philox_known_answers():
    kat = [
        ([0, 0, 0, 0], [0, 0], [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]),
        ([0xFFFFFFFF] * 4, [0xFFFFFFFF] * 2, [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]),
        ([0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344], [0xA4093822, 0x299F31D0],
         [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]),
    ]
    for ctr, key, out in kat:
        assert list(co.philox4x32_10(ctr, key)) == out


def test_philox_uniform_mapping():
    """Element i takes the 16-bit half (i & 1) of word (i >> 1) & 3 of block offset + i // 8; the
    uniform is (a + 1/2) / 65536: inside (0, 1), on the centred 2^-16 grid, never 0 or 1."""
    seed, off = 0x0123456789ABCDEF, 2 ** 32 - 2
    u = co.philox_uniform(4096, seed, off)
    a = u.astype(np.float64) * 65536 - 0.5
    assert u.min() > 0 and u.max() < 1 and np.all(a == np.floor(a))
    for i in (0, 1, 5, 8, 4095):
        c = off + i // 8
        w = co.philox4x32_10([c & 0xFFFFFFFF, c >> 32, 0, 0], [seed & 0xFFFFFFFF, seed >> 32])
        half = (int(w[(i >> 1) & 3]) >> (16 * (i & 1))) & 0xFFFF
        assert u[i] == np.float32((half + 0.5) * 2.0 ** -16)
    assert 0.48 < u.mean() < 0.52 and abs(np.corrcoef(u[:-1], u[1:])[0, 1]) < 0.05
    # the two halves of a word and the four words of a block are all used: 8 distinct draws per block
    blk = co.philox_uniform(8, 1, 0)
    assert len(set(blk.tolist())) == 8


# -------------------------------------------------------------------- requant --
def requant_model(q, zb, sb, gb, lr, u):
    """Exact rational restatement of the update rule (own rounding helper, no float arithmetic):
    the 16.16 fixed-point sum floor(x * 2^16 + 1/2) + a with a = floor(u * 2^16)."""
    z, s, g = frac_of_bits(zb), frac_of_bits(sb), frac_of_bits(gb)
    w = bf16(f32(bf16(f32(q - z)) * s))
    t = f32(w - Fraction(float(np.float32(lr))) * g)
    r16 = f32(f32(1 / s) * 65536)
    y = f32(t * r16 + f32(z * 65536 + Fraction(1, 2)))
    x = min(max(y.numerator // y.denominator, 0), 2 ** 32 - 1)
    ua = f32(Fraction(float(u)) * 65536)
    a = min(max(ua.numerator // ua.denominator, 0), 65535)
    return min(min(x + a, 2 ** 32 - 1) >> 16, 15)


@pytest.mark.parametrize("lr,gstd", [(1e-4, 1e-3), (1.0, 2e-3), (3e-2, 1.0)])
def test_requant_exact_rational_model(lr, gstd):
    N, K = 2, 128
    codes, packed, scales, zeros = make_w4(N, K, int(lr * 1e4) + 3)
    zeros.view(-1)[1] = 7.5
    grad = randn_bf16((N, K), 11, gstd)
    u = torch.rand((N, K), generator=torch.Generator().manual_seed(12), dtype=torch.float32)
    u.view(-1)[::9] = 0.0
    got = co.unpack(co.requant(packed.numpy(), bits(scales), bits(zeros), bits(grad), lr, N, K, u=u.numpy()))
    sb, zb, gb = bits(scales).reshape(-1), bits(zeros).reshape(-1), bits(grad).reshape(-1)
    cf = codes.reshape(-1)
    for i in range(N * K):
        want = requant_model(int(cf[i]), int(zb[i // 128]), int(sb[i // 128]), int(gb[i]), lr, float(u.view(-1)[i]))
        assert got[i] == want, i


def test_requant_invariants():
    N, K = 16, 256
    codes, packed, scales, zeros = make_w4(N, K, 13)
    zero_g = torch.zeros((N, K), dtype=torch.bfloat16)
    half = np.full(N * K, 0.5, np.float32)
    args = (bits(scales), bits(zeros))
    assert np.array_equal(co.requant(packed.numpy(), *args, bits(zero_g), 1e-4, N, K, u=half), packed.numpy().view(np.uint8))
    big = torch.full((N, K), 1e30, dtype=torch.bfloat16)
    assert np.all(co.requant(packed.numpy(), *args, bits(big), 1.0, N, K, u=half) == 0x00)
    assert np.all(co.requant(packed.numpy(), *args, bits(-big), 1.0, N, K, u=half) == 0xFF)
    # the smallest draw (a = 0: u = 2^-17) is a floor: with g = 0 the code can only stay or drop by one
    # (bf16 rounding of w); the largest (a = 65535) is a ceiling: stay or rise by one
    fl = co.unpack(co.requant(packed.numpy(), *args, bits(zero_g), 1e-4, N, K, u=np.zeros(N * K, np.float32)))
    d = codes.reshape(-1).numpy().astype(int) - fl.astype(int)
    assert set(np.unique(d)) <= {0, 1}
    top = np.full(N * K, 1.0 - 2.0 ** -17, np.float32)
    ce = co.unpack(co.requant(packed.numpy(), *args, bits(zero_g), 1e-4, N, K, u=top))
    d = ce.astype(int) - codes.reshape(-1).numpy().astype(int)
    assert set(np.unique(d)) <= {0, 1}
    # only 16 bits of an injected uniform are used, out-of-range values saturate, NaN counts as 0
    g2 = randn_bf16((N, K), 17, 1e-2)
    base = np.random.default_rng(5).random(N * K, dtype=np.float32)
    trunc = np.floor(base.astype(np.float64) * 65536) / 65536
    ra = co.requant(packed.numpy(), *args, bits(g2), 0.05, N, K, u=base)
    assert np.array_equal(ra, co.requant(packed.numpy(), *args, bits(g2), 0.05, N, K, u=trunc.astype(np.float32)))
    odd = base.copy()
    odd[::3], odd[1::3] = -1.0, 7.0
    odd[2::3] = np.nan
    ref = np.where(np.arange(N * K) % 3 == 1, np.float32(1 - 2.0 ** -16), np.float32(0)).astype(np.float32)
    assert np.array_equal(co.requant(packed.numpy(), *args, bits(g2), 0.05, N, K, u=odd),
                          co.requant(packed.numpy(), *args, bits(g2), 0.05, N, K, u=ref))
    # Philox mode == injected mode on the materialised stream
    g = randn_bf16((N, K), 14, 1e-2)
    a = co.requant(packed.numpy(), *args, bits(g), 0.05, N, K, seed=99, offset=5)
    b = co.requant(packed.numpy(), *args, bits(g), 0.05, N, K, u=co.philox_uniform(N * K, 99, 5))
    assert np.array_equal(a, b)


def test_requant_unbiased():
    """E_u[code'] = (w - lr g)/s + z for non-saturating updates: mean over many seeds."""
    N, K = 4, 128
    codes, packed, scales, zeros = make_w4(N, K, 15)
    codes = torch.randint(3, 12, (N, K), generator=torch.Generator().manual_seed(1), dtype=torch.uint8)
    packed = pack_codes(codes)
    g = randn_bf16((N, K), 16, 1.0)
    lr = 2e-3
    w = tr.dequant_4bit_g(packed, scales, zeros, (N, K)).float()
    s = scales.float().repeat_interleave(128).view(N, K)
    z = zeros.float().repeat_interleave(128).view(N, K)
    target = ((w - lr * g.float()) / s + z).numpy().reshape(-1)
    acc = np.zeros(N * K)
    reps = 400
    for r in range(reps):
        acc += co.unpack(co.requant(packed.numpy(), bits(scales), bits(zeros), bits(g), lr, N, K, seed=r, offset=0))
    inside = (target > 0.5) & (target < 14.5)
    assert inside.sum() > 100
    assert np.abs(acc / reps - target)[inside].max() < 0.12  # 4 sigma of a Bernoulli mean over 400 draws


def test_requant_mean_over_all_65536_draws():
    """Every 16-bit draw once per parameter set: the mean new code equals x = (w - lr g)/s + z to
    within half a grid step (2^-17), and the centred grid leaves no common drift over sets whose x
    falls at unrelated places inside a 2^-16 cell (an uncentred grid would show -2^-17)."""
    sets, K = 24, 128
    rows_per_set = 65536 // K
    N = sets * rows_per_set
    rng = np.random.default_rng(21)
    q = rng.integers(2, 14, sets)
    s_bits = bits(torch.tensor(np.abs(rng.normal(0, 0.02, sets)) / 7 + 1e-4).to(torch.bfloat16))
    z_val = rng.integers(6, 10, sets).astype(np.float32)
    g_bits = bits(torch.tensor(rng.normal(0, 1e-3, sets)).to(torch.bfloat16))
    lr = np.float32(1e-4)
    codes = np.repeat(q, 65536).astype(np.uint8)
    packed = co.pack(codes)
    scales = np.repeat(s_bits, rows_per_set).astype(np.uint16)
    zeros = np.repeat(bits(torch.tensor(z_val).to(torch.bfloat16)), rows_per_set).astype(np.uint16)
    grad = np.repeat(g_bits, 65536).astype(np.uint16)
    u = np.tile((np.arange(65536, dtype=np.float64) + 0.5) / 65536, sets).astype(np.float32)
    new = co.unpack(co.requant(packed, scales, zeros, grad, float(lr), N, K, u=u)).reshape(sets, 65536)
    sf = co.bf16_bits_to_f32(s_bits).astype(np.float64)
    gf = co.bf16_bits_to_f32(g_bits).astype(np.float64)
    w = co.bf16_bits_to_f32(co.dequant(co.pack(np.repeat(q, K).astype(np.uint8)), s_bits, bits(torch.tensor(z_val).to(torch.bfloat16)),
                                       sets, K)[:, 0]).astype(np.float64)
    x = (w - float(lr) * gf) / sf + z_val
    err = new.mean(axis=1) - x
    assert np.abs(err).max() <= 2.0 ** -17 + 2.0 ** -20, err
    assert abs(err.mean()) < 2.0 ** -18, err.mean()


def test_reciprocal_divide_exhaustive_over_scales():
    qm, cm, n = co.markstein_check(12345, 300)
    assert n > 5_000_000 and qm == 0 and cm == 0


# ----------------------------------------------------------------------- A8W8 --
def test_a8w8_int32_exact_and_extremes():
    rng = np.random.default_rng(3)
    M, N, K = 33, 48, 256
    x = rng.integers(-128, 128, (M, K), dtype=np.int8)
    w = rng.integers(-128, 128, (N, K), dtype=np.int8)
    sx, sw = rng.random(M, dtype=np.float32), rng.random(N, dtype=np.float32)
    y, acc = co.a8w8(x, w, sx, sw, None, M, N, K)
    assert np.array_equal(acc, (x.astype(np.int64) @ w.astype(np.int64).T).astype(np.int32))
    assert np.array_equal(acc, tr.int8_matmul_i32(torch.from_numpy(x), torch.from_numpy(w)).numpy())
    closed = (acc.astype(np.float32) * sx[:, None]) * sw[None, :]
    assert np.array_equal(y, co.f32_to_bf16_bits(closed).reshape(M, N))
    xe = np.full((2, 8192), 127, np.int8)
    we = np.stack([np.full(8192, 127, np.int8), np.full(8192, -127, np.int8)])
    _, acc = co.a8w8(xe, we, np.ones(2, np.float32), np.ones(2, np.float32), None, 2, 2, 8192, want_y=False)
    assert acc.tolist() == [[132128768, -132128768]] * 2


def test_act_quant_matches_torch_bf16_arithmetic():
    x = randn_bf16((257,), 9, 3.0)
    clampv = x.max()
    want = tr.act_quant_i8(x, clampv).numpy()
    got = co.act_quant_i8(bits(x), float(clampv))
    assert np.array_equal(got, want)
    want2 = tr.act_quant_i8(x, float(clampv)).numpy()  # python-float clamp (the eval path)
    assert np.array_equal(got, want2)


def test_act_quant_dynamic_matches_torch_chain():
    """clampv = input.max() and the int8 values against torch's bf16 tensor operations (utils/quant.py:259-266);
    alpha against numpy float32: clampv times the fp32 reciprocal of 127, rounded to bf16 on request."""
    for seed, shape in [(3, (5, 77)), (4, (64, 128)), (5, (1, 9))]:
        x = randn_bf16(shape, seed, 2.5)
        M, K = shape
        clampv = x.max()
        want8 = tr.act_quant_i8(x, clampv).numpy().reshape(-1)
        for alpha_bf16 in (False, True):
            x8, sx, cv, alpha = co.act_quant_i8_dynamic(bits(x), M, K, alpha_bf16)
            assert cv == float(clampv) and np.array_equal(x8, want8)
            a = np.float32(float(clampv)) * (np.float32(1.0) / np.float32(127.0))
            if alpha_bf16:
                a = np.float32(torch.tensor(float(a)).to(torch.bfloat16).float().item())
            assert alpha == a and np.all(sx == a) and sx.shape == (M,)
    # all-negative tensor: the maximum is the element closest to zero; a NaN anywhere: NaN clamp, all codes zero
    x = -randn_bf16((4, 16), 6).abs() - 1
    x8, sx, cv, _ = co.act_quant_i8_dynamic(bits(x), 4, 16, False)
    assert cv == float(x.max()) and np.array_equal(x8, tr.act_quant_i8(x, x.max()).numpy().reshape(-1))
    x.view(-1)[7] = float("nan")
    x8, sx, cv, alpha = co.act_quant_i8_dynamic(bits(x), 4, 16, True)
    assert np.isnan(cv) and np.isnan(alpha) and np.isnan(sx).all() and not x8.any()
    assert torch.isnan(x.max())


def test_act_quant_per_token_matches_numpy_float32():
    M, K = 9, 72
    x = randn_bf16((M, K), 11, 3.0)
    x[2] = 0                                  # all-zero row
    x[3, 5] = float("nan")                    # NaN in a row
    x[4, 1] = float("inf")
    x[5] *= 1e-30
    x[6, :] = torch.tensor([0.5, -0.5, 1.5, -1.5, 2.5, -2.5] * 12)  # ties (amax = 2.5: x * 50.8)
    x[7, :] = 127.0
    x[7, 3] = -63.5                            # -63.5 * (127 / 127) = -63.5: a tie, to even -64
    x8, sx = co.act_quant_i8_per_token(bits(x), M, K)
    xf = x.float().numpy()
    with np.errstate(all="ignore"):
        amax = np.abs(xf).max(axis=1)          # numpy's max propagates NaN
        want_sx = (amax / np.float32(127.0)).astype(np.float32)
        inv = np.where(amax == 0, np.float32(0), np.float32(127.0) / amax).astype(np.float32)
        r = np.rint(xf * inv[:, None])         # float32 product, half to even
        r = np.where(np.isnan(r), 0, np.clip(r, -128, 127)).astype(np.int8)
    assert np.array_equal(sx.view(np.uint32), want_sx.view(np.uint32))
    assert np.array_equal(x8.reshape(M, K), r)
    assert not x8.reshape(M, K)[2].any() and sx[2] == 0 and np.isnan(sx[3]) and not x8.reshape(M, K)[3].any()
    assert x8.reshape(M, K)[7, 3] == -64 and x8.reshape(M, K)[7, 0] == 127


# ---------------------------------------------------------------------- layout --
def test_gptq_layout_brute_force():
    N, K = 16, 128
    codes, packed, _, _ = make_w4(N, K, 10)
    gptq = co.native_to_gptq(packed.numpy(), N, K)
    for n, k in [(0, 0), (3, 7), (15, 127), (9, 64), (1, 9)]:
        assert (int(gptq[k // 8, n]) >> (4 * (k % 8))) & 15 == int(codes[n, k])
    assert np.array_equal(co.gptq_to_native(gptq, N, K), packed.numpy().view(np.uint8))


# ------------------------------------------- shortcuts of the fused Adam kernel --
def _bf16_rne_bits(x32: np.ndarray) -> np.ndarray:
    u = x32.view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint32)


def test_sqrt_of_bf16_rounds_the_same_within_two_ulps():
    """Every finite bf16 v >= 2^-100: all fp32 values within two ulps of the correctly rounded
    sqrt(v) round to the same bf16 value, so a one-ulp hardware square root may stand in for the
    correctly rounded one before the bf16 rounding (what the fused Adam kernel does)."""
    b = np.arange(0x0000, 0x7F80, dtype=np.uint32)  # all non-negative finite bf16 bit patterns
    v = (b << 16).view(np.float32)
    v = v[v >= np.float32(2.0 ** -100)]
    assert v.size > 28_000
    exact = np.sqrt(v)  # IEEE: correctly rounded in fp32
    want = _bf16_rne_bits(exact)
    for d in (-2, -1, 1, 2):
        near = (exact.view(np.int32) + d).view(np.float32)
        assert np.array_equal(_bf16_rne_bits(near), want), d
    # and the margin is wide: the closest approach to a rounding tie, in fp32 ulps
    frac = exact.view(np.uint32) & 0xFFFF
    assert int(np.abs(frac.astype(np.int64) - 0x8000).min()) > 8


def test_two_step_reciprocal_division_equals_ieee_division():
    """q0 = t*r, q1 = q0 + (t - q0*s)*r, q2 = q1 + (t - q1*s)*r with r = RN(1/s) returns RN(t/s):
    the quotient of the 8-bit moment quantiser (numerators in [0, 255*s], s >= 1e-10), checked on
    random and adversarial operands in float64-backed exact arithmetic."""
    rng = np.random.default_rng(5)
    n = 2_000_000
    s = np.exp(rng.uniform(np.log(1e-10), np.log(1e3), n)).astype(np.float32)
    # numerators: random in [0, 255 s], plus values next to rounding ties of the quotient
    q_target = rng.uniform(0, 255.5, n)
    q_target[: n // 2] = np.floor(q_target[: n // 2]) + 0.5
    t = (q_target * s.astype(np.float64)).astype(np.float32)
    t[: n // 4] = np.nextafter(t[: n // 4], np.float32(np.inf))
    t[n // 4: n // 2: 2] = np.nextafter(t[n // 4: n // 2: 2], np.float32(0))
    want = t / s  # IEEE fp32 division
    r = np.float32(1.0) / s

    def fma(a, b, c):  # exact product and sum in float64 (24 x 24 bits fit), one rounding to fp32
        return (a.astype(np.float64) * b.astype(np.float64) + c.astype(np.float64)).astype(np.float32)

    q0 = t * r
    q1 = fma(fma(-q0, s, t), r, q0)
    q2 = fma(fma(-q1, s, t), r, q1)
    assert np.array_equal(q2.view(np.uint32), want.view(np.uint32))


def test_quotient_of_bf16_rounds_the_same_within_three_ulps():
    """a / b for bf16 a, b: all fp32 values within three ulps of the correctly rounded quotient round
    to the same bf16 value (checked for every pair of significands; the exponents only shift the
    result), so the fused Adam kernel may form bf16(m / d) from a reciprocal and a product."""
    ma = np.arange(128, 256, dtype=np.float32)
    a, b = np.meshgrid(ma, ma, indexing="ij")
    q = (a / b).astype(np.float32).ravel()  # IEEE: correctly rounded, 2^-1 < q < 2
    want = _bf16_rne_bits(q)
    for d in (-3, -2, -1, 1, 2, 3):
        near = (q.view(np.int32) + d).view(np.float32)
        assert np.array_equal(_bf16_rne_bits(near), want), d
    frac = q.view(np.uint32) & 0xFFFF
    assert int(np.abs(frac.astype(np.int64) - 0x8000).min()) > 16  # distance to a tie, in fp32 ulps


# ------------------------------------------------------- 8-bit gradient accumulator --
@pytest.mark.parametrize("N,K,std", [(5, 64, 1e-3), (17, 264, 3.0), (3, 4096, 1e-6)])
def test_gradq8_oracle_matches_torch_bf16_tensor_ops(N, K, std):
    """The C restatement of GradientQTensor (bit = 8) against the chain of torch bf16 tensor
    operations the reference runs (oracle/torch_ref.py spells them as utils/quant.py:856-898 does),
    with the same injected noise: row scales and int8 values, for set_value and two add_ calls."""
    g = torch.Generator().manual_seed(N * 1000 + K)
    dws = [(torch.randn(N, K, generator=g) * std).to(torch.bfloat16) for _ in range(3)]
    dws[0][1] = 0  # an all-zero row takes the 1e-5 floor of the scale
    noises = [(torch.rand(N, K, generator=g) - 0.5).to(torch.bfloat16) for _ in range(3)]
    want_q, want_s = tr.gradq8_set(dws[0], noises[0])
    q, s = co.gradq8(bits(dws[0]), None, None, False, N, K, noise=bits(noises[0]))
    assert np.array_equal(s, bits(want_s).reshape(-1))
    assert np.array_equal(q, want_q.numpy().reshape(-1))
    for dw, nz in zip(dws[1:], noises[1:]):
        want_q = tr.gradq8_add(want_q, want_s, dw, nz)
        q, s2 = co.gradq8(bits(dw), q, s, True, N, K, noise=bits(nz))
        assert np.array_equal(s2, s) and np.array_equal(q, want_q.numpy().reshape(-1))
    assert np.abs(q.astype(int)).max() <= 128 and (q != 0).mean() > 0.5


def test_gradq8_nan_row_gives_nan_scale_as_the_tensor_chain():
    """A NaN in a row of dW: data.abs().amax() and torch.clamp keep it, so the row's scale (and with it the
    dequantised gradient) is NaN in the reference's chain; the restatement does the same, other rows are untouched."""
    N, K = 4, 64
    dw = randn_bf16((N, K), 2, 0.01)
    dw[2, 17] = float("nan")
    nz = (torch.rand(N, K, generator=torch.Generator().manual_seed(3)) - 0.5).to(torch.bfloat16)
    want_q, want_s = tr.gradq8_set(dw, nz)
    q, s = co.gradq8(bits(dw), None, None, False, N, K, noise=bits(nz))
    assert torch.isnan(want_s[2]).all() and np.isnan(co.bf16_bits_to_f32(s)[2])
    keep = [0, 1, 3]
    assert np.array_equal(s[keep], bits(want_s).reshape(-1)[keep])
    assert np.array_equal(q.reshape(N, K)[keep], want_q.numpy()[keep])


def test_gradq8_philox_noise_definition():
    """Without injected noise element i draws (2 b_i - 255) / 512, b_i = byte i & 3 of word (i >> 2) & 3 of the
    Philox block with counter offset + i / 16 (recomputed here from the pinned block function): 256 equally
    spaced bf16 numbers, symmetric about zero; the oracle's result equals the one with that noise injected."""
    N, K, seed, off = 4, 128, 99, 3
    nz = co.gradq8_noise(N * K, seed, off)
    for i in (0, 1, 3, 4, 15, 16, 17, 200, 511):
        c = off + i // 16
        blk = co.philox4x32_10([c & 0xFFFFFFFF, c >> 32, 0, 0], [seed & 0xFFFFFFFF, seed >> 32])
        b = (int(blk[(i >> 2) & 3]) >> (8 * (i & 3))) & 0xFF
        assert float(nz[i]) == (2 * b - 255) / 512
    noise = torch.from_numpy(nz).to(torch.bfloat16)
    assert np.array_equal(noise.float().numpy(), nz)  # every value is a bf16 number
    dw = randn_bf16((N, K), 1, 0.01)
    a, sa = co.gradq8(bits(dw), None, None, False, N, K, seed=seed, offset=off)
    b, sb = co.gradq8(bits(dw), None, None, False, N, K, noise=bits(noise))
    assert np.array_equal(a, b) and np.array_equal(sa, sb)
    big = co.gradq8_noise(1 << 16, 7, 0)
    assert float(np.abs(big).max()) == 255 / 512 and abs(float(big.mean())) < 0.005 and len(np.unique(big)) == 256


def test_bf16_quotient_of_bf16_numbers_from_the_reciprocal_product():
    """The gradient accumulator needs bf16(x / s) for bf16 numbers x and s and takes bf16(fl(x * RN(1/s))).
    Every pair of 8-bit significands (the exponents only shift the result): the product rounds to the same bf16
    number as the exact quotient, and the exact quotient keeps a relative distance of at least 2^-17 from
    every bf16 rounding tie, far more than the product's error of at most 2^-23."""
    from fractions import Fraction
    xs = np.arange(128, 256, dtype=np.float32)
    for e in (-20, 0, 13):
        S, X = np.meshgrid(xs * np.float32(2.0 ** e), xs, indexing="ij")
        r = (np.float32(1.0) / S).astype(np.float32)  # correctly rounded
        prod = (X * r).astype(np.float32)
        quo = (X.astype(np.float64) / S.astype(np.float64))  # 8-bit / 8-bit: the double is within 2^-53 of exact
        def bf16_rne(a32):
            u = a32.astype(np.float32).view(np.uint32).astype(np.uint64)
            return (((u + 0x7FFF + ((u >> 16) & 1)) >> 16) & 0xFFFF).astype(np.uint16)
        assert np.array_equal(bf16_rne(prod), bf16_rne(quo.astype(np.float32)))
    worst = 1.0
    for x in range(128, 256):
        for s_ in range(128, 256):
            qv = Fraction(x, s_)
            while qv < 256:
                qv *= 2
            while qv >= 512:
                qv /= 2
            # qv in [256, 512): bf16 ties are the odd integers here (9 significant bits)
            lo = (qv.numerator // qv.denominator)
            for t in (lo, lo + 1):
                if t % 2 == 1:
                    worst = min(worst, abs(qv - t) / qv)
    assert worst >= Fraction(1, 2 ** 17), float(worst)


# ------------------------------------------------------------- 4-bit residual codec --
CURVES = {0: (2, 0.125, 4, 0.25), 1: (2, 0.2666300266320331, 4, 0.375), 2: (2, 0.37272211741724515, 4, 0.4375),
          3: (2, 0.4330623539159437, 4, 0.46875)}  # three_fold_curve_4bit, utils/quant.py:708-716


@pytest.mark.parametrize("mu", [0, 1, 2, 3])
def test_residual_codec_against_an_exact_transcription_of_the_kernel(mu):
    """Every bf16 input with 2^-14 <= |x| <= 0.5 (and a sample of smaller ones) through a rational-
    arithmetic transcription of quant_kernel_bf, in both readings of `a*b + c` (fused, as nvcc
    compiles it by default, and unfused): the C oracle must equal the fused reading everywhere; the
    inputs on which the two readings differ are counted (a sign or centring mistake in the dither term
    would move thousands of levels, not a handful of ties). Dequantised values: all 16 nibbles."""
    from tests.golden import exact_model as em
    p1, y1, p2, y2 = CURVES[mu]
    k1, b1, k2, b2, k3 = p1, y1, p2 - p1, y2, 8 - p2
    cst = em.codec_constants(k1, b1, k2, b2, k3)
    mags = [b for b in range(0x3880, 0x3F01)] + [0, 1, 0x0080, 0x1234, 0x3000, 0x387F]  # 2^-14 .. 0.5, then small ones
    xb = np.array([m | sgn for m in mags for sgn in (0, 0x8000)], np.uint16)
    xb = np.concatenate([xb, np.zeros((-len(xb)) % 8, np.uint16)])
    q, carry = co.residual_quant(xb.copy(), 0, k1, b1, k2, b2, k3)
    nib = np.array([(int(w) >> (28 - 4 * k)) & 0xF for w in q for k in range(8)])
    differ = 0
    for i, b in enumerate(xb):
        x = em.frac_of_bf16_bits(int(b))
        lf = em.codec_level(x, cst, True)
        want_nib, want_carry = em.codec_nibble(lf)
        assert (nib[i], int(carry[i] == 0x3F80)) == (want_nib, want_carry), (hex(int(b)), lf)
        differ += em.codec_level(x, cst, False) != lf
    assert differ <= len(xb) // 100, differ  # the two readings part only where x*c + v sits on a rounding edge
    print(f"mu={mu}: fused and unfused readings differ on {differ} of {len(xb)} inputs")
    vals = co.residual_dequant(np.array([0x01234567, 0x89ABCDEF], np.uint32), 0, k1, b1, k2, b2, k3)
    for n in range(16):
        assert int(vals[n]) == em.bf16_bits_of_frac(em.codec_value(n, cst, True)), n
    # the dither v = S*499 - round(S*499) lies in [-1/2, 1/2]: it moves a level by at most one and in both
    # directions equally often (a dropped or one-sided dither term would show here)
    moved = []
    for m in range(0x3C00, 0x3F01, 3):
        for sgn in (0, 0x8000):
            x = em.frac_of_bf16_bits(m | sgn)
            plain = dict(cst)
            S = abs(x)
            if S < cst["b1"]:
                base = em.cround(f32(x * cst["c1"]))
            elif S < cst["b2"]:
                base = em.cround(f32(f32(S - cst["b1"]) * cst["c2"])) + cst["t1"]
                base = -base if x < 0 else base
            else:
                base = em.cround(f32(f32(S - cst["b2"]) * cst["c3"])) + cst["t2"]
                base = -base if x < 0 else base
            moved.append(em.codec_level(x, cst, True) - base)
    moved = np.array(moved)
    assert np.abs(moved).max() <= 1 and (moved != 0).mean() > 0.1 and abs(moved.mean()) < 0.08, (moved.mean(),)


def test_deterministic_uniform_quantiser_known_answers():
    """quant_kernel0 (multi_random_quant_kernel.cu:219-239): level = round-half-away(x * 8); levels above 7.5
    store nibble 1 and a carry, otherwise nibble level + 8. Known answers by hand, then every multiple of 1/64
    in [-1, 1] against exact rational arithmetic."""
    from fractions import Fraction
    import math
    x = np.array([0.0, 0.0625, -0.0625, 0.93, 0.9375, -0.5, 0.5, 0.124], np.float32)
    q, carry = co.residual_quant_s(x)
    #        0 -> 8   .5 -> 1 -> 9   -.5 -> -1 -> 7   7.44 -> 7 -> F   7.5 -> 8 -> carry   -4 -> 4   4 -> C   .992 -> 1 -> 9
    assert int(q[0]) == 0x897F14C9 and list(carry) == [0, 0, 0, 0, 1, 0, 0, 0]
    xs = np.arange(-64, 65, dtype=np.float32) / 64
    xs = np.concatenate([xs, np.zeros((-len(xs)) % 8, np.float32)])
    q, carry = co.residual_quant_s(xs)
    nib = [(int(w) >> (28 - 4 * k)) & 0xF for w in q for k in range(8)]
    for i, v in enumerate(xs):
        t = Fraction(float(v)) * 8
        lv = int(math.floor(abs(t) + Fraction(1, 2))) * (1 if t >= 0 else -1)
        want = (1, 1) if lv > 7 else (lv + 8, 0)
        assert (nib[i], int(carry[i])) == want, (float(v), lv)


def test_fp32_quotient_of_bf16_numbers_from_one_residual_correction():
    """The fused Adam kernels form m / d for bf16 m and d as q0 = m r, q = q0 + (m - q0 d) r with the hardware's
    reciprocal r (within one ulp of 1/d) and need the IEEE quotient. Every pair of 8-bit significands, r taken
    as RN(1/d) and as its two neighbours, in exact rational arithmetic: q equals RN(m/d); and the quotient's
    distance from the nearest midpoint of two fp32 numbers is at least 2^-33 (relative)."""
    from fractions import Fraction

    def rn32(fr):  # exact rational -> nearest fp32 (ties to even), as a Fraction; normal range only
        if fr == 0:
            return Fraction(0)
        sgn, a = (1 if fr > 0 else -1), abs(fr)
        e = a.numerator.bit_length() - a.denominator.bit_length()
        if Fraction(2) ** e > a:
            e -= 1
        scale = Fraction(2) ** (e - 23)
        n = a / scale  # in [2^23, 2^24)
        lo = n.numerator // n.denominator
        rem = n - lo
        if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and lo % 2 == 1):
            lo += 1
        return sgn * lo * scale

    worst = Fraction(1)
    for mi in range(128, 256):
        for di in range(128, 256, 1):
            m, d = Fraction(mi, 128), Fraction(di, 128) * 4  # the exponents only scale the result
            exact = m / d
            want = rn32(exact)
            r0 = rn32(1 / d)
            ulp_r = Fraction(2) ** (-23 - 3)  # ulp of a number in [1/8, 1/4)... r in (1/8, 1/4]
            for r in (r0 - ulp_r, r0, r0 + ulp_r):
                q0 = rn32(m * r)
                q = rn32(q0 + (m - q0 * d) * r)
                assert q == want, (mi, di, float(r - r0))
            # distance of the exact quotient from the nearest fp32 midpoint, relative
            e = exact.numerator.bit_length() - exact.denominator.bit_length()
            if Fraction(2) ** e > exact:
                e -= 1
            half = Fraction(2) ** (e - 24)
            n = exact / half  # midpoints are the odd integers here
            lo = n.numerator // n.denominator
            for t in (lo, lo + 1):
                if t % 2 == 1:
                    worst = min(worst, abs(n - t) * half / exact)
    assert worst >= Fraction(1, 2 ** 33), float(worst)


def test_round_half_away_as_trunc_of_a_sum():
    """The codec kernels take roundf(x) (halves away from zero) as trunc(x + copysign(pred(0.5), x)) in fp32.
    The same expression in numpy against the definition on 2^26 floats: every float in [0, 4), the neighbourhoods of
    all half-integers up to 2^12, of 2^22, 2^23 and 2^24, both signs, zeros, infinities."""
    half = np.float32(0.49999997)
    assert half == np.nextafter(np.float32(0.5), np.float32(0))

    def trick(x):
        return np.trunc((x + np.copysign(half, x)).astype(np.float32))

    def want(x):  # floor(|x| + 1/2) with the sign of x, exact in float64
        a = np.abs(x.astype(np.float64))
        return np.copysign(np.floor(a + 0.5), x).astype(np.float32)

    dense = np.arange(0, np.float32(4.0).view(np.uint32) + 1, dtype=np.uint32).view(np.float32)  # all floats in [0, 4]
    parts = [dense[::1] if len(dense) < (1 << 26) else dense[:: len(dense) >> 25]]
    for k in range(0, 4097):
        c = np.float32(k + 0.5).view(np.uint32)
        parts.append(np.arange(int(c) - 40, int(c) + 41, dtype=np.int64).astype(np.uint32).view(np.float32))
    for big in (2.0 ** 22, 2.0 ** 23, 2.0 ** 24, 3.0e38):
        c = np.float32(big).view(np.uint32)
        parts.append(np.arange(int(c) - 2000, int(c) + 2001, dtype=np.int64).astype(np.uint32).view(np.float32))
    parts.append(np.array([0.0, -0.0, np.inf, -np.inf, 0.5, 1.5, 2.5, 0.49999997, 0.50000006], np.float32))
    x = np.concatenate(parts)
    x = np.concatenate([x, -x])
    x = x[np.isfinite(x) | np.isinf(x)]
    got, ref = trick(x), want(x)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), x[got.view(np.uint32) != ref.view(np.uint32)][:10]


def test_w8_requant_oracle_matches_torch_bf16_tensor_ops():
    """Qfunc_8bit_res without a residual codec (utils/quant.py:88-103) as torch runs it on bf16 tensors on the CPU:
    q = t / qs; q.round_(); q.clamp_(-128, 127).to(int8), against the C restatement, with ties, saturating values
    and scales of both signs."""
    N, K = 12, 64
    lat = randn_bf16((N, K), 3, 0.05)
    qs = (torch.rand(N, 1, generator=torch.Generator().manual_seed(4)) * 1e-3 + 1e-4).to(torch.bfloat16)
    qs[3] = -qs[3]
    lat[0, :8] = (torch.tensor([0.5, 1.5, 2.5, -0.5, -1.5, 127.5, -128.5, 300.0]) * qs[0].float()).to(torch.bfloat16)
    lat[1, 0] = float("inf")
    lat[1, 1] = float("-inf")
    want = (lat / qs).round_().clamp_(-128, 127).to(torch.int8).numpy().reshape(-1)
    got = co.w8_requant(bits(lat), bits(qs), N, K)
    assert np.array_equal(got, want)
