"""Fused lbit=4 latent passes (lq_latent_w4_reconstruct / lq_latent_w4_requant) through the C ABI,
bit for bit against (a) the reference's chain of bf16 tensor operations run by torch on the CPU
around the C restatement of the residual codec (oracle/torch_ref.py) and (b) this package's own
unfused module path on the GPU, including whole optimizer steps."""
import numpy as np
import pytest
import torch

from tests.util import make_w4, randn_bf16

pytestmark = pytest.mark.gpu

CURVES = {0: (2, 0.125, 4, 0.25), 1: (2, 0.2666300266320331, 4, 0.375), 2: (2, 0.37272211741724515, 4, 0.4375),
          3: (2, 0.4330623539159437, 4, 0.46875)}


@pytest.fixture(scope="module")
def ops(hip_lib):
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from latentq_llm_amd import ops as _ops
    return _ops


@pytest.mark.parametrize("mu", [0, 1, 2, 3])
@pytest.mark.parametrize("N,K", [(8, 128), (40, 384), (256, 1024)])
def test_reconstruct_matches_the_tensor_op_chain(ops, N, K, mu):
    from oracle import torch_ref as tr
    p1, y1, p2, y2 = CURVES[mu]
    codes, packed, scales, zeros = make_w4(N, K, N + K + mu)
    g = torch.Generator().manual_seed(mu + 1)
    residual = torch.randint(-2 ** 31, 2 ** 31 - 1, (N * K // 8,), generator=g, dtype=torch.int64).to(torch.int32)
    want = tr.latent_w4_reconstruct(packed, scales, zeros, residual, (N, K), CURVES[mu])
    got = ops.latent_w4_reconstruct(packed.cuda(), scales.cuda(), zeros.cuda(), residual.cuda(), (N, K),
                                    p1, y1, p2 - p1, y2, 8 - p2)
    assert torch.equal(got.cpu().view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("mu", [0, 1, 2, 3])
@pytest.mark.parametrize("N,K", [(8, 128), (40, 384), (256, 1024)])
def test_requant_matches_the_tensor_op_chain(ops, N, K, mu):
    from oracle import torch_ref as tr
    p1, y1, p2, y2 = CURVES[mu]
    codes, packed, scales, zeros = make_w4(N, K, N + K + mu)
    # a latent that covers the whole code range, exact half-way points, carries and both clamps
    w = tr.dequant_4bit_g(packed, scales, zeros, (N, K)).float()
    s = scales.float().reshape(N, K // 128, 1).expand(N, K // 128, 128).reshape(N, K)
    noise = torch.rand((N, K), generator=torch.Generator().manual_seed(3)) - 0.5
    latent = w + noise * s * 1.2
    latent.view(-1)[::37] = (w + 0.5 * s).view(-1)[::37]
    latent.view(-1)[5::101] = (w + 40.0 * s).view(-1)[5::101]
    latent.view(-1)[7::103] = (w - 40.0 * s).view(-1)[7::103]
    latent = latent.to(torch.bfloat16)
    want_codes, want_res = tr.latent_w4_requant(latent, scales, zeros, (N, K), CURVES[mu])
    res = torch.empty(N * K // 8, dtype=torch.int32, device="cuda")
    got = ops.latent_w4_requant(latent.cuda(), scales.cuda(), zeros.cuda(), res, (N, K), p1, y1, p2 - p1, y2, 8 - p2)
    assert torch.equal(got.cpu().view(torch.uint8), want_codes.view(torch.uint8))
    assert torch.equal(res.cpu(), want_res)
    # and back: the reconstruction of what was just stored is close to the input (one residual step plus the
    # bf16 rounding of the latent itself, both well below a quarter of a code step)
    back = ops.latent_w4_reconstruct(got, scales.cuda(), zeros.cuda(), res, (N, K), p1, y1, p2 - p1, y2, 8 - p2)
    inside = (latent.float() >= (0 - zeros.float().reshape(N, -1, 1).expand(N, K // 128, 128).reshape(N, K)) * s) & \
             (latent.float() <= (15 - zeros.float().reshape(N, -1, 1).expand(N, K // 128, 128).reshape(N, K)) * s)
    err = ((back.float().cpu() - latent.float()).abs() / s)[inside]
    assert float(err.max()) <= 0.25, float(err.max())


@pytest.mark.parametrize("mu", [0, 1, 2, 3])
@pytest.mark.parametrize("N,K", [(8, 16), (40, 400), (256, 1024)])
def test_w8_latent_passes_match_the_tensor_op_chain(ops, N, K, mu):
    """8-bit weights with a 4-bit residual: reconstruct and re-quantise as single passes against the reference's chain
    of bf16 tensor operations on the CPU around the C codec, bit for bit; with saturating rows, exact halves, carries,
    a NaN, and scales outside the range of the reciprocal form."""
    from oracle import torch_ref as tr
    p1, y1, p2, y2 = CURVES[mu]
    g = torch.Generator().manual_seed(N + K + mu)
    codes = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int8)
    qs = ((torch.randn(N, 1, generator=g) * 0.01).abs() + 1e-3).to(torch.bfloat16)
    if N > 4:
        qs[2], qs[3] = 2.0 ** -50, 2.0 ** 45
    residual = torch.randint(-2 ** 31, 2 ** 31 - 1, (N * K // 8,), generator=g, dtype=torch.int64).to(torch.int32)
    want = tr.latent_w8_reconstruct(codes, qs, residual, CURVES[mu])
    got = ops.latent_w8_reconstruct(codes.cuda(), qs.cuda(), residual.cuda(), p1, y1, p2 - p1, y2, 8 - p2)
    assert torch.equal(got.cpu().view(torch.int16), want.view(torch.int16))
    noise = torch.rand((N, K), generator=g) - 0.5
    latent = (codes.float() + noise * 1.2) * qs.float()
    latent.view(-1)[::37] = ((codes.float() + 0.5) * qs.float()).view(-1)[::37]
    latent.view(-1)[5::101] = (300.0 * qs.float().expand(N, K)).reshape(-1)[5::101]
    latent.view(-1)[7::103] = (-300.0 * qs.float().expand(N, K)).reshape(-1)[7::103]
    latent = latent.to(torch.bfloat16)
    if N > 4:
        latent[4, 3] = float("nan")
    want_codes, want_res = tr.latent_w8_requant(latent.clone(), qs, CURVES[mu])
    res = torch.empty(N * K // 8, dtype=torch.int32, device="cuda")
    got_codes = ops.latent_w8_requant(latent.cuda(), qs.cuda(), res, p1, y1, p2 - p1, y2, 8 - p2)
    keep = ~torch.isnan(latent.float())
    assert torch.equal(got_codes.cpu()[keep], want_codes[keep])
    assert int(got_codes.cpu()[~keep].abs().sum()) == 0      # NaN -> code 0
    if bool(keep.all()):
        assert torch.equal(res.cpu(), want_res)
    else:
        words_ok = keep.view(-1, 8).all(dim=1)
        assert torch.equal(res.cpu()[words_ok], want_res[words_ok])


def _run_steps_w8(Q, fused, steps=4):
    Q.FUSED_LATENT = fused
    torch.manual_seed(0)
    N, K = 128, 256
    g = torch.Generator().manual_seed(5)
    w8 = torch.randint(-120, 121, (N, K), generator=g, dtype=torch.int8)
    qs = ((torch.randn(N, 1, generator=g) * 0.01).abs() + 2e-3).to(torch.bfloat16)
    layer = Q.QLinearA8W8(K, N, bias=False, lbit=4, gbit=16)
    layer.qscales.data = qs.clone()
    layer.weight.set_value(w8, layer.qscales)
    layer = layer.bfloat16().cuda()
    layer.to("cuda")
    layer.weight.requires_grad = True
    layer.add_hook()
    opt = Q.MyAdam([{"params": [layer.weight]}], lr=2e-3, betas=(0.9, 0.999), obit=16, mu_updata_f=20)
    x = randn_bf16((64, K), 11).cuda().requires_grad_(True)
    tgt = randn_bf16((64, N), 12).cuda()
    for _ in range(steps):
        y = layer(x)
        ((y.float() - tgt.float()) ** 2).mean().backward()
        opt.step()
    return layer.weight.data.clone().cpu(), layer.weight.residual.residual_int.clone().cpu(), w8


def test_optimizer_steps_on_8bit_weights_fused_equals_unfused(hip_lib, monkeypatch):
    from latentq_llm_amd import ops as O
    from latentq_llm_amd import quant as Q
    calls = {"reconstruct": 0, "requant": 0}
    rec, req = O.latent_w8_reconstruct, O.latent_w8_requant
    monkeypatch.setattr(O, "latent_w8_reconstruct", lambda *a, **k: (calls.__setitem__("reconstruct", calls["reconstruct"] + 1), rec(*a, **k))[1])
    monkeypatch.setattr(O, "latent_w8_requant", lambda *a, **k: (calls.__setitem__("requant", calls["requant"] + 1), req(*a, **k))[1])
    try:
        c1, r1, w8 = _run_steps_w8(Q, True)
        assert calls == {"reconstruct": 3, "requant": 4}  # the first step has no stored residual yet
        c0, r0, _ = _run_steps_w8(Q, False)
        assert calls == {"reconstruct": 3, "requant": 4}
    finally:
        Q.FUSED_LATENT = True
    assert torch.equal(c1, c0) and torch.equal(r1, r0)
    assert not torch.equal(c1, w8)  # the steps did move the weights


def _run_steps(Q, fused, steps=4):
    Q.FUSED_LATENT = fused
    torch.manual_seed(0)
    N, K = 128, 256
    codes, packed, scales, zeros = make_w4(N, K, 9)
    layer = Q.QLinearA16W4(K, N, bias=False, lbit=4, gbit=16)
    layer.zeros.data = zeros.clone()
    layer.scales.data = scales.clone()
    layer.weight.set_value(packed.clone(), [layer.scales, layer.zeros, layer.wshape])
    layer.to("cuda")
    layer.add_hook()
    opt = Q.MyAdam([{"params": [layer.weight]}], lr=2e-3, betas=(0.9, 0.999), obit=16, mu_updata_f=20)
    x = randn_bf16((64, K), 11).cuda().requires_grad_(True)
    tgt = randn_bf16((64, N), 12).cuda()
    for _ in range(steps):
        y = layer(x)
        ((y.float() - tgt.float()) ** 2).mean().backward()
        opt.step()
    return layer.weight.data.clone().cpu(), layer.weight.residual.residual_int.clone().cpu()


def test_optimizer_steps_fused_equals_unfused(hip_lib, monkeypatch):
    from latentq_llm_amd import ops as O
    from latentq_llm_amd import quant as Q
    calls = {"reconstruct": 0, "requant": 0}
    rec, req = O.latent_w4_reconstruct, O.latent_w4_requant
    monkeypatch.setattr(O, "latent_w4_reconstruct", lambda *a, **k: (calls.__setitem__("reconstruct", calls["reconstruct"] + 1), rec(*a, **k))[1])
    monkeypatch.setattr(O, "latent_w4_requant", lambda *a, **k: (calls.__setitem__("requant", calls["requant"] + 1), req(*a, **k))[1])
    try:
        c1, r1 = _run_steps(Q, True)
        assert calls == {"reconstruct": 3, "requant": 4}  # the first step has no stored residual yet
        c0, r0 = _run_steps(Q, False)
        assert calls == {"reconstruct": 3, "requant": 4}
    finally:
        Q.FUSED_LATENT = True
    assert torch.equal(c1, c0) and torch.equal(r1, r0)
    assert not torch.equal(c1, make_w4(128, 256, 9)[1])  # the steps did move the weights


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.float64, torch.bfloat16])
def test_deterministic_uniform_quantiser_bit_exact(dtype):
    """cuda_module.uniform_quant_s (no dither) on every tensor type the reference dispatches it for, and on bf16:
    words and carries equal the C restatement fed with the same values converted to float."""
    from latentq_llm_amd import quant as Q
    from oracle import c_oracle as co
    g = torch.Generator().manual_seed(11)
    n = 8 * 1000 + 8
    x = (torch.rand(n, generator=g, dtype=torch.float64) * 2.2 - 1.1)
    x[:9] = torch.tensor([0.0, 0.0625, -0.0625, 0.9375, 0.93749, -0.5, 0.5, 1.0, -1.0], dtype=torch.float64)
    x = x.to(dtype)
    want_q, want_c = co.residual_quant_s(x.to(torch.float32).numpy())
    xd = x.cuda()
    q = torch.empty(n // 8, dtype=torch.int32, device="cuda")
    Q.cuda_module.uniform_quant_s(xd, q)
    torch.cuda.synchronize()
    assert np.array_equal(q.cpu().numpy().view(np.uint32), want_q)
    assert xd.dtype == dtype and np.array_equal(xd.cpu().to(torch.float32).numpy(), want_c.astype(np.float32))
    # what the uniform dequantiser makes of the words is within half a step of the input where no carry was taken
    deq = Q.cuda_dequant_linear(q).reshape(-1).float().cpu()
    keep = (want_c == 0) & (x.abs().to(torch.float32).numpy() <= 1.0)
    assert float((deq.numpy()[keep] - x.to(torch.float32).numpy()[keep]).__abs__().max()) <= 0.0625 + 1e-6


@pytest.mark.parametrize("mode,mu", [(0, 0), (0, 1), (0, 2), (0, 3), (1, 0)])
def test_residual_codec_every_bf16_input(ops, mode, mu):
    """All 65 536 bf16 bit patterns (in range, out of range, infinities, NaN) through the codec kernel: packed words
    and carry flags equal the C restatement's, for the four three-segment curves and the uniform mode."""
    from oracle import c_oracle as co
    p1, y1, p2, y2 = CURVES[mu]
    args = (0, p1, y1, p2 - p1, y2, 8 - p2) if mode == 0 else (1,)
    xb = np.arange(65536, dtype=np.uint16)
    want_q, want_c = co.residual_quant(xb.copy(), *args)
    x = torch.from_numpy(xb.view(np.int16).copy()).view(torch.bfloat16).cuda()
    q = torch.empty(65536 // 8, dtype=torch.int32, device="cuda")
    ops.residual_quant(x, q, *args)
    torch.cuda.synchronize()
    got_q = q.cpu().numpy().view(np.uint32)
    got_c = x.cpu().view(torch.int16).numpy().view(np.uint16)
    bad = np.nonzero(got_q != want_q)[0]
    assert bad.size == 0, [(hex(int(w) * 8), hex(int(got_q[w])), hex(int(want_q[w]))) for w in bad[:5]]
    assert np.array_equal(got_c, want_c)
