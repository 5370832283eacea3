"""GPU tests of the 8-bit gradient accumulator (lq_gradq8_quant behind GradientQTensor) and of the
8-bit-weight optimizer update (Qfunc_8bit_res behind MyAdam), through the C ABI and the modules.

Bars: int8 values and bf16 row scales bit-exact against the C oracle (oracle/lq_oracle.c, itself
pinned against torch's bf16 tensor operations on the CPU) for injected and Philox noise, and
bit-exact against the tensor-op chain run on the GPU with the same injected noise.
"""
import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from oracle import torch_ref as tr
from tests.util import bits, make_w4, randn_bf16, rel_l2

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def Q(hip_lib):
    assert torch.cuda.is_available()
    from latentq_llm_amd import quant
    return quant


@pytest.fixture(scope="module")
def ops(hip_lib):
    from latentq_llm_amd import ops as _ops
    return _ops


def _noise(shape, seed):
    return (torch.rand(shape, generator=torch.Generator().manual_seed(seed)) - 0.5).to(torch.bfloat16)


@pytest.mark.parametrize("N,K,std", [(1, 16, 1.0), (7, 144, 1e-3), (33, 2048, 0.02), (16, 4112, 5.0), (4, 11008, 1e-6),
                                     (3, 12304, 0.3), (5, 4096, 0.1), (9, 1040, 2.0), (6, 1024, 1e-2)])
@pytest.mark.parametrize("mode", ["inject", "philox"])
def test_gradq8_set_and_add_bit_exact(ops, N, K, std, mode):
    dws = [randn_bf16((N, K), 50 + i, std) for i in range(3)]
    if N > 2:
        dws[0][1] = 0       # all-zero row: scale takes its floor
        dws[1][2] *= 64     # a micro-batch far above the first one's scale: saturates at +-127/-128
    q = torch.empty((N, K), dtype=torch.int8, device="cuda")
    s = torch.empty((N, 1), dtype=torch.bfloat16, device="cuda")
    want_q, want_s = None, None
    for i, dw in enumerate(dws):
        kw_o = {"noise": bits(_noise((N, K), 60 + i))} if mode == "inject" else {"seed": 5, "offset": 1000 * i}
        kw_h = {"noise": _noise((N, K), 60 + i).cuda()} if mode == "inject" else {"seed": 5, "offset": 1000 * i}
        want_q, want_s = co.gradq8(bits(dw), want_q, want_s, i > 0, N, K, **kw_o)
        ops.gradq8_quant(dw.cuda(), q, s, i > 0, **kw_h)
        assert np.array_equal(bits(s).reshape(-1), want_s), f"scales differ at micro-batch {i}"
        mism = int((q.cpu().numpy().reshape(-1) != want_q).sum())
        assert mism == 0, f"{mism} of {N * K} int8 values differ at micro-batch {i}"


@pytest.mark.parametrize("mode", ["inject", "philox"])
def test_gradq8_edge_values_and_scales(ops, mode):
    """NaN, infinities and huge or tiny magnitudes in dW; scales outside the range in which the kernel replaces the
    division (2^-40 .. 2^40), given to the accumulate form by hand and produced by a row of 1e20-sized values."""
    N, K = 8, 4112
    dw = randn_bf16((N, K), 70, 0.05)
    dw[0, 5] = float("nan")
    dw[1, 6] = float("inf")
    dw[1, 7] = float("-inf")
    dw[2] *= 1e20
    dw[3] *= 1e-30
    dw[4, 100] = 3e38
    dw[5, 9] = -1e-38
    kw_o = {"noise": bits(_noise((N, K), 71))} if mode == "inject" else {"seed": 9, "offset": 2 ** 40}
    kw_h = {"noise": _noise((N, K), 71).cuda()} if mode == "inject" else {"seed": 9, "offset": 2 ** 40}
    q = torch.empty((N, K), dtype=torch.int8, device="cuda")
    s = torch.empty((N, 1), dtype=torch.bfloat16, device="cuda")
    want_q, want_s = co.gradq8(bits(dw), None, None, False, N, K, **kw_o)
    ops.gradq8_quant(dw.cuda(), q, s, False, **kw_h)
    assert np.array_equal(bits(s).reshape(-1), want_s)
    assert np.array_equal(q.cpu().numpy().reshape(-1), want_q)
    # accumulate onto hand-made state with scales from 2^-60 to 2^60
    g = torch.Generator().manual_seed(72)
    q0 = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int8)
    s0 = torch.tensor([2.0 ** e for e in (-60, -41, -40, -1, 7, 40, 41, 60)], dtype=torch.bfloat16).reshape(N, 1)
    dw2 = randn_bf16((N, K), 73, 1.0) * s0.float().to(torch.bfloat16) * 30
    want_q, want_s = co.gradq8(bits(dw2), q0.numpy().reshape(-1).copy(), bits(s0).reshape(-1).copy(), True, N, K, **kw_o)
    qd, sd = q0.cuda(), s0.cuda()
    ops.gradq8_quant(dw2.cuda(), qd, sd, True, **kw_h)
    assert np.array_equal(bits(sd).reshape(-1), want_s)
    assert np.array_equal(qd.cpu().numpy().reshape(-1), want_q)


def test_gradq8_module_path_equals_the_tensor_op_chain_on_the_gpu(Q):
    """GradientQTensor.set_value / add_ through the HIP pass == the same object with FUSED_GRADQ off
    (torch tensor operations on the GPU), for the same injected noise."""
    N, K = 48, 1032
    dws = [randn_bf16((N, K), 70 + i, 0.05).cuda() for i in range(3)]
    nzs = [_noise((N, K), 80 + i).cuda() for i in range(3)]
    a, b = Q.GradientQTensor([N, K], bit=8), Q.GradientQTensor([N, K], bit=8)
    a.set_value(dws[0], noise=nzs[0])
    Q.FUSED_GRADQ = False
    try:
        b.set_value(dws[0], noise=nzs[0])
        for dw, nz in zip(dws[1:], nzs[1:]):
            b.add_(dw, noise=nz)
    finally:
        Q.FUSED_GRADQ = True
    for dw, nz in zip(dws[1:], nzs[1:]):
        a.add_(dw, noise=nz)
    assert a.acc_ite == b.acc_ite == 3
    assert torch.equal(a.scale, b.scale) and torch.equal(a.qdata, b.qdata)
    assert torch.equal(a.get_value(), b.get_value())
    total = sum(d.float() for d in dws)
    step = a.scale.float()
    assert float(((a.get_value().float() - total).abs() / step).max()) <= 3.0  # one rounding step per micro-batch


def test_gradq8_philox_rounding_is_unbiased(ops):
    """Mean of the dequantised int8 gradient over many noise offsets approaches the bf16 gradient."""
    N, K = 8, 256
    dw = randn_bf16((N, K), 90, 0.01).cuda()
    q = torch.empty((N, K), dtype=torch.int8, device="cuda")
    s = torch.empty((N, 1), dtype=torch.bfloat16, device="cuda")
    acc = torch.zeros((N, K), device="cuda")
    reps = 300
    for r in range(reps):
        ops.gradq8_quant(dw, q, s, False, seed=1234, offset=r * (N * K // 16))
        acc += q.float() * s.float()
    err = (acc / reps - dw.float()).abs() / s.float()
    assert float(err.max()) < 0.2  # in units of a quantisation step; a biased rounding would sit near 0.5


def test_qlinear_a16w4_with_8bit_gradient_accumulation(Q):
    """gbit = 8: the backward hook moves dW into the int8 accumulator (set_value, then add_), the
    hand-over list is drained, and the accumulated value stays within the 8-bit step of the bf16 sum."""
    N, K, M = 128, 256, 96
    codes, packed, scales, zeros = make_w4(N, K, 21)
    m = Q.QLinearA16W4(K, N, bias=False, lbit=0, gbit=8)
    m.zeros.data, m.scales.data, m.wshape = zeros.clone(), scales.clone(), [N, K]
    m.weight.set_value(packed, [m.scales, m.zeros, m.wshape])
    m = m.bfloat16().cuda()
    m.to("cuda")
    m.weight.requires_grad = True
    m.add_hook()
    g = m.weight.grad
    assert isinstance(g, Q.GradientQTensor) and g.acc_ite == 0
    x = randn_bf16((M, K), 22).cuda().requires_grad_(True)
    dys = [randn_bf16((M, N), 23 + i).cuda() for i in range(2)]
    used0 = Q.GradientQTensor._noise_offset
    want = torch.zeros((N, K), device="cuda")
    for i, dy in enumerate(dys):
        m(x).backward(dy)
        assert len(Q.dict_temp) == 0
        assert m.weight.grad is g and g.acc_ite == i + 1
        want += dy.float().t() @ x.detach().float()
        assert g.qdata.dtype == torch.int8 and g.qdata.shape == (N, K) and g.scale.shape == (N, 1)
        got = g.get_value()
        assert got.dtype == torch.bfloat16
        # each micro-batch adds at most one rounding step (|noise| <= 1/2 plus the bf16 roundings)
        assert float(((got.float() - want).abs() / g.scale.float()).max()) <= 1.5 * (i + 1)
    assert Q.GradientQTensor._noise_offset == used0 + 2 * (N * K // 16)
    assert rel_l2(g.get_value().float(), want) < 0.05
    # the optimizer consumes the dequantised value and resets the accumulator
    opt = Q.MyAdam([{"params": [m.weight], "weight_decay": 0.0}], lr=1e-3, betas=(0.9, 0.95), obit=8)
    before = m.weight.data.clone()
    opt.step()
    assert g.acc_ite == 0 and g.qdata is None and m.weight.grad is g
    assert (m.weight.data != before).any()


def test_8bit_accumulation_through_the_gemm_epilogue_equals_the_separate_pass(Q, ops):
    """With a multiple of 64 tokens the backward hook forms dW straight into the int8 accumulator from the second
    micro-batch on (GradientQTensor.add_product_: the weight-gradient GEMM's epilogue). The stored codes and scales
    equal, bit for bit, set_value / add_ applied to the separately formed bf16 products with the same noise stream."""
    N, K, M = 128, 256, 192
    codes, packed, scales, zeros = make_w4(N, K, 31)
    m = Q.QLinearA16W4(K, N, bias=False, lbit=0, gbit=8)
    m.zeros.data, m.scales.data, m.wshape = zeros.clone(), scales.clone(), [N, K]
    m.weight.set_value(packed, [m.scales, m.zeros, m.wshape])
    m = m.bfloat16().cuda()
    m.to("cuda")
    m.weight.requires_grad = True
    m.add_hook()
    x = randn_bf16((M, K), 32).cuda().requires_grad_(True)
    dys = [randn_bf16((M, N), 33 + i).cuda() for i in range(3)]
    cls = Q.GradientQTensor
    saved = (cls.noise_seed, cls._noise_offset)
    calls = []
    real = ops.weight_grad_acc8
    try:
        cls.noise_seed, cls._noise_offset = 4242, 1000
        ops.weight_grad_acc8 = lambda *a, **k: (calls.append(1), real(*a, **k))[1]
        for dy in dys:
            m(x).backward(dy)
        g = m.weight.grad
        assert g.acc_ite == 3 and len(calls) == 2 and len(Q.dict_temp) == 0
        # the same three micro-batches through the separate passes
        ref = cls([N, K], bit=8)
        cls.noise_seed, cls._noise_offset = 4242, 1000
        ref.set_value(ops.weight_grad(dys[0], x.detach()))
        for dy in dys[1:]:
            ref.add_(ops.weight_grad(dy, x.detach()))
        assert torch.equal(g.scale, ref.scale) and torch.equal(g.qdata, ref.qdata)
    finally:
        ops.weight_grad_acc8 = real
        cls.noise_seed, cls._noise_offset = saved


def test_fused_mlp_block_with_8bit_gradient_accumulators(Q, ops):
    """A QuantLlamaMLP of three gbit = 8 layers: the fused backward hands its three weight-gradient products to the
    layers' hooks (down, up, gate), the second micro-batch through the GEMM epilogue. Codes and scales equal, bit
    for bit, the separate passes on the same products with the same noise stream."""
    from latentq_llm_amd.fused_mlp import QuantLlamaMLP
    hid, ffn, M = 256, 384, 128

    def layer(n, k, seed):
        _, packed, scales, zeros = make_w4(n, k, seed)
        m = Q.QLinearA16W4(k, n, bias=False, lbit=0, gbit=8)
        m.zeros.data, m.scales.data, m.wshape = zeros.clone(), scales.clone(), [n, k]
        m.weight.set_value(packed, [m.scales, m.zeros, m.wshape])
        m = m.bfloat16().cuda()
        m.to("cuda")
        m.weight.requires_grad = True
        m.add_hook()
        return m

    gate, up, down = layer(ffn, hid, 41), layer(ffn, hid, 42), layer(hid, ffn, 43)
    mlp = QuantLlamaMLP(gate, down, up)
    x = randn_bf16((M, hid), 44).cuda().requires_grad_(True)
    dys = [randn_bf16((M, hid), 45 + i).cuda() for i in range(2)]
    cls = Q.GradientQTensor
    saved = (cls.noise_seed, cls._noise_offset)
    try:
        cls.noise_seed, cls._noise_offset = 777, 5000
        for dy in dys:
            mlp(x).backward(dy)
        assert len(Q.dict_temp) == 0
        for m in (gate, up, down):
            assert isinstance(m.weight.grad, cls) and m.weight.grad.acc_ite == 2
        # the same products through the separate passes, in the hooks' order
        w4 = lambda m: (m.weight.data, m.scales, m.zeros)
        refs = {id(m): cls([m.wshape[0], m.wshape[1]], bit=8) for m in (gate, up, down)}
        cls.noise_seed, cls._noise_offset = 777, 5000
        xd = x.detach()
        h, g, u = ops.a16w4_gate_up_silu(xd, w4(gate), w4(up), (ffn, hid), save=True)
        for i, dy in enumerate(dys):
            dg, du = ops.a16w4_dx_silu_bwd(dy, *w4(down), (hid, ffn), g, u)
            for m, dyl, xin in ((down, dy, h), (up, du, xd), (gate, dg, xd)):
                dw = ops.weight_grad(dyl, xin)
                (refs[id(m)].set_value if i == 0 else refs[id(m)].add_)(dw)
        for m in (gate, up, down):
            assert torch.equal(m.weight.grad.scale, refs[id(m)].scale)
            assert torch.equal(m.weight.grad.qdata, refs[id(m)].qdata)
    finally:
        cls.noise_seed, cls._noise_offset = saved


def test_noise_seed_follows_torch_manual_seed(Q):
    cls = Q.GradientQTensor
    saved = (cls.noise_seed, cls._noise_offset)
    try:
        cls.noise_seed = None
        torch.manual_seed(987654321)
        assert cls._seed() == 987654321 and cls.noise_seed == 987654321
    finally:
        cls.noise_seed, cls._noise_offset = saved


# --------------------------------------------------------------- 8-bit weights in the optimizer --
def _a8w8_layer(Q, N, K, lbit, seed):
    g = torch.Generator().manual_seed(seed)
    w8 = torch.randint(-120, 121, (N, K), generator=g, dtype=torch.int8)
    qs = ((torch.randn(N, 1, generator=g) * 0.01).abs() + 2e-3).to(torch.bfloat16)
    m = Q.QLinearA8W8(K, N, bias=False, lbit=lbit, gbit=16)
    m.qscales.data = qs.clone()
    m.weight.set_value(w8, m.qscales)
    latent = (w8.to(torch.int32) * qs).to(torch.bfloat16)
    if lbit != 4:
        m.weight.residual.data = latent.clone()  # main0.py:339-340
    m = m.bfloat16().cuda()
    m.to("cuda")
    m.weight.requires_grad = True
    m.add_hook()
    return m, w8, qs, latent


def _first_adam_step_cpu(latent, grad, lr, b1, b2, eps):
    """pdata after the first step of MyAdam.update_step (utils/quant.py:1081-1134) from zero moments,
    in torch's bf16 tensor arithmetic on the CPU."""
    exp_avg = (grad * 0).mul_(b1).add_(grad, alpha=1 - b1)
    exp_sq = (grad * 0).mul_(b2).addcmul_(grad, grad, value=1 - b2)
    denom = exp_sq.sqrt_().add_(eps)
    step_size = lr * (1 - b2) ** 0.5 / (1 - b1)
    return latent.clone().addcdiv_(exp_avg, denom, value=-step_size)


@pytest.mark.parametrize("lbit", [16, 0])
def test_myadam_on_8bit_weights_with_a_latent_copy(Q, lbit):
    """wbit = 8 with a latent copy (lbit 16, or lbit 0, the constructor default, filled as main0.py does): one step
    equals round(latent' / qscales) of the stepped latent (Qfunc_8bit_res, utils/quant.py:88-103) and
    stores the stepped latent."""
    N, K, M = 64, 256, 80  # < 65536 elements: bf16 moments, the tensor-op chain on the GPU
    m, w8, qs, latent = _a8w8_layer(Q, N, K, lbit, 31)
    # main0.py:340 assigns the bf16 dequantised weight to residual.data, which turns the fp32 placeholder
    # of lbit = 0 into a bf16 tensor too
    assert m.weight.residual.dtype == torch.bfloat16
    lr, b1, b2 = 2e-2, 0.9, 0.95
    opt = Q.MyAdam([{"params": [m.weight], "weight_decay": 0.0}], lr=lr, betas=(b1, b2), obit=8)
    x = randn_bf16((M, K), 32).cuda().requires_grad_(True)
    m(x).float().pow(2).mean().backward()
    grad = m.weight.grad.detach().cpu().clone()
    opt.step()
    pdata = _first_adam_step_cpu(latent, grad, lr, b1, b2, 1e-8)
    res = m.weight.residual.data
    assert res.dtype == torch.bfloat16
    # the stored latent is the stepped latent (CPU and GPU tensor kernels may differ in the last bf16 bit)
    stored = res.cpu().to(torch.bfloat16)
    assert torch.equal(stored.float(), res.float().cpu())  # an fp32 latent holds bf16 values
    # (a moment that differs in its last bf16 bit moves the update lr * m/d by up to lr * 2^-7)
    tol = pdata.float().abs() * 2.0 ** -7 + lr * 2.0 ** -6
    assert bool(((stored.float() - pdata.float()).abs() <= tol).all())
    assert rel_l2(stored.float(), pdata.float()) < 1e-3
    # and the codes are exactly the re-quantisation of that latent
    want_q, _ = tr.quant_8bit_res(stored, qs)
    got_q = m.weight.data.cpu()
    assert got_q.dtype == torch.int8 and torch.equal(got_q, want_q)
    assert (got_q != w8).float().mean() > 0.2  # the step moved codes
    assert m.weight.grad is None


def test_myadam_on_8bit_weights_with_the_4bit_residual(Q):
    """wbit = 8, lbit = 4 (per-channel ResidualTensor): codes are round(latent'/qscales) plus the
    codec's carry, and codes * qscales + residual reproduces the stepped latent to the codec's step."""
    N, K, M = 64, 256, 80
    m, w8, qs, latent = _a8w8_layer(Q, N, K, 4, 41)
    r = m.weight.residual
    assert isinstance(r, Q.ResidualTensor) and r.qshape == [N, K] and r.init
    lr, b1, b2 = 2e-2, 0.9, 0.95
    opt = Q.MyAdam([{"params": [m.weight], "weight_decay": 0.0}], lr=lr, betas=(b1, b2), obit=8)
    x = randn_bf16((M, K), 42).cuda().requires_grad_(True)
    m(x).float().pow(2).mean().backward()
    grad = m.weight.grad.detach().cpu().clone()
    opt.step()
    pdata = _first_adam_step_cpu(latent, grad, lr, b1, b2, 1e-8)  # the residual is empty on the first step
    base_q, frac = tr.quant_8bit_res(pdata, qs)
    got_q = m.weight.data.cpu()
    d = got_q.int() - base_q.int()
    assert set(d.unique().tolist()) <= {-1, 0, 1, 2} and float(((d == 0) | (d == 1)).float().mean()) > 0.998
    assert float((d == 1).float().mean()) > 0.005  # carries do occur (fractions that round up past level 7)
    assert not r.init and r.weight_scale is not None
    rebuilt = r.add((m.weight.data * m.weight.qparam).to(torch.bfloat16)).float().cpu()
    step = qs.float() / 16
    # one codec step, plus the bf16 roundings of code * scale, of the sum and of the CPU / GPU latents
    tol = 1.6 * step + 3 * pdata.float().abs() * 2.0 ** -8 + lr * 2.0 ** -6
    assert bool(((rebuilt - pdata.float()).abs() <= tol).all())
    assert rel_l2(rebuilt, pdata.float()) < 4e-3
    # a second step runs from the stored residual and keeps the codes in range
    m(x).float().pow(2).mean().backward()
    opt.step()
    assert int(m.weight.data.min()) >= -128 and int(m.weight.data.max()) <= 127
