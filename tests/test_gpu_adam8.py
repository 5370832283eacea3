"""Fused 8-bit Adam step against the chain of tensor operations it replaces (MyAdam.update_step,
reference utils/quant.py:1081-1134 with Qfunc_8bit_opt / DeQfunc_8bit_opt :22-41), on the GPU, bit
for bit over several consecutive steps: the moments, their per-block parameters and the updated
parameter (or the update direction) must all be identical."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    from latentq_llm_amd import ops as o
    return o


def chain_step(q, grad, state, step, lr, betas, eps, param=None):
    """The tensor-op chain, written with the same torch calls as latentq_llm_amd.quant.MyAdam.update_step."""
    beta1, beta2 = betas
    exp_avg = q.DeQfunc_8bit_opt(state["state1"], [state["qmap1"], state["absmax1"]]).to(grad.dtype)
    s2 = q.DeQfunc_8bit_opt(state["state2"], [state["qmap2"], state["absmax2"]])
    exp_avg_sq = (s2 * s2).to(grad.dtype)
    exp_avg.mul_(beta1).add_(grad, alpha=1 - beta1)
    exp_avg_sq.mul_(beta2).addcmul_(grad, grad, value=1 - beta2)
    exp_avg_sqrt = exp_avg_sq.sqrt_()
    denom = exp_avg_sqrt.add_(eps)
    step_size = lr * math.sqrt(1 - beta2 ** step) / (1 - beta1 ** step)
    if param is not None:
        param.addcdiv_(exp_avg, denom, value=-step_size)
        out = param
    else:
        out = (exp_avg / denom).to(torch.bfloat16)
    nblk = len(state["absmax1"])
    s1, qp = q.Qfunc_8bit_opt(exp_avg.float(), blocksize=nblk)
    state["state1"] = s1
    state["qmap1"], state["absmax1"] = qp
    s2q, qp = q.Qfunc_8bit_opt(exp_avg_sqrt.float(), blocksize=nblk)
    state["state2"] = s2q
    state["qmap2"], state["absmax2"] = qp
    return out, step_size


def fresh_state(n, nblk, dev):
    st = {"state1": torch.zeros(n, dtype=torch.uint8, device=dev), "state2": torch.zeros(n, dtype=torch.uint8, device=dev)}
    for name, fill in (("absmax1", 0.0), ("qmap1", 1e-10), ("absmax2", 0.0), ("qmap2", 1e-10)):
        st[name] = torch.full((nblk, 1), fill, dtype=torch.float32, device=dev)
    return st


@pytest.mark.parametrize("n,block", [(2048, 2048), (8192 * 64, 2048), (128 * 37, 128), (1024 * 1024, 2048)])
@pytest.mark.parametrize("with_param", [True, False])
def test_fused_adam8_equals_chain(ops, n, block, with_param):
    from latentq_llm_amd import quant as q
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(n + block)
    nblk = n // block
    ref = fresh_state(n, nblk, dev)
    fus = {k: v.clone() for k, v in ref.items()}
    p_ref = (torch.randn(n, generator=g) * 0.02).to(torch.bfloat16).to(dev)
    p_fus = p_ref.clone()
    lr, betas, eps = 1e-3, (0.9, 0.95), 1e-8
    for step in range(1, 7):
        # gradients with a wide dynamic range, some exact zeros and a few large outliers
        grad = (torch.randn(n, generator=g) * 10.0 ** torch.randint(-6, 0, (n,), generator=g).float())
        grad[::97] = 0.0
        grad[5::1001] *= 1e3
        grad = grad.to(torch.bfloat16).to(dev)
        want, step_size = chain_step(q, grad, ref, step, lr, betas, eps, p_ref if with_param else None)
        if with_param:
            got = ops.adam8_update(grad, fus["state1"], fus["state2"], fus["qmap1"], fus["absmax1"], fus["qmap2"],
                                   fus["absmax2"], betas[0], betas[1], eps, step_size, param=p_fus)
        else:
            got = torch.empty(n, dtype=torch.bfloat16, device=dev)
            ops.adam8_update(grad, fus["state1"], fus["state2"], fus["qmap1"], fus["absmax1"], fus["qmap2"],
                             fus["absmax2"], betas[0], betas[1], eps, step_size, direction=got)
        torch.cuda.synchronize()
        for name in ("qmap1", "absmax1", "qmap2", "absmax2"):
            assert torch.equal(ref[name].view(-1), fus[name].view(-1)), f"step {step}: {name} differs"
        for name in ("state1", "state2"):
            bad = int((ref[name].view(-1) != fus[name].view(-1)).sum())
            assert bad == 0, f"step {step}: {bad} of {n} codes of {name} differ"
        bad = int((want.view(torch.int16) != got.view(torch.int16)).sum())
        assert bad == 0, f"step {step}: {bad} of {n} output elements differ"


def _run_module_steps(Q, fused, lbit, steps=5):
    from tests.util import make_w4, randn_bf16
    Q.FUSED_ADAM8 = fused
    torch.manual_seed(0)
    N, K = 256, 512  # 131072 elements: large enough for uint8 moments (blocks of 2048)
    codes, packed, scales, zeros = make_w4(N, K, 9)
    layer = Q.QLinearA16W4(K, N, bias=False, lbit=lbit, gbit=16)
    layer.zeros.data = zeros.clone()
    layer.scales.data = scales.clone()
    layer.weight.set_value(packed.clone(), [layer.scales, layer.zeros, layer.wshape])
    layer.to("cuda")
    layer.add_hook()
    opt = Q.MyAdam([{"params": [layer.weight]}], lr=2e-3, betas=(0.9, 0.95), obit=8, mu_updata_f=20)
    x = randn_bf16((64, K), 11).cuda().requires_grad_(True)
    tgt = randn_bf16((64, N), 12).cuda()
    for _ in range(steps):
        y = layer(x)
        ((y.float() - tgt.float()) ** 2).mean().backward()
        opt.step()
    st = opt.state[layer.weight]
    assert st["state1"].dtype == torch.uint8
    res = getattr(layer.weight, "residual", None)
    res_words = res.residual_int.clone().cpu() if res is not None and hasattr(res, "residual_int") else torch.zeros(1)
    return (layer.weight.data.clone().cpu(), res_words, st["state1"].clone().cpu(), st["state2"].clone().cpu(),
            st["qmap1"].clone().cpu(), st["absmax1"].clone().cpu(), st["qmap2"].clone().cpu(), st["absmax2"].clone().cpu())


@pytest.mark.parametrize("lbit", [4, 0])
def test_optimizer_steps_with_fused_adam8_equal_the_chain(ops, monkeypatch, lbit):
    """Whole optimizer steps of the module path (latent mode lbit=4 and the stochastic-rounding mode
    lbit=0): codes, moments and block parameters identical with the fused kernels on and off, and
    the fused kernels are what ran: in latent mode the single-kernel step from the second step on
    (the first has no stored residual yet), otherwise the Adam kernel."""
    from latentq_llm_amd import ops as O
    from latentq_llm_amd import quant as Q
    calls = {"adam": 0, "step": 0}
    real_adam, real_step = O.adam8_update, O.adam8_latent_w4_step
    monkeypatch.setattr(O, "adam8_update", lambda *a, **k: (calls.__setitem__("adam", calls["adam"] + 1), real_adam(*a, **k))[1])
    monkeypatch.setattr(O, "adam8_latent_w4_step",
                        lambda *a, **k: (calls.__setitem__("step", calls["step"] + 1), real_step(*a, **k))[1])
    expect = {"adam": 1, "step": 4} if lbit == 4 else {"adam": 5, "step": 0}
    try:
        a = _run_module_steps(Q, True, lbit)
        assert calls == expect
        b = _run_module_steps(Q, False, lbit)
        assert calls == expect
    finally:
        Q.FUSED_ADAM8 = True
    for x, y in zip(a, b):
        assert torch.equal(x, y)


def test_fused_adam8_against_the_cpu_oracle(ops):
    """The same step on the CPU restatement (oracle/torch_ref.py). The CPU and GPU tensor libraries may
    contract a + alpha*b differently and divide by 255 differently (a true division on the CPU, a
    multiplication by the reciprocal on the GPU), and a moment that moves by one bf16 ulp can move its
    block's maximum with it; so the bar here is closeness: block parameters to 1 % (one bf16 ulp is
    0.4 %), moment codes within two steps of 255, outputs within one bf16 ulp."""
    from oracle import torch_ref as R
    dev = torch.device("cuda:0")
    n, block = 2048 * 24, 2048
    nblk = n // block
    g = torch.Generator().manual_seed(3)
    st = [torch.zeros(n, dtype=torch.uint8), torch.full((nblk, 1), 1e-10), torch.zeros(nblk, 1),
          torch.zeros(n, dtype=torch.uint8), torch.full((nblk, 1), 1e-10), torch.zeros(nblk, 1)]
    dst = [t.clone().to(dev) for t in st]
    p = (torch.randn(n, generator=g) * 0.02).to(torch.bfloat16)
    dp = p.clone().to(dev)
    for step in range(1, 5):
        grad = (torch.randn(n, generator=g) * 1e-3).to(torch.bfloat16)
        step_size = 1e-3 * math.sqrt(1 - 0.95 ** step) / (1 - 0.9 ** step)
        p, new = R.adam8_step(grad, st[0], st[1], st[2], st[3], st[4], st[5], 0.9, 0.95, 1e-8, step_size, param=p)
        st = list(new)
        ops.adam8_update(grad.to(dev), dst[0], dst[3], dst[1], dst[2], dst[4], dst[5], 0.9, 0.95, 1e-8, step_size, param=dp)
        for i in (1, 2, 4, 5):
            assert torch.allclose(dst[i].cpu(), st[i], rtol=1e-2, atol=1e-12)
        for i in (0, 3):
            assert int((dst[i].cpu().int() - st[i].int()).abs().max()) <= 2
        assert torch.allclose(dp.cpu().float(), p.float(), rtol=2.0 ** -7, atol=step_size * 2.0 ** -5)
        # carry on from the oracle's state so that differences do not accumulate
        dst = [t.clone().to(dev) for t in st]
        dp = p.clone().to(dev)


@pytest.mark.parametrize("N,K,block", [(64, 2048, 2048), (257, 384, 128), (1024, 4096, 2048)])
def test_single_kernel_latent_step_equals_the_three_passes(ops, N, K, block):
    """lq_adam8_latent_w4_step against lq_latent_w4_reconstruct -> lq_adam8_update -> lq_latent_w4_requant,
    with different curves for the stored residual and for the new one (as after an update of the
    codec's range), over several steps: codes, residual words, moments and block parameters identical."""
    from latentq_llm_amd import quant as q
    from tests.util import make_w4
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(N + K)
    n = N * K
    nblk = n // block
    codes, packed, scales, zeros = make_w4(N, K, 5)
    scales, zeros = scales.to(dev).view(-1), zeros.to(dev).view(-1)
    res = torch.randint(-2**31, 2**31 - 1, (n // 8,), generator=g, dtype=torch.int64).to(torch.int32).to(dev)
    a = {"codes": packed.clone().to(dev), "res": res.clone(), **fresh_state(n, nblk, dev)}
    b = {"codes": packed.clone().to(dev), "res": res.clone(), **fresh_state(n, nblk, dev)}

    def curve(mu):
        p1, y1, p2, y2 = q.three_fold_curve_4bit(mu)
        return (p1, y1, p2 - p1, y2, 8 - p2)
    curves = [curve(0), curve(1), curve(1), curve(2), curve(0)]
    for step in range(1, 5):
        grad = (torch.randn(n, generator=g) * 10.0 ** torch.randint(-5, -1, (n,), generator=g).float()).to(torch.bfloat16).to(dev)
        step_size = 2e-3 * math.sqrt(1 - 0.95 ** step) / (1 - 0.9 ** step)
        dq, qq = curves[step - 1], curves[step]
        latent = ops.latent_w4_reconstruct(a["codes"], scales, zeros, a["res"], (N, K), *dq)
        ops.adam8_update(grad, a["state1"], a["state2"], a["qmap1"], a["absmax1"], a["qmap2"], a["absmax2"],
                         0.9, 0.95, 1e-8, step_size, param=latent.view(-1))
        a["codes"] = ops.latent_w4_requant(latent, scales, zeros, a["res"], (N, K), *qq)
        ops.adam8_latent_w4_step(grad, b["codes"], b["res"], scales, zeros, (N, K), b["state1"], b["state2"], b["qmap1"],
                                 b["absmax1"], b["qmap2"], b["absmax2"], dq, qq, 0.9, 0.95, 1e-8, step_size)
        torch.cuda.synchronize()
        for name in a:
            assert torch.equal(a[name].view(-1), b[name].view(-1)), f"step {step}: {name} differs"
    assert not torch.equal(b["codes"].cpu(), packed)


@pytest.mark.parametrize("N,K,block", [(64, 2048, 2048), (200, 320, 128), (1024, 4096, 2048)])
def test_single_kernel_w8_latent_step_equals_the_three_passes(ops, N, K, block):
    """lq_adam8_latent_w8_step against lq_latent_w8_reconstruct -> lq_adam8_update -> lq_latent_w8_requant on an
    8-bit-weight layer (scales of both signs, one outside the range of the reciprocal product), with different curves
    for the stored residual and for the new one, over several steps: codes, residual words, moments and block
    parameters identical."""
    from latentq_llm_amd import quant as q
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(N + K)
    n = N * K
    nblk = n // block
    codes = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int8)
    qs = ((torch.randn(N, generator=g) * 0.01).abs() + 1e-3).to(torch.bfloat16)
    qs[3] = -qs[3]
    qs[5] = 2.0 ** -50
    qs = qs.to(dev)
    res = torch.randint(-2**31, 2**31 - 1, (n // 8,), generator=g, dtype=torch.int64).to(torch.int32).to(dev)
    a = {"codes": codes.clone().to(dev), "res": res.clone(), **fresh_state(n, nblk, dev)}
    b = {"codes": codes.clone().to(dev), "res": res.clone(), **fresh_state(n, nblk, dev)}

    def curve(mu):
        p1, y1, p2, y2 = q.three_fold_curve_4bit(mu)
        return (p1, y1, p2 - p1, y2, 8 - p2)
    curves = [curve(0), curve(1), curve(1), curve(2), curve(0)]
    for step in range(1, 5):
        grad = (torch.randn(n, generator=g) * 10.0 ** torch.randint(-5, -1, (n,), generator=g).float()).to(torch.bfloat16).to(dev)
        step_size = 2e-3 * math.sqrt(1 - 0.95 ** step) / (1 - 0.9 ** step)
        dq, qq = curves[step - 1], curves[step]
        latent = ops.latent_w8_reconstruct(a["codes"], qs, a["res"], *dq)
        ops.adam8_update(grad, a["state1"], a["state2"], a["qmap1"], a["absmax1"], a["qmap2"], a["absmax2"],
                         0.9, 0.95, 1e-8, step_size, param=latent.view(-1))
        a["codes"] = ops.latent_w8_requant(latent, qs, a["res"], *qq)
        ops.adam8_latent_w8_step(grad, b["codes"], b["res"], qs, b["state1"], b["state2"], b["qmap1"], b["absmax1"],
                                 b["qmap2"], b["absmax2"], dq, qq, 0.9, 0.95, 1e-8, step_size)
        torch.cuda.synchronize()
        for name in a:
            assert torch.equal(a[name].view(-1), b[name].view(-1)), f"step {step}: {name} differs"
    assert not torch.equal(b["codes"].cpu(), codes)


def _run_w8_module_steps(Q, fused, steps=5):
    from tests.util import randn_bf16
    Q.FUSED_ADAM8 = fused
    Q.FUSED_LATENT = fused
    torch.manual_seed(0)
    N, K = 256, 512
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
    opt = Q.MyAdam([{"params": [layer.weight]}], lr=2e-3, betas=(0.9, 0.95), obit=8, mu_updata_f=20)
    x = randn_bf16((64, K), 11).cuda().requires_grad_(True)
    tgt = randn_bf16((64, N), 12).cuda()
    for _ in range(steps):
        y = layer(x)
        ((y.float() - tgt.float()) ** 2).mean().backward()
        opt.step()
    st = opt.state[layer.weight]
    assert st["state1"].dtype == torch.uint8
    return (layer.weight.data.clone().cpu(), layer.weight.residual.residual_int.clone().cpu(), st["state1"].clone().cpu(),
            st["state2"].clone().cpu(), st["qmap1"].clone().cpu(), st["absmax1"].clone().cpu(), st["qmap2"].clone().cpu(),
            st["absmax2"].clone().cpu()), w8


def test_optimizer_steps_on_8bit_weights_with_uint8_moments(ops, monkeypatch):
    """Whole optimizer steps of an 8-bit-weight layer in lbit = 4 mode with uint8 moments: the single-kernel step
    runs from the second step on (the first has no stored residual yet), and codes, residual words, moments and block
    parameters equal those of the chain of tensor operations."""
    from latentq_llm_amd import ops as O
    from latentq_llm_amd import quant as Q
    calls = {"step": 0}
    real_step = O.adam8_latent_w8_step
    monkeypatch.setattr(O, "adam8_latent_w8_step",
                        lambda *a, **k: (calls.__setitem__("step", calls["step"] + 1), real_step(*a, **k))[1])
    try:
        a, w8 = _run_w8_module_steps(Q, True)
        assert calls == {"step": 4}
        b, _ = _run_w8_module_steps(Q, False)
        assert calls == {"step": 4}
    finally:
        Q.FUSED_ADAM8 = True
        Q.FUSED_LATENT = True
    for x, y in zip(a, b):
        assert torch.equal(x, y)
    assert not torch.equal(a[0], w8)
