"""GPU tests of the module API (the drop-in for the reference's utils/quant.py) and of the 4-bit
residual codec, against the torch-CPU restatement of the reference path and the C oracle."""
import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from oracle import torch_ref as tr
from tests.util import bits, from_bits, make_w4, randn_bf16, rel_l2

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def Q(hip_lib):
    assert torch.cuda.is_available()
    from latentq_llm_amd import quant
    return quant


def _make_w4_layer(Q, N, K, seed, bias, lbit, train):
    codes, packed, scales, zeros = make_w4(N, K, seed)
    m = Q.QLinearA16W4(K, N, bias=bias, lbit=lbit, gbit=16)
    m.zeros.data = zeros.clone()
    m.scales.data = scales.clone()
    m.wshape = [N, K]
    m.weight.set_value(packed, [m.scales, m.zeros, m.wshape])
    if bias:
        m.bias.data = randn_bf16((N,), seed + 5).float()
    m = m.bfloat16().cuda()  # nn.Module part (buffers, bias) ...
    m.to("cuda")             # ... then the QuantTensor, as main0.py:499-504 does
    if train:
        m.weight.requires_grad = True
        m.add_hook()
    return m, (packed, scales, zeros)


@pytest.mark.parametrize("lead,N,K,bias", [((4, 40), 256, 384, True), ((300,), 128, 256, False), ((3,), 64, 128, True)])
def test_qlinear_a16w4_forward_backward(Q, lead, N, K, bias):
    m, (packed, scales, zeros) = _make_w4_layer(Q, N, K, 3, bias, lbit=16, train=True)
    x_cpu = randn_bf16(lead + (K,), 4)
    x = x_cpu.cuda().requires_grad_(True)
    y = m(x)
    assert y.shape == lead + (N,) and y.dtype == torch.bfloat16
    b_cpu = None if not bias else m.bias.detach().cpu()
    want_y = tr.w4_forward(x_cpu.reshape(-1, K), packed, scales, zeros, (N, K), b_cpu)
    assert rel_l2(y.detach().float().cpu().reshape(-1, N), want_y.float()) < 1e-2
    dy_cpu = randn_bf16(lead + (N,), 6)
    y.backward(dy_cpu.cuda())
    want_dx, want_dw, _ = tr.w4_backward(dy_cpu.reshape(-1, N), x_cpu.reshape(-1, K), packed, scales, zeros, (N, K))
    assert rel_l2(x.grad.float().cpu().reshape(-1, K), want_dx.float()) < 1e-2
    assert len(Q.dict_temp) == 0, "the backward hook must have consumed dW"
    assert m.weight.grad.shape == (N, K)
    assert rel_l2(m.weight.grad.float().cpu(), want_dw.float()) < 1e-2
    if bias:
        assert m.bias.grad is None  # the reference never produces a bias gradient (flag of the wrong argument)
    # second backward accumulates into weight.grad
    g0 = m.weight.grad.clone()
    m(x).backward(dy_cpu.cuda())
    assert rel_l2(m.weight.grad.float(), 2 * g0.float()) < 1e-2


def test_qlinear_a16w4_eval_and_decode(Q):
    m, (packed, scales, zeros) = _make_w4_layer(Q, 256, 512, 7, True, lbit=16, train=False)
    for tokens in (1, 5, 40):
        x = randn_bf16((tokens, 512), tokens)
        with torch.no_grad():
            y = m(x.cuda())
            y2 = m.forward_eval(x.cuda())
        assert torch.equal(y, y2)
        want = tr.w4_forward(x, packed, scales, zeros, (256, 512), m.bias.detach().cpu())
        assert rel_l2(y.float().cpu(), want.float()) < 1e-2
    m.before_save()
    assert m.qweight.device.type == "cpu" and torch.equal(m.qweight, packed)


def test_dequant_function(Q):
    N, K = 96, 256
    codes, packed, scales, zeros = make_w4(N, K, 8)
    w = Q.DeQfunc_4bit_g(packed.cuda(), [scales.cuda(), zeros.cuda(), [N, K]], torch.bfloat16)
    assert np.array_equal(bits(w), bits(tr.dequant_4bit_g(packed, scales, zeros, (N, K))))


@pytest.mark.parametrize("train", [False, True])
def test_qlinear_a8w8(Q, train):
    N, K, M = 128, 256, 70
    g = torch.Generator().manual_seed(1)
    w8 = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8)
    qs = ((torch.randn(N, 1, generator=g) * 0.01).abs() + 1e-3).to(torch.bfloat16)
    m = Q.QLinearA8W8(K, N, bias=True, lbit=16, gbit=16)
    m.qscales.data = qs.clone()
    m.bias.data = randn_bf16((N,), 2).float()
    m.weight.set_value(w8, m.qscales)
    m = m.bfloat16().cuda()
    m.to("cuda")
    if train:
        m.weight.requires_grad = True
        m.add_hook()
    x_cpu = randn_bf16((M, K), 3)
    x = x_cpu.cuda().requires_grad_(train)
    y = m(x)
    want, x8, clampv = tr.a8w8_forward_dynamic(x_cpu, w8, qs, m.bias.detach().cpu())
    err = rel_l2(y.detach().float().cpu(), want.float())
    print(f"a8w8 module rel_l2={err:.3e} (epilogue rounding of the external cutlass kernel is unpinned)")
    assert err < 1e-2
    if train:
        dy = randn_bf16((M, N), 4)
        y.backward(dy.cuda())
        want_dx, want_dw = tr.a8w8_backward(dy, x8, clampv, w8, qs)
        assert rel_l2(x.grad.float().cpu(), want_dx.float()) < 1e-2
        assert rel_l2(m.weight.grad.float().cpu(), want_dw.float()) < 1e-2


def _a8w8_layer(Q, N, K, seed, bias=True):
    g = torch.Generator().manual_seed(seed)
    w8 = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8)
    qs = ((torch.randn(N, 1, generator=g) * 0.01).abs() + 1e-3).to(torch.bfloat16)
    m = Q.QLinearA8W8(K, N, bias=bias, lbit=16, gbit=16)
    m.qscales.data = qs.clone()
    if bias:
        m.bias.data = randn_bf16((N,), seed + 1).float()
    m.weight.set_value(w8, m.qscales)
    m = m.bfloat16().cuda()
    m.to("cuda")
    return m, w8, qs


def test_qlinear_a8w8_forward_runs_library_kernels_only(Q):
    """The forward of an A8W8 layer (eval and training Function) dispatches no tensor-library operator that launches
    a kernel: the activation maximum, the quantiser, the per-row scales and the scaled int8 GEMM are the library's."""
    from torch.utils._python_dispatch import TorchDispatchMode

    class Record(TorchDispatchMode):
        def __init__(self):
            super().__init__()
            self.names = []

        def __torch_dispatch__(self, func, types, args=(), kwargs=None):
            self.names.append(str(func))
            return func(*args, **(kwargs or {}))

    free = ("aten.empty", "aten.view", "aten.reshape", "aten._unsafe_view", "aten.detach", "aten.alias", "aten.t.",
            "aten._reshape_alias", "aten.select", "aten.slice", "aten.unsqueeze", "aten.expand", "aten.as_strided",
            "aten.is_pinned", "aten.lift_fresh", "aten.new_empty")
    for train in (False, True):
        m, _, _ = _a8w8_layer(Q, 128, 256, 11)
        if train:
            m.weight.requires_grad = True
            m.add_hook()
        x = randn_bf16((70, 256), 3).cuda().requires_grad_(train)
        with Record() as rec:
            y = m(x)
        launching = [n for n in rec.names if not n.startswith(free)]
        assert launching == [], launching
        assert y.shape == (70, 128)


def test_qlinear_a8w8_per_token(Q):
    """act_quant = "per_token": forward against the float64 product of the per-token-quantised activations and the
    dequantised weights, backward against the dense products on the same operands."""
    N, K, M = 128, 256, 70
    m, w8, qs = _a8w8_layer(Q, N, K, 21)
    m.act_quant = "per_token"
    m.weight.requires_grad = True
    m.add_hook()
    x_cpu = randn_bf16((M, K), 3)
    x_cpu[5] *= 30.0
    x = x_cpu.cuda().requires_grad_(True)
    y = m(x)
    x8, sx = co.act_quant_i8_per_token(bits(x_cpu), M, K)
    xq = torch.from_numpy(x8.reshape(M, K).astype(np.float64)) * torch.from_numpy(sx.astype(np.float64))[:, None]
    wf = w8.double() * qs.double()
    want = xq @ wf.t() + m.bias.detach().double().cpu()
    assert rel_l2(y.detach().float().cpu(), want) < 5e-3
    with torch.no_grad():
        assert torch.equal(m.forward_eval(x), y.detach())
    dy = randn_bf16((M, N), 4)
    y.backward(dy.cuda())
    assert rel_l2(x.grad.float().cpu(), dy.double() @ wf) < 1e-2
    assert rel_l2(m.weight.grad.float().cpu(), dy.double().t() @ xq) < 1e-2


def test_qlinear_a8w8_backward_from_codes_equals_dense_path(Q):
    """The A8W8 training Function's input gradient comes from the int8 codes (lq_a8w8_dx); with the switch off the
    dequantised weight is materialised and multiplied densely, as the reference does: same result within the fp32
    accumulation order."""
    N, K, M = 256, 384, 200
    m, w8, qs = _a8w8_layer(Q, N, K, 31, bias=False)
    m.weight.requires_grad = True
    m.add_hook()
    x_cpu, dy = randn_bf16((M, K), 3), randn_bf16((M, N), 4).cuda()
    grads = []
    for fused in (True, False):
        Q.FUSED_A8W8_DX = fused
        try:
            x = x_cpu.cuda().requires_grad_(True)
            m.weight.grad = None
            m(x).backward(dy)
            grads.append(x.grad.clone())
        finally:
            Q.FUSED_A8W8_DX = True
    assert rel_l2(grads[0].float(), grads[1].float()) < 3e-3
    wf = (w8.to(torch.bfloat16) * qs).to(torch.bfloat16).double()
    assert rel_l2(grads[0].cpu(), dy.cpu().double() @ wf) < 4e-3


def test_qlinear_qat_forward(Q):
    N, K, M = 64, 128, 33
    m = Q.QLinearQAT(K, N, bias=False, lbit=16, gbit=16)
    wf = randn_bf16((N, K), 5, 0.05)
    m.qscales.data = (wf.float().abs().amax(dim=1, keepdim=True) / 127).to(torch.bfloat16)
    m.weight.data = wf.clone()
    m = m.bfloat16().cuda()
    m.to("cuda")
    x = randn_bf16((M, K), 6)
    with torch.no_grad():
        y = m(x.cuda())
    w8 = (wf / m.qscales.cpu()).round_().clamp_(-128, 127).to(torch.int8)
    want, _, _ = tr.a8w8_forward_dynamic(x, w8, m.qscales.cpu())
    assert rel_l2(y.float().cpu(), want.float()) < 1e-2


def test_qlinear_qat_training_step_on_library_kernels_equals_the_tensor_chain(Q):
    """QLinearQAT forward + backward: with the weight quantised by the one-pass kernel and the input gradient formed
    from the int8 codes, against the same layer on the tensor-operation chain. Output and weight gradient identical
    bit for bit (same codes, same operands); the input gradient within the reduction-order tolerance."""
    N, K, M = 128, 256, 192
    wf = randn_bf16((N, K), 5, 0.05)
    qs = (wf.float().abs().amax(dim=1, keepdim=True) / 127).to(torch.bfloat16)
    x0 = randn_bf16((M, K), 6)
    dy = randn_bf16((M, N), 7).cuda()

    def run(fused):
        saved = (Q.FUSED_LATENT, Q.FUSED_A8W8_DX)
        Q.FUSED_LATENT, Q.FUSED_A8W8_DX = fused, fused
        try:
            m = Q.QLinearQAT(K, N, bias=False, lbit=16, gbit=16)
            m.qscales.data = qs.clone()
            m.weight.data = wf.clone()
            m = m.bfloat16().cuda()
            m.to("cuda")
            m.weight.requires_grad = True
            m.add_hook()
            x = x0.cuda().requires_grad_(True)
            y = m(x)
            y.backward(dy)
            assert len(Q.dict_temp) == 0
            return y.detach(), x.grad.detach(), m.weight.grad.detach()
        finally:
            Q.FUSED_LATENT, Q.FUSED_A8W8_DX = saved

    y1, dx1, dw1 = run(True)
    y0, dx0, dw0 = run(False)
    assert torch.equal(y1, y0) and torch.equal(dw1, dw0)
    assert rel_l2(dx1.float(), dx0.float()) < 3e-3
    w8 = (wf / qs).round_().clamp_(-128, 127)
    want_dx = dy.double().cpu() @ (w8 * qs).to(torch.bfloat16).double()
    assert rel_l2(dx1.float().cpu(), want_dx) < 3e-3


# ------------------------------------------------------------------ residual codec ----------
@pytest.mark.parametrize("mu", [0, 1, 2, 3])
def test_residual_codec_3fold_bit_exact(Q, mu):
    from latentq_llm_amd import ops
    k1, b1, p2, b2 = Q.three_fold_curve_4bit(mu)
    g = torch.Generator().manual_seed(mu)
    x = (torch.rand(4096 * 8, generator=g) - 0.5).to(torch.bfloat16)
    x[:16] = torch.tensor([0.5, -0.5, 0.0, b1, -b1, b2, -b2, 0.499, -0.499, 0.25, 0.125, -0.125, 0.4375, 0.0625, 1e-3, -1e-3])
    want_q, want_c = co.residual_quant(bits(x), 0, k1, b1, p2 - k1, b2, 8 - p2)
    xg = x.cuda()
    q = torch.empty(4096, dtype=torch.int32, device="cuda")
    ops.residual_quant(xg, q, 0, k1, b1, p2 - k1, b2, 8 - p2)
    assert np.array_equal(q.cpu().numpy().view(np.uint32), want_q)
    assert np.array_equal(bits(xg), want_c)
    back = ops.residual_dequant(q, 0, k1, b1, p2 - k1, b2, 8 - p2)
    assert np.array_equal(bits(back).reshape(-1), co.residual_dequant(want_q, 0, k1, b1, p2 - k1, b2, 8 - p2))
    # reconstruction error bounded by half a step of the coarsest segment (+ bf16 rounding)
    rec = back.float().cpu().reshape(-1) + from_bits(want_c).float()  # a carry means "+1 to the code"
    step = max(b1 / k1, (b2 - b1) / (p2 - k1), (0.5 - b2) / (8 - p2))
    assert float((rec - x.float()).abs().max()) <= step * 0.5 + step * 0.5 + 2e-3


def test_residual_codec_uniform_bit_exact(Q):
    from latentq_llm_amd import ops
    x = (torch.rand(1024 * 8, generator=torch.Generator().manual_seed(9)) - 0.5).to(torch.bfloat16)
    want_q, want_c = co.residual_quant(bits(x), 1)
    xg, q = x.cuda(), torch.empty(1024, dtype=torch.int32, device="cuda")
    ops.residual_quant(xg, q, 1)
    assert np.array_equal(q.cpu().numpy().view(np.uint32), want_q) and np.array_equal(bits(xg), want_c)
    assert np.array_equal(bits(ops.residual_dequant(q, 1)).reshape(-1), co.residual_dequant(want_q, 1))


def test_residual_tensor_round_trip(Q):
    """set_value -> add reconstructs latent = deq(W) + r * scale (utils/quant.py:803-837)."""
    N, K = 32, 256
    rt = Q.ResidualTensor(qshape=[N * K // 128, 128], oshape=[N, K])
    r = ((torch.rand(N, K, generator=torch.Generator().manual_seed(2)) - 0.5) * 0.9).to(torch.bfloat16).cuda()
    scale = torch.full((N * K // 128, 1), 0.01, dtype=torch.bfloat16, device="cuda")
    base = torch.zeros(N, K, dtype=torch.bfloat16, device="cuda")
    assert rt.add(base) is base  # nothing stored yet
    carry = rt.set_value(r.clone(), scale)
    assert carry.shape == (N, K) and set(carry.unique().tolist()) <= {0.0, 1.0}
    rec = rt.add(base).float() / 0.01 + carry.float()
    assert float((rec - r.float()).abs().max()) < 0.07


# ----------------------------------------------------------------------- optimizer ----------
def test_myadam_stochastic_requant_mode(Q):
    """lbit=0: one optimizer step == Adam direction fed to the requant kernel (checked against the
    C oracle with the same Philox stream)."""
    N, K = 512, 256  # >= 65536 elements -> 8-bit moments
    m, (packed, scales, zeros) = _make_w4_layer(Q, N, K, 11, False, lbit=0, train=True)
    assert m.weight.residual is None
    opt = Q.MyAdam([{"params": [m.weight], "weight_decay": 0.0}], lr=5e-3, betas=(0.9, 0.95), obit=8, sr_seed=77)
    x = randn_bf16((64, K), 12).cuda().requires_grad_(True)  # a QLinear only back-propagates through its input
    m(x).float().pow(2).mean().backward()
    grad = m.weight.grad.clone()
    opt.step()
    assert m.weight.grad is None and opt.state[m.weight]["state1"].dtype == torch.uint8
    # first Adam step: exp_avg = (1-b1) g, denom = sqrt((1-b2) g^2) + eps, step_size = lr*sqrt(bc2)/bc1
    g = grad.float()
    exp_avg = (g.to(torch.bfloat16) * 0).mul_(0.9).add_(grad, alpha=1 - 0.9)
    exp_sq = (grad * 0).mul_(0.95).addcmul_(grad, grad, value=1 - 0.95)
    denom = exp_sq.sqrt_().add_(1e-8)
    direction = (exp_avg / denom).to(torch.bfloat16)
    step_size = 5e-3 * (1 - 0.95) ** 0.5 / (1 - 0.9)
    want = co.requant(packed.numpy(), bits(scales), bits(zeros), bits(direction), step_size, N, K, seed=77, offset=0)
    got = m.weight.data.cpu().numpy().view(np.uint8)
    assert np.array_equal(got, want)
    assert (got != packed.numpy().view(np.uint8)).mean() > 0.05  # the step moved codes
    assert opt.sr_offset == N * K // 8  # one Philox block per 8 elements


@pytest.mark.parametrize("lbit", [4, 16])
def test_myadam_latent_modes_run_and_descend(Q, lbit):
    """lbit=4 (4-bit residual codec) and lbit=16 (bf16 latent copy): a few steps on a least-squares
    objective reduce the loss and keep codes in range."""
    N, K = 512, 256
    m, (packed, scales, zeros) = _make_w4_layer(Q, N, K, 13, False, lbit=lbit, train=True)
    if lbit == 16:
        m.weight.residual = Q.DeQfunc_4bit_g(m.weight.data, m.weight.qparam, torch.bfloat16).clone()
    opt = Q.MyAdam([{"params": [m.weight], "weight_decay": 0.0}], lr=2e-4, betas=(0.9, 0.95), obit=8)
    x = randn_bf16((256, K), 14).cuda().requires_grad_(True)
    target = randn_bf16((256, N), 15, 0.1).cuda()
    losses = []
    for _ in range(6):
        loss = (m(x).float() - target.float()).pow(2).mean()
        loss.backward()
        opt.step()
        losses.append(float(loss))
    assert losses[-1] < losses[0]
    codes = Q.python_decompress(m.weight.data)
    assert int(codes.min()) >= 0 and int(codes.max()) <= 15
