"""GPU tests of the library's weight-gradient GEMM (lq_weight_grad: dW = dY^T X with both operands read
transposed out of LDS) and of its int8-accumulator epilogue (lq_weight_grad_acc8).

Bars: the bf16 product against the float64 matrix product (rel-L2 <= 1e-2, printed) plus an integer-exact case and
a one-hot case that pin the operand orientation; the accumulate epilogue bit for bit against the CPU oracle's
GradientQTensor.add_ (oracle/lq_oracle.c::lqo_gradq8) applied to the very bf16 product the store form returns, for
injected and Philox noise.
"""
import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from tests.util import bits, randn_bf16, rel_l2

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops(hip_lib):
    assert torch.cuda.is_available()
    from latentq_llm_amd import ops as _ops
    return _ops


SHAPES = [(64, 8, 8), (128, 256, 256), (192, 264, 520), (2048, 1024, 768), (256, 3072, 768), (64, 1000, 48), (320, 40, 4112)]


@pytest.mark.parametrize("M,N,K", SHAPES)
def test_weight_grad_matches_float64(ops, M, N, K):
    dy, x = randn_bf16((M, N), 1).cuda(), randn_bf16((M, K), 2).cuda()
    dw = ops.weight_grad(dy, x)
    assert dw.shape == (N, K) and dw.dtype == torch.bfloat16
    want = dy.double().t() @ x.double()
    err = rel_l2(dw, want)
    print(f"weight_grad {M}x{N}x{K}: rel_l2={err:.3e} max_abs={float((dw.double() - want).abs().max()):.3e}")
    assert err < 4e-3


def test_weight_grad_orientation_and_exact_integers(ops):
    """One-hot operands: dW[n, k] = sum_m dY[m, n] X[m, k] picks single products (a swapped or transposed operand
    lands elsewhere); small integers: every partial sum is exact in fp32 and the result fits bf16 exactly."""
    M, N, K = 128, 264, 520
    dy = torch.zeros((M, N), dtype=torch.bfloat16)
    x = torch.zeros((M, K), dtype=torch.bfloat16)
    picks = [(0, 0, 0, 1.0, 2.0), (5, 17, 300, 3.0, -0.5), (63, 263, 519, -2.0, 4.0), (64, 100, 7, 1.5, 1.5), (127, 31, 256, 8.0, 0.25)]
    for m, n, k, a, b in picks:
        dy[m, n], x[m, k] = a, b
    dw = ops.weight_grad(dy.cuda(), x.cuda()).cpu()
    want = torch.zeros((N, K))
    for m, n, k, a, b in picks:
        want[n, k] += a * b
    assert torch.equal(dw.float(), want)
    g = torch.Generator().manual_seed(3)
    dyi = torch.randint(-2, 3, (M, N), generator=g).to(torch.bfloat16)
    xi = torch.randint(-2, 3, (M, K), generator=g).to(torch.bfloat16)
    dwi = ops.weight_grad(dyi.cuda(), xi.cuda()).cpu()
    wanti = dyi.double().t() @ xi.double()          # |sum| <= 4 * 128 = 512: bf16 holds integers up to 256 exactly,
    assert float(wanti.abs().max()) <= 256          # and these stay below
    assert torch.equal(dwi.double(), wanti)


def test_weight_grad_falls_back_for_other_token_counts(ops):
    dy, x = randn_bf16((100, 64), 1).cuda(), randn_bf16((100, 128), 2).cuda()
    dw = ops.weight_grad(dy, x)
    assert rel_l2(dw, dy.double().t() @ x.double()) < 4e-3


def _noise(shape, seed):
    return (torch.rand(shape, generator=torch.Generator().manual_seed(seed)) - 0.5).to(torch.bfloat16)


@pytest.mark.parametrize("M,N,K", [(64, 8, 16), (128, 264, 528), (256, 1024, 768), (2048, 512, 1040)])
@pytest.mark.parametrize("mode", ["inject", "philox"])
def test_weight_grad_acc8_epilogue_bit_exact(ops, M, N, K, mode):
    """Two accumulating micro-batches after a set_value: the GEMM's epilogue = the stand-alone accumulate pass on the
    bf16 product the store form returns = the CPU oracle on that product, all bit for bit."""
    dy0, x0 = randn_bf16((M, N), 10, 0.05).cuda(), randn_bf16((M, K), 11).cuda()
    dw0 = ops.weight_grad(dy0, x0)
    q = torch.empty((N, K), dtype=torch.int8, device="cuda")
    s = torch.empty((N, 1), dtype=torch.bfloat16, device="cuda")
    ops.gradq8_quant(dw0, q, s, False, seed=9, offset=0)
    if N > 8:
        s[3] = 2.0 ** -50     # a scale outside the range of the reciprocal form: the whole wave divides
        s[5] = 3e38
    want_q, want_s = q.cpu().numpy().reshape(-1).copy(), bits(s).reshape(-1).copy()
    q2 = q.clone()
    for i in (1, 2):
        dy, x = randn_bf16((M, N), 20 + i, 0.05).cuda(), randn_bf16((M, K), 30 + i).cuda()
        dw = ops.weight_grad(dy, x)
        if mode == "inject":
            nz = _noise((N, K), 40 + i)
            kw_o, kw_h = {"noise": bits(nz)}, {"noise": nz.cuda()}
        else:
            kw_o = kw_h = {"seed": 9, "offset": 777 * i}
        want_q, _ = co.gradq8(bits(dw), want_q, want_s, True, N, K, **kw_o)
        ops.weight_grad_acc8(dy, x, q, s, **kw_h)
        ops.gradq8_quant(dw, q2, s, True, **kw_h)
        assert torch.equal(q, q2), f"epilogue and stand-alone pass differ at micro-batch {i}"
        mism = int((q.cpu().numpy().reshape(-1) != want_q).sum())
        assert mism == 0, f"{mism} of {N * K} int8 values differ from the oracle at micro-batch {i}"
    assert np.array_equal(bits(s).reshape(-1), want_s)  # the scales are read, never written


@pytest.mark.parametrize("M,N,K", SHAPES)
def test_weight_grad_accumulating_form_equals_a_bf16_add(ops, M, N, K):
    """lq_weight_grad_acc: g = bf16(g + bf16(dY^T X)), bit for bit what `g.add_(dW)` makes of the stored product (the
    addition done by the tensor library on the CPU), partial tiles included."""
    dy, x = randn_bf16((M, N), 11).cuda(), randn_bf16((M, K), 12).cuda()
    g0 = randn_bf16((N, K), 13, 20.0)
    dw = ops.weight_grad(dy, x)
    want = g0.clone().add_(dw.cpu())
    g = g0.cuda()
    assert ops.weight_grad_acc(dy, x, g) is g
    assert torch.equal(g.cpu().view(torch.int16), want.view(torch.int16))
    with pytest.raises(ValueError):
        ops.weight_grad_acc(dy, x, g[:, :-8] if K > 8 else g.float())


def test_bf16_gradient_accumulation_through_the_gemm_epilogue(hip_lib):
    """gbit = 16 (the reference's default): from the second micro-batch on the backward hook adds dW onto
    module.weight.grad inside the GEMM; the accumulated gradient equals the sum of the separately formed products,
    added in bf16 one after the other, bit for bit, and no product tensor is materialised."""
    from latentq_llm_amd import ops as O
    from latentq_llm_amd import quant as Q
    from tests.util import make_w4
    N, K, M = 128, 256, 192
    codes, packed, scales, zeros = make_w4(N, K, 31)
    m = Q.QLinearA16W4(K, N, bias=False, lbit=0, gbit=16)
    m.zeros.data, m.scales.data, m.wshape = zeros.clone(), scales.clone(), [N, K]
    m.weight.set_value(packed, [m.scales, m.zeros, m.wshape])
    m = m.bfloat16().cuda()
    m.to("cuda")
    m.weight.requires_grad = True
    m.add_hook()
    x = randn_bf16((M, K), 32).cuda().requires_grad_(True)
    dys = [randn_bf16((M, N), 33 + i).cuda() for i in range(3)]
    calls = {"store": 0, "acc": 0}
    real_store, real_acc = O.weight_grad, O.weight_grad_acc
    try:
        O.weight_grad = lambda *a, **k: (calls.__setitem__("store", calls["store"] + 1), real_store(*a, **k))[1]
        O.weight_grad_acc = lambda *a, **k: (calls.__setitem__("acc", calls["acc"] + 1), real_acc(*a, **k))[1]
        for dy in dys:
            m(x).backward(dy)
        assert calls == {"store": 1, "acc": 2} and len(Q.dict_temp) == 0
    finally:
        O.weight_grad, O.weight_grad_acc = real_store, real_acc
    want = O.weight_grad(dys[0], x.detach())
    for dy in dys[1:]:
        want.add_(O.weight_grad(dy, x.detach()))
    assert torch.equal(m.weight.grad, want)
