"""GPU parity at the full benchmark sizes, through the C ABI.

The C oracle would need minutes for these shapes, so the checks here use what stays cheap and
exact at full size: float64 torch.mm on the host over the oracle's (bit-exact, separately
tested) dequantised weights for the bf16 outputs, float64 matmul of int8 operands (exact below
2^53) for the int32 accumulators, and the adjoint identity for forward against dX.
"""
import numpy as np
import pytest
import torch

from tests.util import bits, from_bits, make_w4, randn_bf16, rel_l2

pytestmark = pytest.mark.gpu

REL_L2_TOL = 1e-2
HID, FFN, TOKENS = 4096, 11008, 2048


@pytest.fixture(scope="module")
def ops(hip_lib):
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from latentq_llm_amd import ops as _ops
    return _ops


@pytest.fixture(scope="module")
def co():
    from oracle import c_oracle
    return c_oracle


def _deq64(co, packed, scales, zeros, N, K):
    return from_bits(co.dequant(packed.numpy(), bits(scales), bits(zeros), N, K)).reshape(N, K).double()


def _report(name, got, want64):
    err = rel_l2(got.float().cpu(), want64)
    mx = float((got.double().cpu() - want64).abs().max())
    print(f"{name}: rel_l2={err:.3e} max_abs={mx:.3e}")
    assert err <= REL_L2_TOL
    return err


@pytest.mark.timeout(900)
def test_llama_mlp_block_2048_tokens(ops, co):
    """Forward down(silu(gate(x)) * up(x)) and dX through all three projections at 2048 tokens.
    Each GEMM is checked on its own inputs (the GPU's own intermediate activations, moved to the
    host), so that an error cannot hide behind the next layer; the block output is checked too."""
    torch.set_num_threads(16)
    gate = make_w4(FFN, HID, 101)[1:]
    up = make_w4(FFN, HID, 102)[1:]
    down = make_w4(HID, FFN, 103)[1:]
    x = randn_bf16((TOKENS, HID), 104)
    dy = randn_bf16((TOKENS, HID), 105)
    Wg, Wu, Wd = _deq64(co, *gate, FFN, HID), _deq64(co, *up, FFN, HID), _deq64(co, *down, HID, FFN)
    dgate, dup, ddown = [[t.cuda() for t in w] for w in (gate, up, down)]
    xg, dyg = x.cuda(), dy.cuda()

    g = ops.a16w4_forward(xg, *dgate, (FFN, HID))
    u = ops.a16w4_forward(xg, *dup, (FFN, HID))
    _report("fwd gate", g, x.double() @ Wg.t())
    _report("fwd up", u, x.double() @ Wu.t())
    act = torch.nn.functional.silu(g)
    h = act * u
    y = ops.a16w4_forward(h, *ddown, (HID, FFN))
    _report("fwd down", y, h.double().cpu() @ Wd.t())
    # whole block against the float64 composition with the same bf16 rounding points
    g64 = (x.double() @ Wg.t()).to(torch.bfloat16)
    u64 = (x.double() @ Wu.t()).to(torch.bfloat16)
    h64 = torch.nn.functional.silu(g64) * u64
    _report("block y", y, h64.double() @ Wd.t())

    dh = ops.a16w4_dx(dyg, *ddown, (HID, FFN))
    _report("dX down", dh, dy.double() @ Wd)
    du = dh * act
    dg = torch.ops.aten.silu_backward(dh * u, g)
    dxg = ops.a16w4_dx(dg, *dgate, (FFN, HID))
    dxu = ops.a16w4_dx(du, *dup, (FFN, HID))
    _report("dX gate", dxg, dg.double().cpu() @ Wg)
    _report("dX up", dxu, du.double().cpu() @ Wu)
    # adjoint identity <x Wg^T, r> = <x, r Wg> on the kernel outputs (r = dg): both sides in float64
    lhs = float((g.double() * dg.double()).sum())
    rhs = float((xg.double() * dxg.double()).sum())
    scale = float(g.double().norm() * dg.double().norm())  # Cauchy-Schwarz scale of either side
    print(f"adjoint: lhs={lhs:.6e} rhs={rhs:.6e} scale={scale:.3e}")
    assert abs(lhs - rhs) <= 1e-2 * scale


@pytest.mark.parametrize("N,K", [(2048, 2048), (8192, 2048), (2048, 8192)])
def test_a8w8_opt_1p3b_shapes(ops, N, K):
    M = 2048
    torch.set_num_threads(16)
    g = torch.Generator().manual_seed(N + K)
    x8 = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int8)
    w8 = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8)
    sx = (torch.randn(M, generator=g) * 0.05).abs() + 1e-4
    sw = (torch.randn(N, generator=g) * 0.01).abs() + 1e-5
    y, acc = ops.a8w8_forward(x8.cuda(), w8.cuda(), sx.cuda(), sw.cuda(), want_acc=True)
    want = (x8.double() @ w8.double().t())  # exact: |acc| < 2^31 << 2^53
    assert torch.equal(acc.cpu().double(), want), "int32 accumulators must be bit-exact"
    want_y = ((want.float() * sx[:, None]) * sw[None, :]).to(torch.bfloat16)
    assert torch.equal(y.cpu(), want_y)  # fp32 epilogue is deterministic: (acc*sx)*sw, one bf16 rounding


@pytest.mark.parametrize("M", [1, 4, 16])
@pytest.mark.parametrize("N,K", [(4096, 4096), (11008, 4096), (4096, 11008)])
def test_gemv_llama7b_shapes(ops, co, N, K, M):
    torch.set_num_threads(16)
    w = make_w4(N, K, N + K + M)[1:]
    x = randn_bf16((M, K), 7 + M)
    W = _deq64(co, *w, N, K)
    y = ops.a16w4_forward(x.cuda(), *[t.cuda() for t in w], (N, K))
    _report(f"gemv N={N} K={K} M={M}", y, x.double() @ W.t())
