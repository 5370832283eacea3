"""Torch-CPU restatement of the reference's Python quantized-linear path — TEST INFRASTRUCTURE ONLY.

Each function follows the tensor-op sequence of the cited reference lines (paths relative to the
reference checkout), so that its results carry the same bf16 rounding points as the reference's
CPU/eager path. It is the "reference CPU dequant path" timed by bench.py's cpu_baseline leg.
Nothing in latentq_llm_amd imports this file.
"""
from __future__ import annotations

import torch

GROUP = 128  # utils/quant.py:44


@torch.no_grad()
def compress(codes: torch.Tensor) -> torch.Tensor:
    """utils/quant.py:4-9 — pairs (even, odd) -> one int8 byte, even index in the high nibble."""
    pairs = codes.reshape(-1, 2).to(torch.int8)
    return ((pairs[:, 0] << 4) + pairs[:, 1]).contiguous()


@torch.no_grad()
def decompress(packed: torch.Tensor) -> torch.Tensor:
    """utils/quant.py:12-19 — int8 bytes -> [n, 2] int8 codes (hi, lo), values 0..15."""
    packed = packed.reshape(-1)
    out = torch.empty((packed.shape[0], 2), dtype=torch.int8)
    out[:, 0] = (packed >> 4) % 16
    out[:, 1] = packed % 16
    return out


@torch.no_grad()
def dequant_4bit_g(packed, scales, zeros, shape, dtype=torch.bfloat16) -> torch.Tensor:
    """utils/quant.py:66-72 — (codes - zeros) * scales on [-1, 128] rows; bf16 arithmetic when
    scales/zeros are bf16 (int8 - bf16 promotes to bf16)."""
    q = decompress(packed).view(-1, GROUP)
    w = (q - zeros.reshape(-1, 1)) * scales.reshape(-1, 1)
    return w.view(shape).to(dtype)


@torch.no_grad()
def quant_4bit_g_rtn(latent, scales, zeros, shape) -> torch.Tensor:
    """utils/quant.py:45-63 without a ResidualTensor: Z = t/s + z, round half-even, clamp, pack."""
    t = latent.reshape(-1, GROUP)
    zq = torch.round(t / scales.reshape(-1, 1) + zeros.reshape(-1, 1))
    return compress(torch.clamp(zq, 0, 15).to(torch.uint8))


@torch.no_grad()
def w4_forward(x, packed, scales, zeros, shape, bias=None):
    """utils/quant.py:116-121."""
    w = dequant_4bit_g(packed, scales, zeros, shape, x.dtype)
    y = x.mm(w.t())
    if bias is not None:
        y += bias
    return y


@torch.no_grad()
def w4_backward(dy, x, packed, scales, zeros, shape, has_bias=False):
    """utils/quant.py:133-146 — returns (dX, dW, dB)."""
    w = dequant_4bit_g(packed, scales, zeros, shape, x.dtype)
    dx = dy.mm(w)
    dw = dy.t().mm(x)
    db = dy.sum(0) if has_bias else None
    return dx, dw, db


@torch.no_grad()
def llama_mlp_forward(x, gate, up, down):
    """HF LlamaMLP with its three nn.Linear replaced by A16W4 linears (main0.py:300-343):
    down(silu(gate(x)) * up(x)); each argument is (packed, scales, zeros, shape)."""
    g = w4_forward(x, *gate)
    u = w4_forward(x, *up)
    h = torch.nn.functional.silu(g) * u
    return w4_forward(h, *down), (g, u, h)


@torch.no_grad()
def act_quant_i8(x, clampv):
    """utils/quant.py:264-266."""
    x8 = x * 127. / clampv
    x8.round_().clamp_(-128, 127)
    return x8.to(torch.int8)


@torch.no_grad()
def int8_matmul_i32(x8, w8):
    """Exact integer X8 . W8^T (what the cutlass kernel accumulates)."""
    return torch.matmul(x8.to(torch.int32), w8.to(torch.int32).t())


@torch.no_grad()
def a8w8_forward_dynamic(x, w8, qscales, bias=None):
    """utils/quant.py:258-272. The external kernel's output rounding is not visible in the
    reference; modelled here as bf16(alpha * acc + bias') followed by the bf16 `* qscales`."""
    clampv = x.max()
    x8 = act_quant_i8(x, clampv)
    acc = int8_matmul_i32(x8, w8).to(torch.float32)
    alpha = (clampv / 127.).to(torch.float32)
    qs = qscales.reshape(-1)
    b = (bias / qs).to(torch.float32) if bias is not None else torch.zeros_like(qs, dtype=torch.float32)
    inner = (alpha * acc + b).to(torch.bfloat16)
    return inner * qs.view(1, -1), x8, clampv


@torch.no_grad()
def a8w8_backward(dy, x8, clampv, w8, qscales):
    """Intended semantics of utils/quant.py:276-293 (as in :196-206): Wf = W8.to(bf16) * qscales."""
    xf = x8.to(dy.dtype) * (clampv / 127.)
    wf = w8.to(dy.dtype) * qscales
    return dy.mm(wf), dy.t().mm(xf)
