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


@torch.no_grad()
def latent_w4_reconstruct(packed, scales, zeros, residual_int, shape, curve):
    """Latent weight in lbit=4 mode, the reference's chain on CPU tensors: DeQfunc_4bit_g
    (utils/quant.py:66-72) + ResidualTensor.add (utils/quant.py:826-837) with the residual decoded
    by the C restatement of the codec. curve = (p1, y1, p2, y2) of three_fold_curve_4bit."""
    import numpy as np
    from . import c_oracle as co
    p1, y1, p2, y2 = curve
    w = dequant_4bit_g(packed, scales, zeros, shape)                      # bf16
    r_bits = co.residual_dequant(residual_int.numpy().view(np.uint32), 0, p1, y1, p2 - p1, y2, 8 - p2)
    r = torch.from_numpy(r_bits.view(np.int16).copy()).view(torch.bfloat16)
    r = (r.view(-1, 128) * scales.reshape(-1, 1)).to(torch.bfloat16)       # bf16 * bf16 -> bf16
    return r.view(shape).add(w.view(shape))


@torch.no_grad()
def latent_w4_requant(latent, scales, zeros, shape, curve):
    """Qfunc_4bit_g_res with a ResidualTensor handle (utils/quant.py:45-63, 803-811) on CPU tensors.
    Returns (packed codes int8, residual words int32)."""
    import numpy as np
    from . import c_oracle as co
    p1, y1, p2, y2 = curve
    t = latent.view(-1, 128)
    Z = t / scales.reshape(-1, 1) + zeros.reshape(-1, 1)
    q = torch.round(Z)
    f = (Z - q).to(torch.bfloat16).contiguous()
    words, carry_bits = co.residual_quant(f.view(torch.int16).numpy().view(np.uint16), 0, p1, y1, p2 - p1, y2, 8 - p2)
    carry = torch.from_numpy(carry_bits.view(np.int16).copy()).view(torch.bfloat16).view(shape)
    q = q.view(shape) + carry
    codes = compress(torch.clamp(q, 0, 15).to(torch.uint8))
    return codes, torch.from_numpy(words.view(np.int32).copy())


@torch.no_grad()
def quant_8bit_opt(tensor, nblocks):
    """utils/quant.py:22-33 — block-wise asymmetric uint8 quantiser of an optimizer moment
    (the reference's ``blocksize`` argument is the NUMBER of blocks)."""
    shape = tensor.shape
    blocks = tensor.reshape(nblocks, -1)
    lo, hi = torch.aminmax(blocks, dim=1, keepdim=True)
    scale = (hi - lo) / 255 + 1e-10
    q = torch.clamp(torch.round((hi - blocks) / scale), 0, 255)
    return q.to(torch.uint8).reshape(shape), scale, hi


@torch.no_grad()
def dequant_8bit_opt(q, scale, hi):
    """utils/quant.py:35-41."""
    return (hi - q.reshape(scale.shape[0], -1).to(torch.float32) * scale).reshape(q.shape)


@torch.no_grad()
def adam8_step(grad, state1, scale1, max1, state2, scale2, max2, beta1, beta2, eps, step_size, param=None):
    """utils/quant.py:1081-1134 for uint8 moments and no weight decay: returns the updated parameter
    (or, with param=None, the update direction bf16(m / d) that the stochastic-rounding requantizer
    takes) and the re-quantised moments (state1, scale1, max1, state2, scale2, max2)."""
    nblk = scale1.shape[0]
    exp_avg = dequant_8bit_opt(state1, scale1, max1).to(grad.dtype)
    s2 = dequant_8bit_opt(state2, scale2, max2)
    exp_avg_sq = (s2 * s2).to(grad.dtype)
    exp_avg.mul_(beta1).add_(grad, alpha=1 - beta1)
    exp_avg_sq.mul_(beta2).addcmul_(grad, grad, value=1 - beta2)
    exp_avg_sqrt = exp_avg_sq.sqrt_()
    denom = exp_avg_sqrt.add_(eps)
    if param is not None:
        out = param.clone().addcdiv_(exp_avg, denom, value=-step_size)
    else:
        out = (exp_avg / denom).to(torch.bfloat16)
    q1, sc1, mx1 = quant_8bit_opt(exp_avg.float(), nblk)
    q2, sc2, mx2 = quant_8bit_opt(exp_avg_sqrt.float(), nblk)
    return out, (q1, sc1, mx1, q2, sc2, mx2)


# ------------------------------------------------------------------ A8W8 latent re-quantiser ---
def quant_8bit_res(latent, qscales, carry=None):
    """Qfunc_8bit_res, utils/quant.py:88-103, without the residual handle: q = round(latent / qscales)
    (torch.round: half to even), plus the carry the residual codec returned (lbit = 4), clamped to
    [-128, 127] as int8. Also returns the residual latent / qscales - q that the handle receives."""
    q = latent / qscales
    q = q.round()
    res = latent / qscales - q
    if carry is not None:
        q = q + carry
    return q.clamp(-128, 127).to(torch.int8), res


@torch.no_grad()
def latent_w8_reconstruct(codes, qscales, residual_int, curve):
    """Latent weight of an 8-bit-weight layer in lbit = 4 mode, the reference's chain on CPU tensors:
    (p.data * p.qparam).to(bf16) (utils/quant.py:1069-1070) + ResidualTensor.add (:826-837) with the residual decoded by
    the C restatement of the codec. codes int8 [N,K], qscales bf16 [N,1]."""
    import numpy as np
    from . import c_oracle as co
    p1, y1, p2, y2 = curve
    w = (codes * qscales).to(torch.bfloat16)
    r_bits = co.residual_dequant(residual_int.numpy().view(np.uint32), 0, p1, y1, p2 - p1, y2, 8 - p2)
    r = torch.from_numpy(r_bits.view(np.int16).copy()).view(torch.bfloat16)
    r = (r.view(codes.shape) * qscales).to(torch.bfloat16)
    return r.add(w)


@torch.no_grad()
def latent_w8_requant(latent, qscales, curve):
    """Qfunc_8bit_res with a ResidualTensor handle (utils/quant.py:88-103, 803-811) on CPU tensors: returns
    (codes int8 [N,K], residual words int32)."""
    import numpy as np
    from . import c_oracle as co
    p1, y1, p2, y2 = curve
    q = latent / qscales
    q.round_()
    f = (latent / qscales - q).to(torch.bfloat16).contiguous()
    words, carry_bits = co.residual_quant(f.view(torch.int16).numpy().view(np.uint16), 0, p1, y1, p2 - p1, y2, 8 - p2)
    carry = torch.from_numpy(carry_bits.view(np.int16).copy()).view(torch.bfloat16).view(latent.shape)
    q += carry
    return q.clamp_(-128, 127).to(torch.int8), torch.from_numpy(words.view(np.int32).copy())


# --------------------------------------------------------------- 8-bit gradient accumulator ---
def gradq8_find_param(data):
    """GradientQTensor.find_param, utils/quant.py:856-861 (bit = 8)."""
    vmax = data.abs().amax(dim=1, keepdim=True) * 4
    return (torch.clamp(vmax, min=1e-5) / 127).to(data.dtype)


def gradq8_quant(fdata, scale, noise):
    """GradientQTensor.quant, utils/quant.py:864-868, with the uniform_(-0.5, 0.5) noise injected."""
    return torch.clamp(torch.round(fdata / scale + noise), -128, 127).to(torch.int8)


def gradq8_set(fdata, noise):
    """set_value, utils/quant.py:877-885: (qdata, scale)."""
    scale = gradq8_find_param(fdata)
    return gradq8_quant(fdata, scale, noise), scale


def gradq8_add(qdata, scale, fdata, noise):
    """add_, utils/quant.py:891-898: quant(dequant() + fdata) with the scale of the first micro-batch."""
    odata = qdata.to(fdata.dtype) * scale
    return gradq8_quant(odata + fdata, scale, noise)
