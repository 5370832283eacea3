"""Drop-in for the reference's ``utils/quant.py`` with the hot ops on the gfx950 HIP kernels.

Same public names, constructor arguments, buffer names and calling conventions as the reference
module (``utils/quant.py``; used by ``main0.py:36, 208, 300-343, 454-504`` and ``Demo2.py:25,
37-104``), so ``from utils.quant import ...`` can be pointed here unchanged. What differs is
underneath: dequantise+matmul, the int8 GEMM with its scale epilogue, the 4-bit residual codec
and the stochastic latent requantizer are single HIP kernels reached through the C ABI
(``latentq_llm_amd.ops``); there is no Triton, no torch_int/cutlass and no JIT-compiled CUDA
extension. GPU tensors are mandatory for those ops (no CPU fallback).

Deliberate deviations from the reference, all on purpose:
  * ``QLinearFunctionA8W8_dynamic.backward`` multiplies an int8 tensor in place by a bf16 scale
    (utils/quant.py:281-283), which stock PyTorch rejects; the semantics of its siblings
    (utils/quant.py:200-201) are used: ``W8.to(bf16) * qscales``.
  * the dynamic A8W8 forward keeps ``clampv = input.max()`` on the device instead of ``.item()``
    (utils/quant.py:220, 320): same value, no host sync.
  * ``lbit=0`` on a 4-bit weight (the constructor default, which in the reference leaves an
    uninitialised fp32 latent copy that main0.py never fills) selects the stochastic-rounding latent
    requantizer: no stored residual, the optimizer calls ``ops.requant_sr`` once per parameter
    (kernel 1). An 8-bit weight with ``lbit=0`` keeps the reference's fp32 latent copy.
  * ``MyAdam.step`` does not synchronise the device and empty the cache after every parameter
    (utils/quant.py:985, 1137).
"""
from __future__ import annotations

import math
from functools import reduce
from typing import Optional, Union

import torch
import torch.nn as nn

from . import ops

GROUPSIZE = 128  # utils/quant.py:44
# lbit = 4 latent passes (codes + residual -> latent, latent -> codes + residual) as single HIP
# kernels; False runs the reference's chain of tensor operations around the codec kernel instead
# (same bits either way).
FUSED_LATENT = True
# The Adam step on uint8 moments (dequantise both moments, update them, apply the update, re-quantise
# them per block) as one HIP kernel; False runs the chain of tensor operations (same bits either way).
FUSED_ADAM8 = True
# The 8-bit gradient accumulator (row scales + stochastic rounding to int8, and the accumulate form) as
# one HIP pass per micro-batch; False runs the reference's tensor operations with torch's uniform_ noise.
FUSED_GRADQ = True
# The input gradient of an 8-bit-weight layer from its int8 codes (the dequantised weight formed inside the GEMM);
# False materialises W8 * qscales and multiplies densely, as the reference does.
FUSED_A8W8_DX = True
EXT_type = torch.bfloat16  # utils/quant.py:722

# dW travels from the autograd Functions to the full-backward hook through this list
# (utils/quant.py:109-110, 398-411).
dict_temp = []


# --------------------------------------------------------------------------- nibble packing --
@torch.no_grad()
def python_compress(fdata, bit=4):
    """Two 4-bit codes per int8 byte, even index in the high nibble (utils/quant.py:4-9)."""
    assert bit == 4
    pairs = fdata.reshape(-1, 2).to(torch.uint8)
    return ((pairs[:, 0] << 4) | (pairs[:, 1] & 0xF)).view(torch.int8).contiguous()


@torch.no_grad()
def python_decompress(int_data, bit=4):
    """int8 bytes -> [n, 2] int8 codes in 0..15 (utils/quant.py:12-19)."""
    assert bit == 4
    b = int_data.reshape(-1).view(torch.uint8)
    return torch.stack(((b >> 4), (b & 0xF)), dim=1).to(torch.int8)


# ------------------------------------------------------------------ 8-bit optimizer states --
@torch.no_grad()
def Qfunc_8bit_opt(tensor, blocksize=1, qparam=None):
    """Block-wise asymmetric uint8 quantizer of an optimizer moment (utils/quant.py:22-33):
    ``blocksize`` is the NUMBER of blocks; q = clamp(round((max - x)/scale), 0, 255)."""
    shape = tensor.shape
    blocks = tensor.view(blocksize, -1)
    if qparam is None:
        lo, hi = torch.aminmax(blocks, dim=1, keepdim=True)
        scale = (hi - lo) / 255 + 1e-10
    else:
        scale, hi = qparam
    q = torch.clamp_(torch.round_((hi - blocks).div_(scale)), 0, 255)
    return q.to(torch.uint8).view(shape), [scale, hi]


@torch.no_grad()
def DeQfunc_8bit_opt(qtensor, qparam, dtype=torch.float32):
    """Inverse of Qfunc_8bit_opt (utils/quant.py:35-41)."""
    scale, hi = qparam
    shape = qtensor.shape
    x = hi - qtensor.view(scale.shape[0], -1).to(dtype) * scale
    return x.view(shape).to(dtype)


# ----------------------------------------------------------------- W4 group (de)quantizers --
def _flat_qparam(qparam):
    scales, zeros, shape = qparam
    return scales.contiguous().reshape(-1), zeros.contiguous().reshape(-1), list(shape)


@torch.no_grad()
def DeQfunc_4bit_g(qtensor, qparam, dtype=torch.float32):
    """bf16((codes - zeros) * scales) per 128-element group (utils/quant.py:66-72), one HIP pass."""
    scales, zeros, shape = _flat_qparam(qparam)
    w = ops.a16w4_dequant(qtensor.contiguous(), scales.to(torch.bfloat16), zeros.to(torch.bfloat16), shape)
    return w if dtype == torch.bfloat16 else w.to(dtype)


@torch.no_grad()
def Qfunc_4bit_g_res(tensor, residual_handle, qparam, groupsize=GROUPSIZE):
    """Round-to-nearest group quantizer with residual memory (utils/quant.py:45-63):
    Z = t/s + z; q = round(Z); the fractional part goes to the 4-bit residual codec, whose carry
    is added back; clamp to [0, 15] and pack."""
    scales, zeros, shape = qparam
    scales = scales.contiguous().reshape(-1, 1)
    zeros = zeros.contiguous().reshape(-1, 1)
    if (FUSED_LATENT and isinstance(residual_handle, ResidualTensor) and groupsize == GROUPSIZE and tensor.is_cuda
            and tensor.dtype == torch.bfloat16 and scales.dtype == torch.bfloat16 and zeros.dtype == torch.bfloat16
            and residual_handle.residual_int.is_cuda):
        # one HIP pass with the rounding points of the chain below (lq_latent_w4_requant)
        p1, y1, p2, y2 = three_fold_curve_4bit(residual_handle.mu)
        codes = ops.latent_w4_requant(tensor.data.contiguous(), scales, zeros, residual_handle.residual_int.view(-1),
                                      tuple(shape), p1, y1, p2 - p1, y2, 8 - p2)
        residual_handle.weight_scale = scales
        residual_handle.lock_mu = residual_handle.mu
        residual_handle.init = False
        return codes
    t = tensor.data.view(-1, groupsize)
    Z = t / scales + zeros
    q = torch.round(Z)
    if isinstance(residual_handle, ResidualTensor):
        carry = residual_handle.set_value((Z - q).view(shape), scales)
        q = q.view(shape) + carry
    else:
        residual_handle.data = t.view(shape).to(residual_handle.dtype)
    return python_compress(torch.clamp(q, 0, 15).to(torch.uint8))


@torch.no_grad()
def Qfunc_8bit_res(tensor, residual_handle, qscales):
    """Per-channel int8 re-quantizer with residual memory (utils/quant.py:88-103)."""
    shape = tensor.shape
    if (FUSED_LATENT and not isinstance(residual_handle, ResidualTensor) and tensor.is_cuda and tensor.dim() == 2
            and tensor.dtype == torch.bfloat16 and tensor.is_contiguous() and tensor.shape[1] % 8 == 0
            and tensor.data_ptr() % 16 == 0 and torch.is_tensor(qscales) and qscales.dtype == torch.bfloat16
            and qscales.is_contiguous() and qscales.dim() == 2 and tuple(qscales.shape) == (tensor.shape[0], 1)):
        # the chain below as one pass (same roundings)
        if residual_handle is not None:
            residual_handle.data = tensor.to(residual_handle.dtype)
        return ops.w8_requant(tensor, qscales)
    if (FUSED_LATENT and isinstance(residual_handle, ResidualTensor) and tensor.is_cuda and tensor.dim() == 2
            and tensor.dtype == torch.bfloat16 and tensor.is_contiguous() and tensor.shape[1] % 16 == 0
            and tensor.data_ptr() % 16 == 0 and torch.is_tensor(qscales) and qscales.dtype == torch.bfloat16
            and qscales.is_contiguous() and qscales.dim() == 2 and tuple(qscales.shape) == (tensor.shape[0], 1)
            and residual_handle.residual_int.is_cuda):
        # the chain below with the residual codec inside, as one pass (lq_latent_w8_requant; same roundings)
        p1, y1, p2, y2 = three_fold_curve_4bit(residual_handle.mu)
        codes = ops.latent_w8_requant(tensor, qscales.view(-1), residual_handle.residual_int.view(-1), p1, y1, p2 - p1, y2, 8 - p2)
        residual_handle.weight_scale = qscales
        residual_handle.lock_mu = residual_handle.mu
        residual_handle.init = False
        return codes
    q = tensor / qscales
    q.round_()
    if isinstance(residual_handle, ResidualTensor):
        carry = residual_handle.set_value((tensor / qscales - q).view(shape), qscales)
        q += carry
    elif residual_handle is not None:
        residual_handle.data = tensor.to(residual_handle.dtype)
    return q.clamp_(-128, 127).to(torch.int8)


# ---------------------------------------------------------------------- pending weight gradient --
class _PendingWeightGrad(object):
    """dW = dY^T X of one backward, not formed yet: the autograd Functions hand this to the backward hook through
    dict_temp, and the hook either forms the product straight into an int8 gradient accumulator
    (``GradientQTensor.add_product_``: the GEMM's epilogue does the accumulation and dW is never stored) or
    materialises the bf16 tensor (``tensor()``), which is what every other consumer gets."""
    __slots__ = ("dy", "x")

    def __init__(self, dy, x):
        self.dy, self.x = dy, x

    def tensor(self):
        return ops.weight_grad(self.dy, self.x)


def _pending_dw(grad_output, input):
    """What a Function's backward appends to dict_temp: the pending product where the library's own GEMM can form it
    (contiguous bf16 GPU operands, a multiple of 64 tokens), the product itself otherwise."""
    if FUSED_GRADQ and ops._weight_grad_native_ok(grad_output, input):
        return _PendingWeightGrad(grad_output, input)
    return ops.weight_grad(grad_output, input)


# ------------------------------------------------------------------------ autograd: A16W4 --
# The reference gates the bias gradient on needs_input_grad[2] (utils/quant.py:143, 208, 249, 290,
# 371), which is the flag of the non-tensor qparam argument and therefore always False: QLinear
# biases never receive a gradient there. Kept as is so that training runs match the reference.
_BIAS_FLAG = 2

def _as_bf16_2d(x):
    return x.contiguous() if x.dtype == torch.bfloat16 else x.to(torch.bfloat16).contiguous()


def _w4_linear(input, weight_d, qparamw4, bias):
    scales, zeros, shape = _flat_qparam(qparamw4)
    b = None if bias is None else bias.detach().to(torch.bfloat16).contiguous()
    y = ops.a16w4_forward(_as_bf16_2d(input), weight_d, scales, zeros, shape, b)
    return y if input.dtype == torch.bfloat16 else y.to(input.dtype)


class QLinearFunctionW4(torch.autograd.Function):
    """Training A16W4 linear (utils/quant.py:112-146): Y = X deq(W)^T + b; backward re-reads the
    packed codes (never a materialised W): dX on the HIP dequant-GEMM, dW = dY^T X pushed to
    dict_temp for the backward hook, dB = sum dY."""

    @staticmethod
    def forward(input, weight_d, qparamw4, bias):
        return _w4_linear(input, weight_d, qparamw4, bias)

    @staticmethod
    def setup_context(ctx, inputs, output):
        input, weight_d, qparamw4, bias = inputs
        ctx.save_for_backward(input, weight_d.data, bias)
        ctx.save_qparamw4 = qparamw4

    @staticmethod
    def backward(ctx, grad_output):
        input, weight_d, bias = ctx.saved_tensors
        scales, zeros, shape = _flat_qparam(ctx.save_qparamw4)
        grad_input = grad_bias = None
        dy = _as_bf16_2d(grad_output)
        if ctx.needs_input_grad[0]:
            grad_input = ops.a16w4_dx(dy, weight_d, scales, zeros, shape)
            if grad_input.dtype != input.dtype:
                grad_input = grad_input.to(input.dtype)
        dict_temp.append(_pending_dw(dy, _as_bf16_2d(input)))  # dW = dY^T X (utils/quant.py:141-142)
        if bias is not None and ctx.needs_input_grad[_BIAS_FLAG]:
            grad_bias = grad_output.sum(0)
        return grad_input, None, None, grad_bias


class QLinearFunctionW4_eval(torch.autograd.Function):
    """Inference A16W4 linear (utils/quant.py:149-169): no state saved, no gradients."""

    @staticmethod
    def forward(input, weight_d, qparamw4, bias):
        return _w4_linear(input, weight_d, qparamw4, bias)

    @staticmethod
    def setup_context(ctx, inputs, output):
        pass

    @staticmethod
    def backward(ctx, grad_output):
        return None, None, None, None


# ------------------------------------------------------------------------- autograd: A8W8 --
def _clamp_tensor(clampv, device):
    if torch.is_tensor(clampv):
        return clampv.detach().to(device=device, dtype=torch.float32).reshape(1)
    return torch.tensor([float(clampv)], dtype=torch.float32, device=device)


def _qs_bias(qscales, bias):
    """The per-channel scales and the bias as the int8 GEMM reads them (bf16 [N]); no kernel runs when the module's
    buffers already have that form."""
    sw = qscales.detach().reshape(-1)
    if sw.dtype not in (torch.bfloat16, torch.float32):
        sw = sw.float()
    b = None if bias is None else bias.detach().to(torch.bfloat16).contiguous()
    return sw.contiguous(), b


def _a8w8_linear(input, weight_i8, qscales, bias, clampv, alpha_in_bf16):
    """Static clamp value: x8 = clamp(round(x*127/clampv)); Y = ((x8 . W8^T) * alpha) * qscales + bias with
    alpha = clampv/127: the cutlass call `linear_a8_w8_bbf16_obf16(x8, W8, bias/qs, alpha) * qs`
    of utils/quant.py:178-183 as one int8-MFMA kernel with a fused epilogue. Returns (Y, x8)."""
    x = _as_bf16_2d(input)
    cv = _clamp_tensor(clampv, x.device)
    x8 = ops.act_quant_i8(x, cv)
    if alpha_in_bf16:  # the training Function divides a 0-dim bf16 tensor: alpha is bf16-rounded
        alpha = (cv.to(torch.bfloat16) / 127.).float()
    else:
        alpha = cv / 127.
    sx = alpha.expand(x.shape[0]).contiguous()
    sw, b = _qs_bias(qscales, bias)
    y = ops.a8w8_forward(x8, weight_i8.contiguous(), sx, sw, b)
    return (y if input.dtype == torch.bfloat16 else y.to(input.dtype)), x8


def _a8w8_linear_dynamic(input, weight_i8, qscales, bias, alpha_in_bf16, per_token=False):
    """The dynamic layers' forward (utils/quant.py:259-271, 319-329), HIP kernels only: the activation quantiser
    finds clampv = input.max() on the device and writes the int8 activations and the per-row scales, the int8 GEMM
    reads the module's bf16 qscales directly. per_token: one scale per token row from the row's own |max| instead.
    Returns (Y, x8, scale): scale is the quantiser's fp32 work buffer ([0] = clampv, [1] = alpha) or, per token,
    the fp32 [M] row scales."""
    x = _as_bf16_2d(input)
    sw, b = _qs_bias(qscales, bias)
    if x.shape[0] == 0:
        y = torch.empty((0, weight_i8.shape[0]), dtype=input.dtype, device=x.device)
        return y, torch.empty((0, x.shape[1]), dtype=torch.int8, device=x.device), torch.zeros(2, device=x.device)
    if per_token:
        x8, sx = ops.act_quant_i8_per_token(x)
        scale = sx
    else:
        x8, sx, scale = ops.act_quant_i8_dynamic(x, alpha_in_bf16)
    y = ops.a8w8_forward(x8, weight_i8.contiguous(), sx, sw, b)
    return (y if input.dtype == torch.bfloat16 else y.to(input.dtype)), x8, scale


def _per_token(qparamaw):
    """qparamaw is (clampv, qscales) as in the reference, or (clampv, qscales, "per_token")."""
    return len(qparamaw) > 2 and qparamaw[2] == "per_token"


def _fake_quant_activation(input, clampv):
    s = 127. / clampv
    if (FUSED_A8W8_DX and torch.is_tensor(s) and s.numel() == 1 and s.dtype == torch.bfloat16 and s.is_cuda
            and input.is_cuda and input.dtype == torch.bfloat16 and input.is_contiguous() and input.data_ptr() % 16 == 0):
        return ops.act_fake_quant(input, s.reshape(1))  # the chain below as one pass
    return (input * s).round_().clamp_(-128, 127).div_(s)


def _a8w8_backward_common(ctx, grad_output, input_f, weight_f, bias, detach_dw=False):
    """grad_input = dY . Wf and dW = dY^T . Xf on the dequantised operands (utils/quant.py:203-210). weight_f is the
    dense weight, or an (int8 codes, qscales) pair: then dX comes from the codes (ops.a8w8_dx: bf16(W8 * qs) is formed
    inside the GEMM, the values the reference's `weight_d.to(dtype) * qscales` holds) whenever the kernel takes the
    shapes. detach_dw is kept for the call sites' symmetry with the reference (the product has no history here)."""
    grad_input = grad_bias = None
    if ctx.needs_input_grad[0]:
        if isinstance(weight_f, tuple):
            w8, qscales = weight_f
            dy = grad_output if grad_output.is_contiguous() else grad_output.contiguous()
            qs = qscales.detach().reshape(-1)
            if FUSED_A8W8_DX and ops.a8w8_dx_ok(dy, w8, qs):
                grad_input = ops.a8w8_dx(dy, w8, qs)
            else:
                grad_input = grad_output.mm((w8.to(grad_output.dtype) * qscales).to(grad_output.dtype))
        else:
            grad_input = grad_output.mm(weight_f)
    dict_temp.append(_pending_dw(grad_output, input_f))
    if bias is not None and ctx.needs_input_grad[_BIAS_FLAG]:
        grad_bias = grad_output.sum(0)
    return grad_input, None, None, grad_bias


class QLinearFunctionA8W8_static(torch.autograd.Function):
    """Static activation clamp (utils/quant.py:172-211)."""

    @staticmethod
    def forward(input, weight_d, qparamaw, bias):
        clampv, qscales = qparamaw
        return _a8w8_linear(input, weight_d, qscales, bias, clampv, alpha_in_bf16=False)[0]

    @staticmethod
    def setup_context(ctx, inputs, output):
        input, weight_d, qparamaw, bias = inputs
        ctx.save_for_backward(input, weight_d.data, bias)
        ctx.save_qparamaw = qparamaw

    @staticmethod
    def backward(ctx, grad_output):
        input, weight_d, bias = ctx.saved_tensors
        clampv, qscales = ctx.save_qparamaw
        input_f = _fake_quant_activation(input, clampv)
        return _a8w8_backward_common(ctx, grad_output, input_f, (weight_d, qscales), bias, detach_dw=False)


class QLinearFunctionA8W8_dynamic0(torch.autograd.Function):
    """Dynamic clamp = input.max(), saves the bf16 input (utils/quant.py:214-252)."""

    @staticmethod
    def forward(ctx, input, weight_d, qparamaw, bias):
        qscales = qparamaw[1]
        out, _, work = _a8w8_linear_dynamic(input, weight_d, qscales, bias, alpha_in_bf16=False)
        ctx.save_for_backward(input, weight_d.data, bias)
        ctx.save_qparamaw = (work, qscales)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        input, weight_d, bias = ctx.saved_tensors
        work, qscales = ctx.save_qparamaw
        input_f = _fake_quant_activation(input, work[0].to(input.dtype))  # clampv = input.max(), a 0-dim tensor
        return _a8w8_backward_common(ctx, grad_output, input_f, (weight_d, qscales), bias, detach_dw=True)


class QLinearFunctionA8W8_dynamic(torch.autograd.Function):
    """Dynamic clamp, saves the int8 activations (utils/quant.py:254-293). This is the Function
    QLinearA8W8 dispatches to when training."""

    @staticmethod
    def forward(ctx, input, weight_d, qparamaw, bias):
        qscales = qparamaw[1]
        per_token = _per_token(qparamaw)
        out, x8, scale = _a8w8_linear_dynamic(input, weight_d, qscales, bias, alpha_in_bf16=True, per_token=per_token)
        ctx.save_qparamaw = (scale, qscales, per_token)
        ctx.save_for_backward(x8, weight_d.data, bias)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        x8, weight_d, bias = ctx.saved_tensors
        scale, qscales, per_token = ctx.save_qparamaw
        # x8 * (clampv / 127.): the quantiser left that bf16-valued alpha in scale[1]; per token: the row scales
        sv = scale.view(-1) if per_token else scale.view(-1)[1:2]
        if grad_output.dtype == torch.bfloat16 and ops.act_dequant_ok(x8, sv, per_token):
            input_f = ops.act_dequant_i8(x8, sv, per_token)  # the two tensor operations below as one pass
        else:
            s = scale.view(-1, 1) if per_token else scale[1]
            input_f = x8.to(grad_output.dtype) * s.to(grad_output.dtype)
        return _a8w8_backward_common(ctx, grad_output, input_f, (weight_d, qscales), bias, detach_dw=True)


class QLinearFunctionA8W8_static_eval(torch.autograd.Function):
    """utils/quant.py:296-312."""

    @staticmethod
    def forward(ctx, input, weight_d, qparamaw, bias):
        clampv, qscales = qparamaw
        return _a8w8_linear(input, weight_d, qscales, bias, clampv, alpha_in_bf16=False)[0]

    @staticmethod
    def backward(ctx, grad_output):
        return None, None, None, None


class QLinearFunctionA8W8_dynamic_eval(torch.autograd.Function):
    """utils/quant.py:314-331 (clamp = input.max(), kept on the device)."""

    @staticmethod
    def forward(ctx, input, weight_d, qparamaw, bias):
        return _a8w8_linear_dynamic(input, weight_d, qparamaw[1], bias, alpha_in_bf16=False, per_token=_per_token(qparamaw))[0]

    @staticmethod
    def backward(ctx, grad_output):
        return None, None, None, None


def _qat_weight_i8(weight_f, qscales):
    """clamp(round(weight_f / qscales), -128, 127) as int8 (utils/quant.py:345-346): one pass (lq_w8_requant, the
    same chain as Qfunc_8bit_res without a residual) where the kernel takes the operands."""
    if (FUSED_LATENT and weight_f.is_cuda and weight_f.dim() == 2 and weight_f.dtype == torch.bfloat16
            and weight_f.is_contiguous() and weight_f.shape[1] % 8 == 0 and weight_f.data_ptr() % 16 == 0
            and torch.is_tensor(qscales) and qscales.dtype == torch.bfloat16 and qscales.is_contiguous()
            and qscales.is_cuda and tuple(qscales.shape) == (weight_f.shape[0], 1)):
        return ops.w8_requant(weight_f, qscales)
    return (weight_f / qscales).round_().clamp_(-128, 127).to(torch.int8)


class QLinearFunctionQAT_dynamic(torch.autograd.Function):
    """bf16 latent weight, quantised to int8 on the fly (utils/quant.py:334-374)."""

    @staticmethod
    def forward(ctx, input, weight_f, qparamaw, bias):
        qscales = qparamaw[1]
        out, _, work = _a8w8_linear_dynamic(input, _qat_weight_i8(weight_f, qscales), qscales, bias, alpha_in_bf16=False)
        ctx.save_for_backward(input, weight_f.data, bias)
        ctx.save_qparamaw = (work, qscales)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        input, weight_f, bias = ctx.saved_tensors
        work, qscales = ctx.save_qparamaw
        input_f = _fake_quant_activation(input, work[0].to(input.dtype))
        # the fake-quantised weight (utils/quant.py:363-365) is bf16(w8 * qscales) for the int8 codes of the forward:
        # handed over as codes, so that the input gradient forms it inside its GEMM
        if weight_f.dtype == torch.bfloat16 and input.dtype == torch.bfloat16:
            weight_q = (_qat_weight_i8(weight_f, qscales), qscales)
        else:
            weight_q = (weight_f / qscales).round_().clamp_(-128, 127).mul_(qscales).to(input.dtype)
        return _a8w8_backward_common(ctx, grad_output, input_f, weight_q, bias, detach_dw=False)


class QLinearFunctionQAT_dynamic_eval(torch.autograd.Function):
    """utils/quant.py:376-394."""

    @staticmethod
    def forward(ctx, input, weight_f, qparamaw, bias):
        qscales = qparamaw[1]
        return _a8w8_linear_dynamic(input, _qat_weight_i8(weight_f, qscales), qscales, bias, alpha_in_bf16=False)[0]

    @staticmethod
    def backward(ctx, grad_output):
        return None, None, None, None


# -------------------------------------------------------------------------- backward hook --
def backward_hook_fn(module, grad_out, grad_in):
    """Full-backward hook: move the pending dW into module.weight.grad (utils/quant.py:398-411)."""
    assert len(dict_temp) == 1
    dw = dict_temp.pop()
    g = module.weight.grad
    if isinstance(dw, _PendingWeightGrad):
        if isinstance(g, GradientQTensor) and g.acc_ite > 0 and g.can_add_product(dw.dy, dw.x):
            g.add_product_(dw.dy, dw.x)
            return
        if FUSED_GRADQ and torch.is_tensor(g) and ops.weight_grad_acc_ok(dw.dy, dw.x, g):
            ops.weight_grad_acc(dw.dy, dw.x, g)  # g.add_(dW) as the GEMM's epilogue
            return
        dw = dw.tensor()
    if isinstance(g, GradientQTensor):
        if g.acc_ite == 0:
            g.set_value(dw)
        else:
            g.add_(dw)
    elif g is None:
        module.weight.grad = dw
    else:
        g.add_(dw)


# -------------------------------------------------------------------------------- modules --
class _QLinearBase(nn.Module):
    _repr_name = "QLinear"

    def __init__(self, input_features, output_features, bias):
        super().__init__()
        self.input_features = input_features
        self.output_features = output_features
        if bias:
            self.bias = nn.Parameter(torch.empty(output_features))
        else:
            self.register_parameter('bias', None)
        self.register_buffer('qweight', torch.tensor([]))  # filled by before_save()
        self.wshape = [output_features, input_features]
        self.hook_handle = None

    def add_hook(self):
        self.hook_handle = self.register_full_backward_hook(backward_hook_fn)

    def _apply_fn(self, fn, x):
        out = fn.apply(x.reshape(-1, x.shape[-1]), self.weight.data, self._qparam(), self.bias)
        return out.reshape(x.shape[:-1] + (self.output_features,))

    def forward(self, x):
        return self._apply_fn(self._fn_eval if self.hook_handle is None else self._fn_train, x)

    def forward_eval(self, x):
        return self._apply_fn(self._fn_eval, x)

    def before_save(self):
        self.qweight.data = self.weight.data.cpu()

    def extra_repr(self):
        return '{} input_features={}, output_features={}, bias={}'.format(
            self._repr_name, self.input_features, self.output_features, self.bias is not None)


class QLinearA16W4(_QLinearBase):
    """A16W4 linear (utils/quant.py:413-482). Buffers: qweight, zeros, scales (bf16 [(N*K/128),1]);
    ``weight`` is a QuantTensor holding the packed codes."""
    _repr_name = "QLinearA16W4"
    _fn_train, _fn_eval = QLinearFunctionW4, QLinearFunctionW4_eval

    def __init__(self, input_features, output_features, bias=True, lbit=0, gbit=16):
        super().__init__(input_features, output_features, bias)
        self.groupsize = GROUPSIZE
        ngroups = math.ceil(input_features / GROUPSIZE) * output_features
        self.register_buffer('zeros', torch.zeros((ngroups, 1), dtype=torch.bfloat16))
        self.register_buffer('scales', torch.zeros((ngroups, 1), dtype=torch.bfloat16))
        self.weight = QuantTensor([output_features, input_features], lbit=lbit, wbit=4, gbit=gbit)

    def _qparam(self):
        return self.weight.qparam

    def to(self, device: Optional[Union[int, torch.device]]):
        """Moves the QuantTensor and re-binds its qparam to the moved buffers; returns None like
        the reference (utils/quant.py:462-469)."""
        self.weight = self.weight.to(device=device)
        self.zeros = self.zeros.to(device=device)
        self.scales = self.scales.to(device=device)
        self.weight.set_value(None, [self.scales, self.zeros, self.wshape])
        if self.bias is not None:
            self.bias.data = self.bias.data.to(device)


class QLinearA8W8(_QLinearBase):
    """A8W8 linear (utils/quant.py:485-541). Buffers: qweight, clampv[1], qscales bf16 [N,1]."""
    _repr_name = "QLinearA8W8"
    _fn_train, _fn_eval = QLinearFunctionA8W8_dynamic, QLinearFunctionA8W8_dynamic_eval

    def __init__(self, input_features, output_features, bias=True, lbit=0, gbit=8):
        super().__init__(input_features, output_features, bias)
        self.register_buffer('clampv', torch.ones(1))
        self.register_buffer('qscales', torch.zeros(output_features, 1, dtype=torch.bfloat16))
        self.weight = QuantTensor([output_features, input_features], lbit=lbit, wbit=8, gbit=gbit)
        # "per_tensor": the reference's activation quantiser (one clamp value = input.max()); "per_token": one
        # scale per token row (an addition; set the attribute after construction)
        self.act_quant = "per_tensor"

    def _qparam(self):
        # the dynamic Functions ignore the stored clamp (utils/quant.py:259-260): no .item() sync here
        if self.act_quant == "per_token":
            return (self.clampv, self.qscales.data, "per_token")
        return (self.clampv, self.qscales.data)

    def to(self, device: Optional[Union[int, torch.device]]):
        self.weight = self.weight.to(device=device)
        self.qscales = self.qscales.to(device=device)
        self.weight.set_value(None, self.qscales)
        if self.bias is not None:
            self.bias.data = self.bias.data.to(device)


class QLinearQAT(_QLinearBase):
    """bf16 latent weight + int8 fake-quant forward (utils/quant.py:544-599)."""
    _repr_name = "QLinearQAT"
    _fn_train, _fn_eval = QLinearFunctionQAT_dynamic, QLinearFunctionQAT_dynamic_eval

    def __init__(self, input_features, output_features, bias=True, lbit=0, gbit=16):
        super().__init__(input_features, output_features, bias)
        self.register_buffer('clampv', torch.ones(1))
        self.register_buffer('qscales', torch.zeros(output_features, 1, dtype=torch.bfloat16))
        assert gbit == 16
        self.weight = FPTensor(torch.empty((output_features, input_features), dtype=torch.bfloat16))

    def _qparam(self):
        return (self.clampv, self.qscales.data)

    def before_save(self):
        self.qweight.data = _qat_weight_i8(self.weight.data, self.qscales).cpu()

    def to(self, device: Optional[Union[int, torch.device]]):
        self.weight = self.weight.to(device=device)
        if self.bias is not None:
            self.bias.data = self.bias.data.to(device)


# ---------------------------------------------------------------------- latent containers --
def prodx(ls):
    return reduce(lambda x, y: x * y, ls)


class _LatentBase(object):
    """Shared behaviour of the non-tensor "parameters" handed to the optimizer."""

    def numel(self):
        return prodx(self.shape)

    def get_self(self):
        return self

    def __repr__(self):
        return "Quant value:\n{}\n with param:\n{}".format(getattr(self, 'data', None), self.qparam)

    def requires_grad_(self, boolv):
        self.requires_grad = boolv
        return self

    @property
    def device(self):
        return self.data.device

    @property
    def type(self):
        return self.data.type


class QuantTensor(_LatentBase):
    """Packed weight + latent information (utils/quant.py:606-663). ``lbit`` selects how the
    sub-LSB part of the latent weight is kept: 4 -> ResidualTensor (4-bit codec), 16 -> a bf16 copy,
    anything else -> an fp32 copy as in the reference, except that a 4-bit weight with lbit 0 stores
    nothing (stochastic-rounding requantizer). An 8-bit weight always keeps a latent: main0.py:339-340
    fills ``residual.data`` of a default-constructed QLinearA8W8."""

    def __init__(self, shape, wbit=8, gbit=8, lbit=4):
        self.shape = shape
        self.wbit = wbit
        self.initial = False
        self.qparam = None
        self.lbit = lbit
        if lbit == 4:
            channels = shape[0] if wbit == 8 else prodx(shape) // GROUPSIZE
            self.residual = ResidualTensor(qshape=[channels, prodx(shape) // channels], oshape=shape)
        elif lbit == 16:
            self.residual = torch.empty(shape, dtype=torch.bfloat16)
        elif lbit == 0 and wbit == 4:
            self.residual = None
        else:
            self.residual = torch.empty(shape, dtype=torch.float32)
        self.requires_grad = True
        self.grad = None if gbit == 16 else GradientQTensor(self.shape, bit=gbit)

    def set_value(self, data, qparam=None):
        if data is not None:
            self.data = data.clone()
        self.qparam = qparam
        self.initial = True
        self.requires_grad = True

    def to(self, device=None, dtype=None):
        if device is not None:
            self.data = self.data.to(device)
            if isinstance(self.residual, ResidualTensor):
                self.residual.residual_int = self.residual.residual_int.to(device)
            elif self.residual is not None:
                self.residual = self.residual.to(device)
        return self


class FPTensor(_LatentBase):
    """Plain bf16 latent weight of the QAT layer (utils/quant.py:666-705)."""

    def __init__(self, data, gbit=16):
        self.data = data
        self.shape = data.shape
        self.initial = False
        self.qparam = None
        self.requires_grad = True
        self.grad = None if gbit == 16 else GradientQTensor(self.shape, bit=gbit)

    def to(self, device=None, dtype=None):
        if device is not None:
            self.data = self.data.to(device)
        return self


# ------------------------------------------------------------------- 4-bit residual codec --
def three_fold_curve_4bit(mu):
    """(levels, breakpoint) pairs of the companding curve per mu level (utils/quant.py:708-716)."""
    table = {3: (2, 0.4330623539159437, 4, 0.46875), 2: (2, 0.37272211741724515, 4, 0.4375),
             1: (2, 0.2666300266320331, 4, 0.375)}
    return table.get(mu, (2, 0.125, 4, 0.25))


class _ResidualCodec(object):
    """Stands in for the reference's JIT-built ``cuda_module`` (utils/quant.py:718-719,
    multi_random_quant.cpp:38-54) with the same five entry points, backed by the HIP codec."""

    @staticmethod
    def quant(fp, q, k1, b1, k2, b2, k3):
        ops.residual_quant(fp, q.view(-1), 0, int(k1), b1, int(k2), b2, int(k3))

    @staticmethod
    def dequant(q, fp, k1, b1, k2, b2, k3):
        fp.copy_(ops.residual_dequant(q.view(-1), 0, int(k1), b1, int(k2), b2, int(k3)).view(fp.shape))

    @staticmethod
    def uniform_quant(fp, q):
        ops.residual_quant(fp, q.view(-1), 1)

    @staticmethod
    def uniform_quant_s(fp, q):
        """multi_random_quant.cpp:33-36: fp32 / fp16 / fp64 as the reference dispatches it, bf16 in addition."""
        ops.residual_quant_s(fp, q.view(-1))

    @staticmethod
    def uniform_dequant(q, fp):
        fp.copy_(ops.residual_dequant(q.view(-1), 1).view(fp.shape))


cuda_module = _ResidualCodec()


@torch.no_grad()
def cuda_quant_linear(residual_fp, q_tensor):
    """utils/quant.py:723-733."""
    residual_fp = residual_fp.to(EXT_type)
    assert residual_fp.is_contiguous()
    if not residual_fp.is_cuda:
        return python_quant_linear(residual_fp)
    cuda_module.uniform_quant(residual_fp, q_tensor)
    return residual_fp


@torch.no_grad()
def cuda_quant_3fold(residual_fp, q_tensor, p1, y1, p2, y2):
    """utils/quant.py:735-742: returns the carry tensor (the overwritten bf16 copy of the input)."""
    residual_fp = residual_fp.to(EXT_type)
    if not residual_fp.is_contiguous() or residual_fp.data_ptr() % 16:
        residual_fp = residual_fp.contiguous().clone()
    assert residual_fp.is_cuda
    cuda_module.quant(residual_fp, q_tensor, p1, y1, p2 - p1, y2, 8 - p2)
    return residual_fp


@torch.no_grad()
def cuda_dequant_linear(residual_int):
    """utils/quant.py:746-755."""
    assert residual_int.is_contiguous()
    if not residual_int.is_cuda:
        return python_dequant_linear(residual_int)
    return ops.residual_dequant(residual_int.view(-1), 1)


@torch.no_grad()
def cuda_dequant_3fold(residual_int, p1, y1, p2, y2):
    """utils/quant.py:757-763."""
    assert residual_int.is_cuda and residual_int.is_contiguous()
    return ops.residual_dequant(residual_int.view(-1), 0, int(p1), y1, int(p2 - p1), y2, int(8 - p2))


@torch.no_grad()
def python_quant_linear(residual_fp):
    """CPU stochastic uniform 4-bit quantizer (utils/quant.py:765-778): round((x+.5)*16 + U(-.5,.5)),
    level 16 wraps to 0 with a carry; eight nibbles per int32, MSB first."""
    lv = (residual_fp + 0.5) * 16
    lv.add_(torch.empty_like(lv).uniform_(-0.5, 0.5)).round_()
    over = lv > 15.9
    lv[over] = 0.
    carry = torch.zeros_like(residual_fp)
    carry[over] = 1.
    nib = lv.view(-1, 8).to(torch.int32)
    shifts = torch.arange(28, -4, -4, dtype=torch.int32, device=nib.device)
    return (nib << shifts).sum(dim=1, dtype=torch.int32).contiguous(), carry


@torch.no_grad()
def python_dequant_linear(residual_int):
    """utils/quant.py:781-788."""
    shifts = torch.arange(28, -4, -4, dtype=torch.int32, device=residual_int.device)
    nib = (residual_int.view(-1, 1) >> shifts) % 16
    return nib.to(torch.float32) / 16 - 0.5


class ResidualTensor(object):
    """Z - round(Z) in [-0.5, 0.5] at 4 bits per element (utils/quant.py:790-841)."""

    def __init__(self, qshape, oshape):
        self.weight_scale = None
        self.qshape = qshape
        self.oshape = oshape
        self.lock_mu = self.mu = 0
        numel_h = prodx(oshape)
        assert numel_h % 8 == 0
        dev = 'cuda' if torch.cuda.is_available() else 'cpu'
        self.residual_int = torch.empty((numel_h // 8, 1), dtype=torch.int32, device=dev)
        self.name = 'residual'
        self.init = True

    def set_value(self, residual_fp, weight_scale=None):
        p1, y1, p2, y2 = three_fold_curve_4bit(self.mu)
        adj = cuda_quant_3fold(residual_fp, self.residual_int, p1, y1, p2, y2)
        if weight_scale is not None:
            self.weight_scale = weight_scale
        self.lock_mu = self.mu
        self.init = False
        return adj

    def update_mu(self, optmizer_std):
        """Pick the companding curve from the ratio scale / typical update (utils/quant.py:813-824);
        as in the reference the `> 75.8` test is overwritten by the chain below it."""
        mu = (self.weight_scale / (optmizer_std + 1e-8)).mean().item()
        self.mu = 2 if mu > 36.5 else (1 if mu > 16.2 else 0)
        if self.mu != self.lock_mu:
            print(f'{self.name} now mu level is {mu}({self.mu}), pre is {self.lock_mu}')

    def dequant(self):
        p1, y1, p2, y2 = three_fold_curve_4bit(self.lock_mu)
        return cuda_dequant_3fold(self.residual_int, p1, y1, p2, y2)

    def add(self, tensor: torch.Tensor):
        if self.init:
            return tensor
        r = (self.dequant().view(self.qshape) * self.weight_scale).to(dtype=tensor.dtype)
        return r.view(self.oshape).add(tensor)

    def __repr__(self):
        return "ResidualTensor !"


class GradientQTensor(object):
    """Gradient accumulator of a quantised weight (utils/quant.py:846-922): for ``bit <= 8`` an int8
    tensor with one scale per output row and stochastic rounding, otherwise the plain tensor.

    On the GPU with a bf16 gradient the 8-bit forms are one HIP pass each (``ops.gradq8_quant``):
    ``set_value`` finds the row scales and quantises, ``add_`` quantises ``dequant() + fdata`` with
    the scales of the first micro-batch, both with the bf16 rounding points of the reference's
    tensor operations. The rounding noise comes from the library's Philox stream (``noise_seed`` and
    a running counter shared by all instances); ``noise=`` injects a bf16 tensor instead. Anything
    else (CPU tensors, other dtypes, FUSED_GRADQ off) runs the tensor-op chain with ``uniform_``."""

    # Key of the rounding-noise stream. None: taken from torch.initial_seed() at first use, so that
    # torch.manual_seed() before training changes the noise as it does for the reference's uniform_(); set it to
    # an integer to fix the stream by hand. The counter offset is a host-side count passed with every launch: a
    # launch captured into a HIP graph would replay the same noise, so accumulators must not be captured.
    noise_seed = None
    _noise_offset = 0  # Philox blocks consumed so far by all instances

    @classmethod
    def _seed(cls):
        if cls.noise_seed is None:
            cls.noise_seed = torch.initial_seed() & (2 ** 64 - 1)
        return cls.noise_seed

    def __init__(self, shape, bit=8):
        self.acc_ite = 0
        self.bit = bit
        self.qdata = 0
        self.scale = None
        self.qzero = None
        self.shape = shape
        self.fixscale = False

    def find_param(self, data):
        """Row scale 4 * max|row| / 127, floored at 1e-5 / 127 (utils/quant.py:856-861; the factor 4
        leaves head room for the micro-batches that add_ accumulates)."""
        self.vmax = data.abs().amax(dim=1, keepdim=True) * 4
        self.scale = (torch.clamp(self.vmax, min=1e-5) / (2 ** (self.bit - 1) - 1)).to(data.dtype)

    def _hip_ok(self, fdata):
        return (FUSED_GRADQ and self.bit == 8 and fdata.is_cuda and fdata.dtype == torch.bfloat16 and fdata.dim() == 2
                and fdata.is_contiguous() and fdata.shape[1] % 16 == 0 and fdata.data_ptr() % 16 == 0)

    def _hip_quant(self, fdata, accumulate, noise):
        cls = GradientQTensor
        if not accumulate:
            self.qdata = torch.empty(fdata.shape, dtype=torch.int8, device=fdata.device)
            self.scale = torch.empty((fdata.shape[0], 1), dtype=torch.bfloat16, device=fdata.device)
        ops.gradq8_quant(fdata, self.qdata, self.scale, accumulate, noise=noise, seed=cls._seed(), offset=cls._noise_offset)
        if noise is None:
            cls._noise_offset += (fdata.numel() + 15) // 16

    def quant(self, fdata, noise=None):
        if noise is None:
            noise = torch.empty_like(fdata).uniform_(-0.5, 0.5)
        q = torch.round(fdata / self.scale + noise)
        self.qdata = torch.clamp(q, -2 ** (self.bit - 1), 2 ** (self.bit - 1) - 1).to(torch.int8)

    def dequant(self):
        return self.qdata.to(self.fdtype) * self.scale

    def set_value(self, fdata, noise=None):
        if self.bit > 8:
            self.qdata = fdata
            return
        self.fdtype = fdata.dtype
        if self._hip_ok(fdata) and not self.fixscale:
            self._hip_quant(fdata, False, noise)
        else:
            if not (self.fixscale and self.scale is None):
                self.find_param(fdata)
            self.quant(fdata, noise)
        self.acc_ite = 1

    def zero(self):
        self.acc_ite = 0
        self.qdata = None

    def add_(self, fdata, noise=None):
        if self.bit > 8:
            self.qdata += fdata
            return
        self.acc_ite += 1
        if (self._hip_ok(fdata) and isinstance(self.qdata, torch.Tensor) and self.qdata.is_cuda and self.qdata.is_contiguous()
                and self.scale is not None and self.scale.dtype == torch.bfloat16 and self.scale.is_contiguous()
                and self.fdtype == torch.bfloat16):
            self._hip_quant(fdata, True, noise)
        else:
            self.quant(self.dequant() + fdata, noise)

    def can_add_product(self, dy, x):
        """Whether add_product_ applies: an 8-bit accumulator that already holds a micro-batch, on the GPU, and
        operands the weight-gradient GEMM takes."""
        return (FUSED_GRADQ and self.bit == 8 and isinstance(self.qdata, torch.Tensor) and self.qdata.is_cuda
                and self.qdata.is_contiguous() and self.qdata.dtype == torch.int8 and self.scale is not None
                and self.scale.dtype == torch.bfloat16 and self.scale.is_contiguous()
                and getattr(self, "fdtype", None) == torch.bfloat16 and ops._weight_grad_native_ok(dy, x, 16)
                and tuple(self.qdata.shape) == (dy.shape[1], x.shape[1]))

    def add_product_(self, dy, x, noise=None):
        """add_(dy.t().mm(x)) without the product ever being stored: the GEMM's epilogue re-quantises
        dequant() + dW in place (ops.weight_grad_acc8), bit for bit what add_ does with the bf16 product."""
        cls = GradientQTensor
        self.acc_ite += 1
        ops.weight_grad_acc8(dy, x, self.qdata, self.scale, noise=noise, seed=cls._seed(), offset=cls._noise_offset)
        if noise is None:
            cls._noise_offset += (self.qdata.numel() + 15) // 16

    def get_value(self):
        return self.qdata if self.bit > 8 else self.dequant()

    def __repr__(self):
        return f"GradientQTensor bitwidth {self.bit} !"

    def to(self, device):
        self.qdata = self.qdata.to(device)
        if self.bit <= 8:
            self.scale = self.scale.to(device)
            if self.qzero is not None:
                self.qzero = self.qzero.to(device)
        return self

    @property
    def device(self):
        return self.qdata.device


# ------------------------------------------------------------------------------ optimizer --
class MyAdam(torch.optim.Adam):
    """Adam over a mix of nn.Parameters and QuantTensor/FPTensor latents with optional block-wise
    8-bit moments (utils/quant.py:927-1148). For a QuantTensor the latent weight is rebuilt
    (dequantised codes + stored residual), stepped, and re-quantised; with ``lbit=0`` the whole
    rebuild/step/re-quantise tail is one call of the stochastic-rounding requantizer.

    ``sr_seed`` seeds the Philox stream of that requantizer; every call consumes N*K/8 counters."""

    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), obit=8, mu_updata_f=20, cpu=False, sr_seed=0):
        super().__init__(params, lr=lr, betas=betas)
        self.initialized = False
        self.obit = obit
        self.mu_updata_f = mu_updata_f
        self.statedevice = 'cpu' if cpu else 'cuda'
        self.sr_seed = sr_seed
        self.sr_offset = 0

    def add_param_group(self, param_group):
        """Accepts QuantTensor / FPTensor objects next to tensors (utils/quant.py:934-959)."""
        assert isinstance(param_group, dict), "param group must be a dict"
        params = param_group['params']
        if isinstance(params, torch.Tensor):
            param_group['params'] = [params]
        elif isinstance(params, set):
            raise TypeError('optimizer parameters need to be organized in ordered collections, but '
                            'the ordering of tensors in sets will change between runs. Please use a list instead.')
        else:
            param_group['params'] = list(params)
        for name, default in self.defaults.items():
            param_group.setdefault(name, default)
        seen = set()
        for group in self.param_groups:
            seen.update(group['params'])
        if not seen.isdisjoint(param_group['params']):
            raise ValueError("some parameters appear in more than one parameter group")
        self.param_groups.append(param_group)

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        for gindex, group in enumerate(self.param_groups):
            for pindex, p in enumerate(group["params"]):
                if p.grad is None:
                    continue
                if len(self.state[p]) == 0:
                    self.init_state(group, p, gindex, pindex)
                self.update_step(group, p, gindex, pindex)
        return loss

    def to_gpu(self):
        for group in self.param_groups:
            for p in group["params"]:
                if p in self.state:
                    for k, v in self.state[p].items():
                        if isinstance(v, torch.Tensor) and not getattr(v, 'is_paged', False):
                            self.state[p][k] = v.to(p.device)

    def get_config(self, gindex, pindex, group):
        return {"betas": group["betas"], "eps": group["eps"], "weight_decay": group["weight_decay"],
                "lr": group["lr"], "block_wise": True}

    def get_state_buffer(self, pshape, pdevice, dtype=torch.float32):
        return torch.zeros(pshape, dtype=dtype, device=pdevice)

    @torch.no_grad()
    def init_state(self, group, p, gindex, pindex):
        """bf16 moments for small tensors or obit=16, else uint8 moments with one (scale, max) pair
        per block of 2048 (or 128) elements (utils/quant.py:1014-1059)."""
        config = self.get_config(gindex, pindex, group)
        dtype = torch.uint8 if self.obit == 8 else torch.bfloat16
        if p.numel() < 65536:
            dtype = torch.bfloat16
        state = self.state[p]
        state["step"] = 0
        sdev = self.statedevice if (self.statedevice == 'cpu' or torch.cuda.is_available()) else 'cpu'
        state["state1"] = self.get_state_buffer(p.shape, sdev, dtype=dtype)
        state["state2"] = self.get_state_buffer(p.shape, sdev, dtype=dtype)
        if dtype == torch.uint8:
            n = p.numel()
            if not config["block_wise"]:
                blocks = 1
            elif n % 2048 == 0:
                blocks = n // 2048
            else:
                assert n % 128 == 0
                blocks = n // 128
            for name, fill in (("absmax1", 0.0), ("qmap1", 1e-10), ("absmax2", 0.0), ("qmap2", 1e-10)):
                state[name] = torch.full((blocks, 1), fill, dtype=torch.float32, device=p.device)

    def _latent(self, p, dtype):
        """Latent weight of a QuantTensor: dequantised codes + residual (utils/quant.py:1066-1079)."""
        if isinstance(p.residual, ResidualTensor):
            if p.wbit == 8:
                r, qs = p.residual, p.qparam
                if (FUSED_LATENT and not r.init and dtype == torch.bfloat16 and p.data.is_cuda and p.data.dtype == torch.int8
                        and p.data.dim() == 2 and p.data.is_contiguous() and p.data.shape[1] % 16 == 0
                        and torch.is_tensor(qs) and qs.dtype == torch.bfloat16 and qs.is_contiguous()
                        and tuple(qs.shape) == (p.data.shape[0], 1) and r.weight_scale is not None
                        and r.weight_scale.data_ptr() == qs.data_ptr() and r.residual_int.is_cuda):
                    p1, y1, p2, y2 = three_fold_curve_4bit(r.lock_mu)
                    return ops.latent_w8_reconstruct(p.data, qs.view(-1), r.residual_int.view(-1), p1, y1, p2 - p1, y2, 8 - p2)
                return p.residual.add((p.data * p.qparam).to(dtype))
            if p.wbit == 4:
                r = p.residual
                scales, zeros, shape = _flat_qparam(p.qparam)
                if (FUSED_LATENT and not r.init and dtype == torch.bfloat16 and p.data.is_cuda
                        and scales.dtype == torch.bfloat16 and zeros.dtype == torch.bfloat16
                        and r.weight_scale is not None and r.weight_scale.dtype == torch.bfloat16
                        and r.weight_scale.data_ptr() == scales.data_ptr() and r.weight_scale.numel() == scales.numel()):
                    p1, y1, p2, y2 = three_fold_curve_4bit(r.lock_mu)
                    return ops.latent_w4_reconstruct(p.data.contiguous(), scales, zeros, r.residual_int.view(-1),
                                                     tuple(shape), p1, y1, p2 - p1, y2, 8 - p2)
                return p.residual.add(DeQfunc_4bit_g(p.data, p.qparam, dtype))
            raise AssertionError("wbit must be 4 or 8")
        return p.residual.data.to(dtype)

    @torch.no_grad()
    def update_step(self, group, p, gindex, pindex):
        state = self.state[p]
        config = self.get_config(gindex, pindex, group)
        grad = p.grad
        is_q = isinstance(p, QuantTensor)
        sr_mode = is_q and p.wbit == 4 and p.residual is None
        if is_q and isinstance(grad, GradientQTensor):
            grad = grad.get_value()
        q8 = state["state1"].dtype == torch.uint8
        mu_step = (state["step"] + 1 > 250 and (state["step"] + 1) % self.mu_updata_f == (self.mu_updata_f - 1)
                   and isinstance(getattr(p, 'residual', None), ResidualTensor))
        adam8_ok = (FUSED_ADAM8 and q8 and config["weight_decay"] == 0 and not mu_step and grad.is_cuda
                    and grad.dtype == torch.bfloat16 and grad.is_contiguous()
                    and all(state[k].device == grad.device and state[k].is_contiguous()
                            for k in ("state1", "state2", "qmap1", "absmax1", "qmap2", "absmax2"))
                    and p.numel() // len(state["absmax1"]) in (2048, 128))
        if adam8_ok and FUSED_LATENT and is_q and not sr_mode and self._fused_latent_step(group, p, state, config, grad):
            return
        if is_q:
            pdata = None if sr_mode else self._latent(p, grad.dtype)
        else:
            pdata = p.data

        if adam8_ok and (sr_mode or (pdata.dtype == torch.bfloat16 and pdata.is_contiguous())):
            # the whole chain below as one kernel (moments, their block parameters and pdata updated in place)
            beta1, beta2 = config["betas"]
            state["step"] += 1
            bias_correction1 = 1 - beta1 ** state["step"]
            bias_correction2 = 1 - beta2 ** state["step"]
            step_size = config["lr"] * math.sqrt(bias_correction2) / bias_correction1
            direction = torch.empty_like(grad) if sr_mode else None
            ops.adam8_update(grad, state["state1"], state["state2"], state["qmap1"], state["absmax1"], state["qmap2"],
                             state["absmax2"], beta1, beta2, group["eps"], step_size,
                             param=None if sr_mode else pdata, direction=direction)
            self._requantise(p, pdata, direction if sr_mode else None, step_size, is_q, sr_mode)
            return
        if q8:
            exp_avg = DeQfunc_8bit_opt(state["state1"].to(grad.device), [state["qmap1"], state["absmax1"]]).to(grad.dtype)
            s2 = DeQfunc_8bit_opt(state["state2"].to(grad.device), [state["qmap2"], state["absmax2"]])
            exp_avg_sq = (s2 * s2).to(grad.dtype)
        else:
            exp_avg = state["state1"].to(grad.device)
            exp_avg_sq = (state["state2"] * state["state2"]).to(grad.device)

        beta1, beta2 = config["betas"]
        state["step"] += 1
        if config["weight_decay"] != 0:
            wd_base = DeQfunc_4bit_g(p.data, p.qparam, grad.dtype) if sr_mode else pdata
            grad = grad.add(wd_base, alpha=config["weight_decay"])

        exp_avg.mul_(beta1).add_(grad, alpha=1 - beta1)
        exp_avg_sq.mul_(beta2).addcmul_(grad, grad, value=1 - beta2)
        exp_avg_sqrt = exp_avg_sq.sqrt_()
        denom = exp_avg_sqrt.add_(group["eps"])
        bias_correction1 = 1 - beta1 ** state["step"]
        bias_correction2 = 1 - beta2 ** state["step"]
        step_size = config["lr"] * math.sqrt(bias_correction2) / bias_correction1

        if sr_mode:
            direction = (exp_avg / denom).to(torch.bfloat16).contiguous()
        else:
            pdata.addcdiv_(exp_avg, denom, value=-step_size)

        if (state["step"] > 250 and state["step"] % self.mu_updata_f == (self.mu_updata_f - 1)
                and isinstance(getattr(p, 'residual', None), ResidualTensor)):
            std = torch.mean((abs(exp_avg) / denom).view(p.residual.qshape), dim=1, keepdim=True) * step_size
            p.residual.update_mu(std)

        if q8:
            nblk = len(state["absmax1"])
            s1, qp = Qfunc_8bit_opt(exp_avg.float(), blocksize=nblk)
            state["state1"] = s1.to(state["state1"].device)
            state["qmap1"], state["absmax1"] = qp
            s2q, qp = Qfunc_8bit_opt(exp_avg_sqrt.float(), blocksize=nblk)
            state["state2"] = s2q.to(state["state2"].device)
            state["qmap2"], state["absmax2"] = qp
        else:
            state["state1"] = exp_avg
            state["state2"] = exp_avg_sq  # holds sqrt(v) + eps after the in-place ops above, as in the reference

        self._requantise(p, pdata, direction if sr_mode else None, step_size, is_q, sr_mode)

    def _fused_latent_step(self, group, p, state, config, grad):
        """The whole step of an lbit = 4 layer (latent from codes + residual, Adam on uint8 moments,
        back to codes + residual) as one kernel, when every piece is in the form the kernel takes;
        returns False to let the separate passes run."""
        r = p.residual
        if not (p.wbit in (4, 8) and isinstance(r, ResidualTensor) and not r.init and p.data.is_cuda
                and p.data.is_contiguous() and r.residual_int.is_cuda and r.residual_int.is_contiguous()):
            return False
        moments = (state["state1"], state["state2"], state["qmap1"], state["absmax1"], state["qmap2"], state["absmax2"])
        if p.wbit == 8:
            # 8-bit weights: int8 codes [N, K], one bf16 scale per row (the conditions of _latent and Qfunc_8bit_res)
            qs = p.qparam
            if not (p.data.dtype == torch.int8 and p.data.dim() == 2 and p.data.shape[1] % 16 == 0 and torch.is_tensor(qs)
                    and qs.dtype == torch.bfloat16 and qs.is_contiguous() and tuple(qs.shape) == (p.data.shape[0], 1)
                    and r.weight_scale is not None and r.weight_scale.data_ptr() == qs.data_ptr()):
                return False
            beta1, beta2 = config["betas"]
            state["step"] += 1
            step_size = config["lr"] * math.sqrt(1 - beta2 ** state["step"]) / (1 - beta1 ** state["step"])
            p1, y1, p2, y2 = three_fold_curve_4bit(r.lock_mu)
            q1, z1, q2, z2 = three_fold_curve_4bit(r.mu)
            ops.adam8_latent_w8_step(grad, p.data, r.residual_int.view(-1), qs.view(-1), *moments,
                                     (p1, y1, p2 - p1, y2, 8 - p2), (q1, z1, q2 - q1, z2, 8 - q2), beta1, beta2,
                                     group["eps"], step_size)
            r.weight_scale = qs
            r.lock_mu = r.mu
            if isinstance(p.grad, GradientQTensor):
                p.grad.zero()
            else:
                p.grad = None
            return True
        scales, zeros, shape = _flat_qparam(p.qparam)
        if not (scales.dtype == torch.bfloat16 and zeros.dtype == torch.bfloat16 and scales.is_contiguous()
                and zeros.is_contiguous() and r.weight_scale is not None and r.weight_scale.dtype == torch.bfloat16
                and r.weight_scale.data_ptr() == scales.data_ptr() and r.weight_scale.numel() == scales.numel()):
            return False
        beta1, beta2 = config["betas"]
        state["step"] += 1
        step_size = config["lr"] * math.sqrt(1 - beta2 ** state["step"]) / (1 - beta1 ** state["step"])
        p1, y1, p2, y2 = three_fold_curve_4bit(r.lock_mu)
        q1, z1, q2, z2 = three_fold_curve_4bit(r.mu)
        ops.adam8_latent_w4_step(grad, p.data, r.residual_int.view(-1), scales, zeros, tuple(shape), *moments,
                                 (p1, y1, p2 - p1, y2, 8 - p2), (q1, z1, q2 - q1, z2, 8 - q2), beta1, beta2,
                                 group["eps"], step_size)
        r.weight_scale = scales.contiguous().reshape(-1, 1)
        r.lock_mu = r.mu
        if isinstance(p.grad, GradientQTensor):
            p.grad.zero()
        else:
            p.grad = None
        return True

    def _requantise(self, p, pdata, direction, step_size, is_q, sr_mode):
        """Back from the updated latent weight (or, in stochastic-rounding mode, from the update
        direction) to codes, and the gradient released (utils/quant.py:1139-1148)."""
        if is_q:
            if sr_mode:
                scales, zeros, shape = _flat_qparam(p.qparam)
                p.data = ops.requant_sr(p.data, scales, zeros, direction.view(shape), step_size, shape,
                                        seed=self.sr_seed, offset=self.sr_offset)
                self.sr_offset += (p.numel() + 7) // 8
            elif p.wbit == 8:
                p.data = Qfunc_8bit_res(pdata, p.residual, qscales=p.qparam)
            elif p.wbit == 4:
                p.data = Qfunc_4bit_g_res(pdata, p.residual, qparam=p.qparam)
        if isinstance(p.grad, GradientQTensor):
            p.grad.zero()
        else:
            p.grad = None
