"""Checkpoint formats on either side of the quantized-linear hot path.

The reference's fine-tuning script feeds its modules from three on-disk formats:

* the PTQ producer's *native* A16W4 format (``PTQ/quant/quant_linear.py:445-471``): flat int8
  codes, two per byte, high nibble first, ``[N, K]`` row-major; fp16 ``scales`` / ``zeros`` of
  shape ``[N*K/128, 1]``. ``main0.py:316-320`` hands these to ``QLinearA16W4`` unchanged (cast to
  bf16) -- see :func:`load_a16w4`.
* the GPTQ format (``PTQ/quant/quant_linear.py:343-389``): ``qweight`` int32 ``[K/8, N]`` with
  code ``(k, n)`` at bits ``4*(k%8)`` of word ``[k/8, n]``; ``qzeros`` int32 ``[G, N/8]`` holding
  ``zero - 1`` at bits ``4*(n%8)`` of word ``[g, n/8]``; ``scales`` fp16 ``[G, N]``; ``g_idx[k]`` =
  group of input feature ``k``. :func:`gptq_to_native` / :func:`native_to_gptq` convert between
  it and the native layout on the device (the code transposition is the HIP repack kernel).
* the A8W8 format (``main0.py:329-340``): ``qweight`` uint8 ``[N, K]`` with an offset of 128,
  per-channel ``scales``, ``inp_absmax`` for the activation clamp -- see :func:`load_a8w8`.

Nothing here runs on the hot path; it prepares the buffers the kernels stream.
"""
from __future__ import annotations

import torch

from . import ops

GROUP = 128


def unpack_gptq_zeros(qzeros: torch.Tensor, N: int) -> torch.Tensor:
    """int32 ``[G, N/8]`` -> integer zero points ``[G, N]`` (stored value + 1, the ``- 1`` of
    ``PTQ/quant/quant_linear.py:373`` undone as its dequantiser does at ``:339``)."""
    shifts = torch.arange(0, 32, 4, device=qzeros.device, dtype=torch.int32)
    z = (qzeros.unsqueeze(-1) >> shifts) & 0xF
    return z.reshape(qzeros.shape[0], -1)[:, :N] + 1


def pack_gptq_zeros(zeros_gn: torch.Tensor) -> torch.Tensor:
    """Integer zero points ``[G, N]`` (N a multiple of 8) -> int32 ``[G, N/8]`` holding ``zero - 1``."""
    G, N = zeros_gn.shape
    if N % 8:
        raise ValueError("N must be a multiple of 8")
    z = (zeros_gn.to(torch.int64) - 1) & 0xF
    shifts = torch.arange(0, 32, 4, device=zeros_gn.device, dtype=torch.int64)
    words = (z.reshape(G, N // 8, 8) << shifts).sum(-1)
    words = torch.where(words >= 2 ** 31, words - 2 ** 32, words)
    return words.to(torch.int32)


def _check_g_idx(g_idx, K: int, group: int):
    if g_idx is None:
        return
    want = torch.arange(K, device=g_idx.device) // group
    if not torch.equal(g_idx.to(want.dtype), want):
        raise ValueError("only the trivial g_idx (k // group, no activation reordering) maps onto the native layout")


@torch.no_grad()
def gptq_to_native(qweight, qzeros, scales, g_idx=None, group: int = GROUP):
    """GPTQ tensors of one linear layer -> ``(codes int8[N*K/2], scales bf16[N*G,1], zeros bf16[N*G,1], (N, K))``
    in the layout ``QLinearA16W4`` holds (groups of a row contiguous)."""
    if group != GROUP:
        raise ValueError(f"group size must be {GROUP}")
    K, N = qweight.shape[0] * 8, qweight.shape[1]
    G = K // group
    if K % group or scales.shape != (G, N) or qzeros.shape[0] != G:
        raise ValueError("shapes do not describe a group-128 GPTQ layer")
    _check_g_idx(g_idx, K, group)
    codes = ops.repack_gptq_to_native(qweight.contiguous(), (N, K))
    zeros = unpack_gptq_zeros(qzeros, N)
    s = scales.t().contiguous().to(torch.bfloat16).reshape(N * G, 1)
    z = zeros.t().contiguous().to(torch.bfloat16).reshape(N * G, 1)
    return codes, s, z, (N, K)


@torch.no_grad()
def native_to_gptq(codes, scales, zeros, shape, group: int = GROUP):
    """Inverse of :func:`gptq_to_native`: ``(qweight int32[K/8,N], qzeros int32[G,N/8], scales fp16[G,N], g_idx)``.
    Zero points must be integers in 1..16 (what the 4-bit ``zero - 1`` field can hold)."""
    if group != GROUP:
        raise ValueError(f"group size must be {GROUP}")
    N, K = shape
    G = K // group
    zi = zeros.reshape(N, G).float()
    if not torch.equal(zi, zi.round()) or zi.min() < 1 or zi.max() > 16:
        raise ValueError("GPTQ stores zero - 1 in 4 bits: zero points must be integers in 1..16")
    qweight = ops.repack_native_to_gptq(codes, (N, K))
    qzeros = pack_gptq_zeros(zi.t().contiguous().to(torch.int32))
    s = scales.reshape(N, G).t().contiguous().to(torch.float16)
    g_idx = (torch.arange(K, device=codes.device) // group).to(torch.int32)
    return qweight, qzeros, s, g_idx


@torch.no_grad()
def load_a16w4(layer, ckt: dict, prefix: str):
    """Fill a ``QLinearA16W4`` from the native-format checkpoint entries ``prefix + '.qweight' /
    '.scales' / '.zeros' / '.bias'`` exactly as ``main0.py:316-320, 341-342`` does."""
    layer.lname = prefix
    layer.zeros.data = ckt[prefix + ".zeros"].to(torch.bfloat16)
    layer.scales.data = ckt[prefix + ".scales"].to(torch.bfloat16)
    layer.weight.set_value(ckt[prefix + ".qweight"], [layer.scales, layer.zeros, layer.wshape])
    if layer.bias is not None and prefix + ".bias" in ckt:
        layer.bias.data = ckt[prefix + ".bias"].to(torch.bfloat16)
    return layer


@torch.no_grad()
def a8w8_weight_from_checkpoint(qweight_u8: torch.Tensor) -> torch.Tensor:
    """uint8 with offset 128 -> int8 (``main0.py:334``)."""
    return (qweight_u8.to(torch.int32) - 128).to(torch.int8)


@torch.no_grad()
def load_a8w8(layer, ckt: dict, prefix: str):
    """Fill a ``QLinearA8W8`` from ``prefix + '.qweight' (uint8) / '.scales' / '.inp_absmax' / '.bias'``
    as ``main0.py:329-342`` does for ``lbit != 4`` (the latent copy is the dequantised weight)."""
    layer.lname = prefix
    layer.clampv.data = ckt[prefix + ".inp_absmax"].max().reshape(layer.clampv.shape).to(layer.clampv.dtype)
    layer.qscales.data = ckt[prefix + ".scales"].to(torch.bfloat16).reshape(layer.qscales.shape)
    w8 = a8w8_weight_from_checkpoint(ckt[prefix + ".qweight"])
    layer.weight.set_value(w8, layer.qscales)
    residual = getattr(layer.weight, "residual", None)
    if isinstance(residual, torch.Tensor):
        layer.weight.residual.data = (w8.to(torch.int32) * layer.qscales).to(torch.bfloat16)
    if layer.bias is not None and prefix + ".bias" in ckt:
        layer.bias.data = ckt[prefix + ".bias"].to(torch.bfloat16)
    return layer
