"""Gated MLP with the gate / up products and the SiLU product in one launch.

Mirrors the reference's GPTQ-side ``QuantLlamaMLP`` / ``make_fused_mlp`` (PTQ/quant/fused_mlp.py:177-254)
for this package's ``QLinearA16W4`` layers (native code layout): ``forward`` is
``down_proj(silu(gate_proj(x)) * up_proj(x))`` with the first three operations done by
``lq_a16w4_gate_up_silu`` on fp32 accumulators, as the reference's Triton kernel does (:160-166).
The reference's fused MLP is inference only. Here a block whose layers are being trained (backward hooks
installed, or an input that needs a gradient) runs four launches forward and backward with the
tensor-library glue folded into the GEMM epilogues (``_FusedMLPTrain``), and hands the three weight
gradients to the layers' accumulators exactly as their own backward hooks would.
"""
from __future__ import annotations

import torch
import torch.nn as nn

from . import ops

# Up to 16 tokens the fused product is one GEMV pass over both matrices, from FUSED_MIN_TOKENS on the MFMA kernel.
# In between the two products go through the ordinary forward (GEMV chunks or the split reduction, whichever the
# library picks) and the SiLU product is formed on their bf16 results: the fused kernel's 128-row tiles would be
# mostly empty (on the 7B matrices it takes 51 us from 17 to 192 tokens, the composed path 44 us at 17 tokens, 54
# at 64, 84 at 192).
FUSED_MIN_TOKENS = 64


def _w4(layer):
    return (layer.weight.data, layer.scales, layer.zeros)


class _FusedMLPTrain(torch.autograd.Function):
    """down(silu(gate(x)) * up(x)) for layers in training. Forward: the gate / up launch also stores the two
    products (lq_a16w4_gate_up_silu_save), then the down projection. Backward: the down projection's dX with the
    backward of silu(g) * u as its epilogue (lq_a16w4_dx_silu_bwd), then the gate and the up dX summed in one
    launch (lq_a16w4_dx_pair); dW of the three layers as QLinearFunctionW4.backward forms them (utils/quant.py:141-142),
    delivered through dict_temp and backward_hook_fn (utils/quant.py:398-411) layer by layer."""

    @staticmethod
    def forward(ctx, x2, mlp):
        gate, up, down = mlp.gate_proj, mlp.up_proj, mlp.down_proj
        inter, K = mlp.intermediate_size, mlp.infeatures
        h, g, u = ops.a16w4_gate_up_silu(x2, _w4(gate), _w4(up), (inter, K), save=True)
        bias = None if down.bias is None else down.bias.detach().to(torch.bfloat16).contiguous()
        y = ops.a16w4_forward(h, *_w4(down), (mlp.outfeatures, inter), bias)
        ctx.save_for_backward(x2, g, u, h)
        ctx.mlp = mlp
        return y

    @staticmethod
    def backward(ctx, grad_output):
        from .quant import _pending_dw, backward_hook_fn, dict_temp
        x2, g, u, h = ctx.saved_tensors
        mlp = ctx.mlp
        gate, up, down = mlp.gate_proj, mlp.up_proj, mlp.down_proj
        inter, K = mlp.intermediate_size, mlp.infeatures
        dy = grad_output.to(torch.bfloat16).contiguous()
        dg, du = ops.a16w4_dx_silu_bwd(dy, *_w4(down), (mlp.outfeatures, inter), g, u)
        dx = None
        if ctx.needs_input_grad[0]:
            dx = ops.a16w4_dx_pair(dg, _w4(gate), du, _w4(up), (inter, K))
        for layer, dyl, xin in ((down, dy, h), (up, du, x2), (gate, dg, x2)):
            if layer.hook_handle is not None:
                dict_temp.append(_pending_dw(dyl, xin))
                backward_hook_fn(layer, None, None)
        return dx, None


class QuantLlamaMLP(nn.Module):
    """PTQ/quant/fused_mlp.py:177-218 on QLinearA16W4 layers: keeps the three projections as submodules (their
    buffers stay where checkpoints expect them) and fuses gate / up / SiLU in ``forward``."""

    def __init__(self, gate_proj, down_proj, up_proj):
        super().__init__()
        if tuple(gate_proj.wshape) != tuple(up_proj.wshape):
            raise ValueError("gate_proj and up_proj must have the same shape")
        if gate_proj.bias is not None or up_proj.bias is not None:
            raise ValueError("the fused gate / up product takes no bias")
        self.gate_proj, self.down_proj, self.up_proj = gate_proj, down_proj, up_proj
        self.intermediate_size, self.infeatures = int(gate_proj.wshape[0]), int(gate_proj.wshape[1])
        self.outfeatures = int(down_proj.wshape[0])

    def _training(self, x):
        return torch.is_grad_enabled() and (x.requires_grad or any(
            layer.hook_handle is not None for layer in (self.gate_proj, self.up_proj, self.down_proj)))

    def forward(self, x):
        if not self._training(x):
            return self.down_proj(self.fused_gate_up(x))
        x2 = x.reshape(-1, x.shape[-1])
        M, K = x2.shape
        if (x2.dtype == torch.bfloat16 and M > 0 and K % 256 == 0 and self.intermediate_size % 64 == 0
                and self.outfeatures % 64 == 0):
            y = _FusedMLPTrain.apply(x2.contiguous(), self)
            return y.reshape(x.shape[:-1] + (self.outfeatures,))
        # shapes the fused launches do not take: the layers' own forward, which autograd follows
        return self.down_proj(torch.nn.functional.silu(self.gate_proj(x)) * self.up_proj(x))

    def fused_gate_up(self, x):
        """silu(gate_proj(x)) * up_proj(x), shape x.shape[:-1] + (intermediate_size,). Inference only: the result
        carries no autograd history (forward() takes the training path where one is needed)."""
        if self._training(x):
            raise RuntimeError("fused_gate_up has no backward: call the module (forward) when training")
        out_shape = x.shape[:-1] + (self.intermediate_size,)
        x2 = x.reshape(-1, x.shape[-1])
        M, K = x2.shape
        if x2.dtype == torch.bfloat16 and (0 < M <= 16 or (M >= FUSED_MIN_TOKENS and K % 256 == 0)):
            if not x2.is_contiguous():
                x2 = x2.contiguous()
            h = ops.a16w4_gate_up_silu(x2, _w4(self.gate_proj), _w4(self.up_proj), (self.intermediate_size, K))
        else:
            h = torch.nn.functional.silu(self.gate_proj.forward_eval(x2)) * self.up_proj.forward_eval(x2)
        return h.reshape(out_shape)


def make_fused_mlp(m, parent_name=""):
    """Replace every gated MLP (a module with QLinearA16W4 children named gate_proj, up_proj and down_proj, e.g.
    transformers' LlamaMLP after the layer swap of main0.py:300-343) by a QuantLlamaMLP
    (PTQ/quant/fused_mlp.py:241-254)."""
    from .quant import QLinearA16W4
    kids = dict(m.named_children())
    if all(isinstance(kids.get(k), QLinearA16W4) for k in ("gate_proj", "up_proj", "down_proj")) and not isinstance(m, QuantLlamaMLP):
        return QuantLlamaMLP(m.gate_proj, m.down_proj, m.up_proj)
    for name, child in m.named_children():
        new = make_fused_mlp(child, parent_name=f"{parent_name}.{name}")
        if new is not child:
            setattr(m, name, new)
    return m
