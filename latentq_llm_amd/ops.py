"""Tensor-level wrappers over the C ABI: validate, allocate outputs with torch, pass raw pointers
and the current HIP stream. PyTorch is used for device memory and streams only."""
from __future__ import annotations

import torch

from . import _C

GROUP = 128


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _chk(t: torch.Tensor, dtype, name: str):
    if not t.is_cuda:
        raise _C.LatentQError(f"{name} must be a GPU tensor: the HIP kernels have no CPU fallback")
    if t.dtype != dtype:
        raise TypeError(f"{name}: expected {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")


def _codes_ok(codes: torch.Tensor, N: int, K: int):
    if codes.dtype not in (torch.int8, torch.uint8):
        raise TypeError(f"codes: expected int8/uint8 bytes, got {codes.dtype}")
    if not codes.is_cuda or not codes.is_contiguous():
        raise ValueError("codes must be a contiguous GPU tensor")
    if codes.numel() != N * K // 2:
        raise ValueError(f"codes has {codes.numel()} bytes, expected N*K/2 = {N * K // 2}")


def _qparam_ok(scales, zeros, N, K):
    _chk(scales, torch.bfloat16, "scales")
    _chk(zeros, torch.bfloat16, "zeros")
    n = N * K // GROUP
    if scales.numel() != n or zeros.numel() != n:
        raise ValueError(f"scales/zeros need {n} entries, got {scales.numel()}/{zeros.numel()}")


def requant_sr(codes, scales, zeros, grad, lr: float, shape, u=None, seed: int = 0, offset: int = 0, out=None):
    """New packed codes after one stochastic-rounding latent update (see include/latentq.h, lq_requant_sr)."""
    N, K = shape
    _codes_ok(codes, N, K)
    _qparam_ok(scales, zeros, N, K)
    _chk(grad, torch.bfloat16, "grad")
    if grad.numel() != N * K:
        raise ValueError("grad must have N*K elements")
    if u is not None:
        _chk(u, torch.float32, "u")
        if u.numel() != N * K:
            raise ValueError("u must have N*K elements")
    if out is None:
        out = torch.empty_like(codes)
    else:
        _codes_ok(out, N, K)
    with torch.cuda.device(codes.device):
        _C.call("lq_requant_sr", codes.data_ptr(), out.data_ptr(), scales.data_ptr(), zeros.data_ptr(),
                grad.data_ptr(), float(lr), N, K, GROUP, None if u is None else u.data_ptr(),
                seed & (2**64 - 1), offset & (2**64 - 1), _stream(codes))
    return out


def philox_uniform(n: int, seed: int, offset: int = 0, device="cuda"):
    out = torch.empty(n, dtype=torch.float32, device=device)
    with torch.cuda.device(out.device):
        _C.call("lq_philox_uniform", out.data_ptr(), n, seed & (2**64 - 1), offset & (2**64 - 1), _stream(out))
    return out


# Scratch for the split-reduction GEMM of skinny problems (fp32 partial tiles); the library itself
# never allocates. Outside graph capture: one buffer of WORKSPACE_MAX_BYTES per (device, stream),
# allocated on first need and never resized, so its address is stable; at most WORKSPACE_MAX_STREAMS
# streams per device keep one (least recently used first out; a dropped buffer goes back to the
# caching allocator's pool of the stream it was allocated on, which orders its reuse after the
# kernels that still read it). Under graph capture: a buffer of the size the call needs from the
# capturing graph's own memory pool, which lives as long as the graph and is reused by later
# calls of the same capture.
_WORKSPACE = {}
WORKSPACE_MAX_BYTES = 64 << 20
WORKSPACE_MAX_STREAMS = 8


def _workspace(t, rows, cols):
    """(tensor, pointer, bytes) of a scratch buffer for a rows x cols fp32 result cut into up to 8
    slices, or (None, None, 0) when the problem is not one the split reduction is meant for (more than
    2048 rows). The caller keeps the tensor referenced until its launch is enqueued."""
    if rows > 2048:
        return None, None, 0
    if torch.cuda.is_current_stream_capturing():
        buf = torch.empty(min(8 * rows * cols * 4, WORKSPACE_MAX_BYTES), dtype=torch.uint8, device=t.device)
        return buf, buf.data_ptr(), buf.numel()
    key = (t.device.index, _stream(t))
    buf = _WORKSPACE.pop(key, None)
    if buf is None:
        buf = torch.empty(WORKSPACE_MAX_BYTES, dtype=torch.uint8, device=t.device)
        same_device = [k for k in _WORKSPACE if k[0] == key[0]]
        for k in same_device[: max(0, len(same_device) - (WORKSPACE_MAX_STREAMS - 1))]:
            del _WORKSPACE[k]
    _WORKSPACE[key] = buf  # (re)inserted last: dict order is the recency order
    return buf, buf.data_ptr(), buf.numel()


def a16w4_forward(x, codes, scales, zeros, shape, bias=None, out=None):
    """Y[M,N] = X[M,K] . deq(W)[N,K]^T (+ bias) in bf16 with fp32 accumulation."""
    N, K = shape
    _chk(x, torch.bfloat16, "x")
    if x.dim() != 2 or x.shape[1] != K:
        raise ValueError(f"x must be [M,{K}], got {tuple(x.shape)}")
    _codes_ok(codes, N, K)
    _qparam_ok(scales, zeros, N, K)
    if bias is not None:
        _chk(bias, torch.bfloat16, "bias")
        if bias.numel() != N:
            raise ValueError("bias must have N elements")
    M = x.shape[0]
    if out is None:
        y = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    else:
        _chk(out, torch.bfloat16, "out")
        if tuple(out.shape) != (M, N):
            raise ValueError(f"out must be [{M},{N}]")
        y = out
    if M == 0:
        return y
    with torch.cuda.device(x.device):
        keep, ws, ws_bytes = _workspace(x, M, N) if M > 16 else (None, None, 0)
        _C.call("lq_a16w4_fwd_ws", x.data_ptr(), codes.data_ptr(), scales.data_ptr(), zeros.data_ptr(),
                None if bias is None else bias.data_ptr(), y.data_ptr(), M, N, K, GROUP, ws, ws_bytes, _stream(x))
        del keep
    return y


STATIC_SCRATCH_BYTES = 32 << 20


def a16w4_forward_static(x, codes, scales, zeros, shape, out, bias=None):
    """a16w4_forward through the entry point that allocates nothing (lq_a16w4_fwd_static): the split
    reduction of skinny problems uses the library's static scratch array, and ``out`` is mandatory.
    Raises LatentQError when M > 16 and 8*M*N exceeds STATIC_SCRATCH_BYTES."""
    N, K = shape
    _chk(x, torch.bfloat16, "x")
    if x.dim() != 2 or x.shape[1] != K:
        raise ValueError(f"x must be [M,{K}], got {tuple(x.shape)}")
    _codes_ok(codes, N, K)
    _qparam_ok(scales, zeros, N, K)
    _chk(out, torch.bfloat16, "out")
    M = x.shape[0]
    if tuple(out.shape) != (M, N):
        raise ValueError(f"out must be [{M},{N}]")
    if bias is not None:
        _chk(bias, torch.bfloat16, "bias")
        if bias.numel() != N:
            raise ValueError("bias must have N elements")
    if M:
        with torch.cuda.device(x.device):
            _C.call("lq_a16w4_fwd_static", x.data_ptr(), codes.data_ptr(), scales.data_ptr(), zeros.data_ptr(),
                    None if bias is None else bias.data_ptr(), out.data_ptr(), M, N, K, GROUP, _stream(x))
    return out


def a16w4_gate_up_silu(x, gate, up, shape, out=None, save=False):
    """h[M,N] = silu(X . deq(Wgate)^T) * (X . deq(Wup)^T) in one launch (lq_a16w4_gate_up_silu); gate and up are
    (codes, scales, zeros) triples of two [N, K] matrices. Needs K % 256 == 0 above 16 tokens.
    save=True (lq_a16w4_gate_up_silu_save) also stores the two products and returns (h, g, u)."""
    N, K = shape
    _chk(x, torch.bfloat16, "x")
    if x.dim() != 2 or x.shape[1] != K:
        raise ValueError(f"x must be [M,{K}], got {tuple(x.shape)}")
    for w in (gate, up):
        _codes_ok(w[0], N, K)
        _qparam_ok(w[1], w[2], N, K)
    M = x.shape[0]
    if out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    else:
        _chk(out, torch.bfloat16, "out")
        if tuple(out.shape) != (M, N):
            raise ValueError(f"out must be [{M},{N}]")
    g = torch.empty_like(out) if save else None
    u = torch.empty_like(out) if save else None
    if M:
        with torch.cuda.device(x.device):
            if save:
                _C.call("lq_a16w4_gate_up_silu_save", x.data_ptr(), gate[0].data_ptr(), gate[1].data_ptr(), gate[2].data_ptr(),
                        up[0].data_ptr(), up[1].data_ptr(), up[2].data_ptr(), out.data_ptr(), g.data_ptr(), u.data_ptr(),
                        M, N, K, GROUP, _stream(x))
            else:
                _C.call("lq_a16w4_gate_up_silu", x.data_ptr(), gate[0].data_ptr(), gate[1].data_ptr(), gate[2].data_ptr(),
                        up[0].data_ptr(), up[1].data_ptr(), up[2].data_ptr(), out.data_ptr(), M, N, K, GROUP, _stream(x))
    return (out, g, u) if save else out


def a16w4_dx_silu_bwd(dy, codes, scales, zeros, shape, g, u):
    """The backward of a gated MLP's down projection with the backward of h = silu(g) * u as its epilogue
    (lq_a16w4_dx_silu_bwd): returns (dg, du), bf16 [M, K] each, for dy [M, N] and the saved products g, u [M, K]."""
    N, K = shape
    _chk(dy, torch.bfloat16, "dy")
    if dy.dim() != 2 or dy.shape[1] != N:
        raise ValueError(f"dy must be [M,{N}], got {tuple(dy.shape)}")
    _codes_ok(codes, N, K)
    _qparam_ok(scales, zeros, N, K)
    M = dy.shape[0]
    for t, name in ((g, "g"), (u, "u")):
        _chk(t, torch.bfloat16, name)
        if tuple(t.shape) != (M, K):
            raise ValueError(f"{name} must be [{M},{K}]")
    dg = torch.empty((M, K), dtype=torch.bfloat16, device=dy.device)
    du = torch.empty((M, K), dtype=torch.bfloat16, device=dy.device)
    if M:
        with torch.cuda.device(dy.device):
            _C.call("lq_a16w4_dx_silu_bwd", dy.data_ptr(), codes.data_ptr(), scales.data_ptr(), zeros.data_ptr(), g.data_ptr(),
                    u.data_ptr(), dg.data_ptr(), du.data_ptr(), M, N, K, GROUP, _stream(dy))
    return dg, du


def a16w4_dx(dy, codes, scales, zeros, shape, out=None, accumulate=False):
    """dX[M,K] = dY[M,N] . deq(W)[N,K]; accumulate=True: out = bf16(out + bf16(dY . deq(W))) (lq_a16w4_dx_acc)."""
    N, K = shape
    _chk(dy, torch.bfloat16, "dy")
    if dy.dim() != 2 or dy.shape[1] != N:
        raise ValueError(f"dy must be [M,{N}], got {tuple(dy.shape)}")
    _codes_ok(codes, N, K)
    _qparam_ok(scales, zeros, N, K)
    M = dy.shape[0]
    if out is None:
        dx = torch.empty((M, K), dtype=torch.bfloat16, device=dy.device)
    else:
        _chk(out, torch.bfloat16, "out")
        if tuple(out.shape) != (M, K):
            raise ValueError(f"out must be [{M},{K}]")
        dx = out
    if M == 0:
        return dx
    if accumulate:
        if out is None:
            raise ValueError("accumulate=True needs out")
        with torch.cuda.device(dy.device):
            _C.call("lq_a16w4_dx_acc", dy.data_ptr(), codes.data_ptr(), scales.data_ptr(), zeros.data_ptr(), dx.data_ptr(),
                    M, N, K, GROUP, _stream(dy))
        return dx
    with torch.cuda.device(dy.device):
        keep, ws, ws_bytes = _workspace(dy, M, K)
        _C.call("lq_a16w4_dx_ws", dy.data_ptr(), codes.data_ptr(), scales.data_ptr(), zeros.data_ptr(), dx.data_ptr(),
                M, N, K, GROUP, ws, ws_bytes, _stream(dy))
        del keep
    return dx


def a16w4_dx_pair(dy1, w1, dy2, w2, shape, out=None):
    """dX[M,K] = bf16(dY1 . deq(W1) + dY2 . deq(W2)) in one launch (lq_a16w4_dx_pair); w1, w2 = (codes, scales, zeros)
    of two [N, K] matrices."""
    N, K = shape
    for name, dy, w in (("dy1", dy1, w1), ("dy2", dy2, w2)):
        _chk(dy, torch.bfloat16, name)
        if dy.dim() != 2 or dy.shape[1] != N:
            raise ValueError(f"{name} must be [M,{N}], got {tuple(dy.shape)}")
        _codes_ok(w[0], N, K)
        _qparam_ok(w[1], w[2], N, K)
    if dy1.shape != dy2.shape:
        raise ValueError("dy1 and dy2 must have the same shape")
    M = dy1.shape[0]
    if out is None:
        out = torch.empty((M, K), dtype=torch.bfloat16, device=dy1.device)
    else:
        _chk(out, torch.bfloat16, "out")
        if tuple(out.shape) != (M, K):
            raise ValueError(f"out must be [{M},{K}]")
    if M == 0:
        return out
    with torch.cuda.device(dy1.device):
        _C.call("lq_a16w4_dx_pair", dy1.data_ptr(), w1[0].data_ptr(), w1[1].data_ptr(), w1[2].data_ptr(), dy2.data_ptr(),
                w2[0].data_ptr(), w2[1].data_ptr(), w2[2].data_ptr(), out.data_ptr(), M, N, K, GROUP, _stream(dy1))
    return out


PLAN_KERNELS = {0: "gemv", 1: "gemv_chunks", 2: "direct_128x256", 3: "staged_128x128", 4: "staged_256x128",
                5: "direct_128x128"}


def a16w4_plan(M: int, shape, backward: bool = False, workspace_bytes: int = WORKSPACE_MAX_BYTES, compute_units: int = 0):
    """(kernel name, splits, steps per slice) the forward / dX entry points would use for M tokens on an
    [N, K] matrix; compute_units = 0 asks the current device. Launches nothing (works without a GPU when
    compute_units is given)."""
    import ctypes
    N, K = shape
    k, sp, per = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    _C.call("lq_a16w4_plan", int(bool(backward)), M, N, K, workspace_bytes, compute_units, ctypes.addressof(k),
            ctypes.addressof(sp), ctypes.addressof(per))
    return PLAN_KERNELS[k.value], sp.value, per.value


def a16w4_dequant(codes, scales, zeros, shape):
    N, K = shape
    _codes_ok(codes, N, K)
    _qparam_ok(scales, zeros, N, K)
    w = torch.empty((N, K), dtype=torch.bfloat16, device=codes.device)
    with torch.cuda.device(codes.device):
        _C.call("lq_a16w4_dequant", codes.data_ptr(), scales.data_ptr(), zeros.data_ptr(), w.data_ptr(), N, K, GROUP,
                _stream(codes))
    return w


def w8_requant(latent, qscales):
    """int8 codes of a bf16 latent weight [N, K] with one bf16 scale per row (lq_w8_requant)."""
    _chk(latent, torch.bfloat16, "latent")
    _chk(qscales, torch.bfloat16, "qscales")
    if latent.dim() != 2 or qscales.numel() != latent.shape[0]:
        raise ValueError("latent must be [N, K] and qscales hold N entries")
    N, K = latent.shape
    out = torch.empty((N, K), dtype=torch.int8, device=latent.device)
    with torch.cuda.device(latent.device):
        _C.call("lq_w8_requant", latent.data_ptr(), qscales.data_ptr(), out.data_ptr(), N, K, _stream(latent))
    return out


def a8w8_forward(x8, w8, sx, sw, bias=None, want_acc: bool = False):
    """bf16 Y = ((int32 X8.W8^T) * sx[m]) * sw[n] (+ bias); optionally also the int32 accumulators.
    sw is fp32 [N], or the bf16 per-channel scales as the modules store them (lq_a8w8_fwd_qs)."""
    _chk(x8, torch.int8, "x8")
    _chk(w8, torch.int8, "w8")
    _chk(sx, torch.float32, "sx")
    if sw.dtype not in (torch.float32, torch.bfloat16):
        raise TypeError(f"sw: expected float32 or bfloat16, got {sw.dtype}")
    _chk(sw, sw.dtype, "sw")
    M, K = x8.shape
    N, K2 = w8.shape
    if K != K2:
        raise ValueError("x8 and w8 disagree on K")
    if sx.numel() != M or sw.numel() != N:
        raise ValueError("sx must have M entries and sw N entries")
    if bias is not None:
        _chk(bias, torch.bfloat16, "bias")
        if bias.numel() != N:
            raise ValueError("bias must have N elements")
    y = torch.empty((M, N), dtype=torch.bfloat16, device=x8.device)
    acc = torch.empty((M, N), dtype=torch.int32, device=x8.device) if want_acc else None
    if M > 0:
        with torch.cuda.device(x8.device):
            _C.call("lq_a8w8_fwd" if sw.dtype == torch.float32 else "lq_a8w8_fwd_qs", x8.data_ptr(), w8.data_ptr(),
                    sx.data_ptr(), sw.data_ptr(), None if bias is None else bias.data_ptr(), y.data_ptr(),
                    None if acc is None else acc.data_ptr(), M, N, K, _stream(x8))
    return (y, acc) if want_acc else y


def a8w8_dx_ok(dy, w8, qscales):
    """Whether a8w8_dx takes these operands (the layers fall back to the dense product otherwise)."""
    return (dy.is_cuda and dy.dtype == torch.bfloat16 and dy.dim() == 2 and dy.is_contiguous() and w8.is_cuda
            and w8.dtype == torch.int8 and w8.dim() == 2 and w8.is_contiguous() and qscales.is_cuda
            and qscales.dtype == torch.bfloat16 and qscales.is_contiguous() and qscales.numel() == w8.shape[0]
            and dy.shape[1] == w8.shape[0] and w8.shape[0] % 64 == 0 and w8.shape[1] % 128 == 0 and dy.shape[0] > 0
            and dy.data_ptr() % 16 == 0 and w8.data_ptr() % 16 == 0)


def a8w8_dx(dy, w8, qscales):
    """dX[M,K] = dY[M,N] . bf16(W8 * qscales)[N,K] from the int8 codes (lq_a8w8_dx)."""
    if not a8w8_dx_ok(dy, w8, qscales):
        raise ValueError("a8w8_dx needs contiguous GPU operands: dy bf16 [M,N], w8 int8 [N,K], qscales bf16 [N], N % 64 == 0, K % 128 == 0")
    M, N = dy.shape
    K = w8.shape[1]
    dx = torch.empty((M, K), dtype=torch.bfloat16, device=dy.device)
    with torch.cuda.device(dy.device):
        _C.call("lq_a8w8_dx", dy.data_ptr(), w8.data_ptr(), qscales.data_ptr(), dx.data_ptr(), M, N, K, _stream(dy))
    return dx


def act_quant_i8(x, clampv):
    """int8 activations clamp(rne(x*127/clampv)); clampv is a 1-element fp32 GPU tensor (no host sync)."""
    _chk(x, torch.bfloat16, "x")
    _chk(clampv, torch.float32, "clampv")
    out = torch.empty(x.shape, dtype=torch.int8, device=x.device)
    if x.numel():
        with torch.cuda.device(x.device):
            _C.call("lq_act_quant_i8", x.data_ptr(), clampv.data_ptr(), out.data_ptr(), x.numel(), _stream(x))
    return out


ACT_WORK_FLOATS = 1032


def act_quant_i8_dynamic(x, alpha_bf16: bool = False):
    """The dynamic layers' activation quantiser with clampv = x.max() found on the device
    (lq_act_quant_i8_dynamic): returns (x8 int8 [M,K], sx fp32 [M] filled with alpha = clampv/127, work) where
    work[0:1] is the clamp value and work[1:2] alpha, both fp32 device tensors. x: bf16 [M, K], M*K > 0."""
    _chk(x, torch.bfloat16, "x")
    if x.dim() != 2 or x.numel() == 0:
        raise ValueError("x must be a non-empty [M, K] matrix")
    M, K = x.shape
    x8 = torch.empty((M, K), dtype=torch.int8, device=x.device)
    sx = torch.empty(M, dtype=torch.float32, device=x.device)
    work = torch.empty(ACT_WORK_FLOATS, dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        _C.call("lq_act_quant_i8_dynamic", x.data_ptr(), x8.data_ptr(), sx.data_ptr(), work.data_ptr(), M, K,
                int(bool(alpha_bf16)), _stream(x))
    return x8, sx, work


def act_quant_i8_per_token(x):
    """Per-token activation quantiser (lq_act_quant_i8_per_token): (x8 int8 [M,K], sx fp32 [M] = rowmax|x| / 127)."""
    _chk(x, torch.bfloat16, "x")
    if x.dim() != 2 or x.numel() == 0 or x.shape[1] % 8:
        raise ValueError("x must be a non-empty [M, K] matrix with K a multiple of 8")
    M, K = x.shape
    x8 = torch.empty((M, K), dtype=torch.int8, device=x.device)
    sx = torch.empty(M, dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        _C.call("lq_act_quant_i8_per_token", x.data_ptr(), x8.data_ptr(), sx.data_ptr(), M, K, _stream(x))
    return x8, sx


def act_fake_quant(x, s):
    """bf16(clamp(round(bf16(x * s)), -128, 127) / s) (lq_act_fake_quant): x bf16 of any shape, s one bf16 number on
    the device; the values of ``(x * s).round_().clamp_(-128, 127).div_(s)``."""
    _chk(x, torch.bfloat16, "x")
    _chk(s, torch.bfloat16, "s")
    if s.numel() != 1:
        raise ValueError("s must hold one element")
    out = torch.empty_like(x)
    if x.numel():
        with torch.cuda.device(x.device):
            _C.call("lq_act_fake_quant", x.data_ptr(), s.data_ptr(), out.data_ptr(), x.numel(), _stream(x))
    return out


def act_dequant_ok(x8, scale, per_token: bool) -> bool:
    """Whether act_dequant_i8 takes these operands."""
    return (x8.is_cuda and x8.dtype == torch.int8 and x8.dim() == 2 and x8.is_contiguous() and x8.numel() > 0
            and x8.shape[1] % 16 == 0 and x8.data_ptr() % 16 == 0 and torch.is_tensor(scale) and scale.is_cuda
            and scale.dtype == torch.float32 and scale.is_contiguous()
            and scale.numel() == (x8.shape[0] if per_token else 1))


def act_dequant_i8(x8, scale, per_token: bool):
    """bf16(x8 * bf16(scale)) (lq_act_dequant_i8): scale fp32 [M] (per token) or one element; the values of
    ``x8.to(torch.bfloat16) * scale.to(torch.bfloat16)``."""
    _chk(x8, torch.int8, "x8")
    _chk(scale, torch.float32, "scale")
    if x8.dim() != 2 or x8.numel() == 0 or x8.shape[1] % 16:
        raise ValueError("x8 must be a non-empty [M, K] matrix with K a multiple of 16")
    M, K = x8.shape
    if scale.numel() != (M if per_token else 1):
        raise ValueError("scale must hold one value per row (per token) or one value")
    out = torch.empty((M, K), dtype=torch.bfloat16, device=x8.device)
    with torch.cuda.device(x8.device):
        _C.call("lq_act_dequant_i8", x8.data_ptr(), scale.data_ptr(), 1 if per_token else 0, out.data_ptr(), M, K, _stream(x8))
    return out


def adam8_update(grad, state1, state2, scale1, max1, scale2, max2, beta1, beta2, eps, step_size, param=None,
                 direction=None):
    """One Adam step on uint8 block-wise moments (all updated in place). Either ``param`` (bf16, updated in
    place: param -= step_size * m / d) or ``direction`` (bf16, receives m / d) is given."""
    _chk(grad, torch.bfloat16, "grad")
    n = grad.numel()
    for t, name in ((state1, "state1"), (state2, "state2")):
        _chk(t, torch.uint8, name)
        if t.numel() != n:
            raise ValueError(f"{name} must hold as many elements as grad")
    nblk = scale1.numel()
    if nblk == 0 or n % nblk:
        raise ValueError("the number of blocks must divide the number of elements")
    for t, name in ((scale1, "scale1"), (max1, "max1"), (scale2, "scale2"), (max2, "max2")):
        _chk(t, torch.float32, name)
        if t.numel() != nblk:
            raise ValueError(f"{name} must hold one value per block")
    if (param is None) == (direction is None):
        raise ValueError("give exactly one of param and direction")
    out = param if param is not None else direction
    _chk(out, torch.bfloat16, "param" if param is not None else "direction")
    if out.numel() != n:
        raise ValueError("param / direction must hold as many elements as grad")
    with torch.cuda.device(grad.device):
        _C.call("lq_adam8_update", grad.data_ptr(), param.data_ptr() if param is not None else None,
                direction.data_ptr() if direction is not None else None, state1.data_ptr(), state2.data_ptr(),
                scale1.data_ptr(), max1.data_ptr(), scale2.data_ptr(), max2.data_ptr(), n, n // nblk,
                float(beta1), float(beta2), float(eps), float(step_size), _stream(grad))
    return out


def adam8_latent_w4_step(grad, codes, residual_int, scales, zeros, shape, state1, state2, scale1, max1, scale2, max2,
                         dequant_curve, quant_curve, beta1, beta2, eps, step_size):
    """The Adam step of an lbit = 4 layer in one pass: codes (packed, N*K/2 bytes), residual_int
    (int32[N*K/8]) and the uint8 moments with their block parameters are all updated in place.
    The curves are (k1, b1, k2, b2, k3) tuples: the one the residual was stored with and the
    current one."""
    N, K = shape
    _chk(grad, torch.bfloat16, "grad")
    if grad.numel() != N * K:
        raise ValueError("grad must hold N*K elements")
    _codes_ok(codes, N, K)
    _qparam_ok(scales, zeros, N, K)
    _chk(residual_int, torch.int32, "residual_int")
    if residual_int.numel() != N * K // 8:
        raise ValueError("residual_int must hold N*K/8 words")
    n = N * K
    for t, name in ((state1, "state1"), (state2, "state2")):
        _chk(t, torch.uint8, name)
        if t.numel() != n:
            raise ValueError(f"{name} must hold N*K elements")
    nblk = scale1.numel()
    if nblk == 0 or n % nblk:
        raise ValueError("the number of blocks must divide the number of elements")
    for t, name in ((scale1, "scale1"), (max1, "max1"), (scale2, "scale2"), (max2, "max2")):
        _chk(t, torch.float32, name)
        if t.numel() != nblk:
            raise ValueError(f"{name} must hold one value per block")
    d, q = dequant_curve, quant_curve
    with torch.cuda.device(grad.device):
        _C.call("lq_adam8_latent_w4_step", grad.data_ptr(), codes.data_ptr(), residual_int.data_ptr(), scales.data_ptr(),
                zeros.data_ptr(), state1.data_ptr(), state2.data_ptr(), scale1.data_ptr(), max1.data_ptr(),
                scale2.data_ptr(), max2.data_ptr(), N, K, 128, n // nblk,
                int(d[0]), float(d[1]), int(d[2]), float(d[3]), int(d[4]),
                int(q[0]), float(q[1]), int(q[2]), float(q[3]), int(q[4]),
                float(beta1), float(beta2), float(eps), float(step_size), _stream(grad))
    return codes


def adam8_latent_w8_step(grad, codes, residual_int, qscales, state1, state2, scale1, max1, scale2, max2,
                         dequant_curve, quant_curve, beta1, beta2, eps, step_size):
    """The Adam step of an 8-bit-weight layer in lbit = 4 mode in one pass: codes (int8 [N, K]), residual_int
    (int32[N*K/8]) and the uint8 moments with their block parameters are all updated in place; qscales bf16 [N].
    The curves are (k1, b1, k2, b2, k3) tuples: the one the residual was stored with and the current one."""
    _chk(grad, torch.bfloat16, "grad")
    _chk(codes, torch.int8, "codes")
    if codes.dim() != 2 or codes.shape[1] % 8:
        raise ValueError("codes must be int8 [N, K] with K a multiple of 8")
    N, K = codes.shape
    n = N * K
    if grad.numel() != n:
        raise ValueError("grad must hold N*K elements")
    _chk(qscales, torch.bfloat16, "qscales")
    if qscales.numel() != N:
        raise ValueError("qscales must hold one value per row")
    _chk(residual_int, torch.int32, "residual_int")
    if residual_int.numel() != n // 8:
        raise ValueError("residual_int must hold N*K/8 words")
    for t, name in ((state1, "state1"), (state2, "state2")):
        _chk(t, torch.uint8, name)
        if t.numel() != n:
            raise ValueError(f"{name} must hold N*K elements")
    nblk = scale1.numel()
    if nblk == 0 or n % nblk:
        raise ValueError("the number of blocks must divide the number of elements")
    for t, name in ((scale1, "scale1"), (max1, "max1"), (scale2, "scale2"), (max2, "max2")):
        _chk(t, torch.float32, name)
        if t.numel() != nblk:
            raise ValueError(f"{name} must hold one value per block")
    d, q = dequant_curve, quant_curve
    with torch.cuda.device(grad.device):
        _C.call("lq_adam8_latent_w8_step", grad.data_ptr(), codes.data_ptr(), residual_int.data_ptr(), qscales.data_ptr(),
                state1.data_ptr(), state2.data_ptr(), scale1.data_ptr(), max1.data_ptr(), scale2.data_ptr(),
                max2.data_ptr(), N, K, n // nblk,
                int(d[0]), float(d[1]), int(d[2]), float(d[3]), int(d[4]),
                int(q[0]), float(q[1]), int(q[2]), float(q[3]), int(q[4]),
                float(beta1), float(beta2), float(eps), float(step_size), _stream(grad))
    return codes


def gradq8_quant(dw, q, scale, accumulate: bool, noise=None, seed: int = 0, offset: int = 0):
    """The 8-bit gradient accumulator in one pass (lq_gradq8_quant): dw bf16 [N, K]; q int8 [N, K] and
    scale bf16 [N, 1] are updated in place (scale only when ``accumulate`` is False). ``noise`` is an
    optional bf16 [N, K] tensor of rounding noise; without it the Philox stream (seed, offset) is used."""
    _chk(dw, torch.bfloat16, "dw")
    _chk(q, torch.int8, "q")
    _chk(scale, torch.bfloat16, "scale")
    if dw.dim() != 2 or tuple(q.shape) != tuple(dw.shape) or scale.numel() != dw.shape[0]:
        raise ValueError("dw and q must be [N, K] and scale must hold N entries")
    if noise is not None:
        _chk(noise, torch.bfloat16, "noise")
        if tuple(noise.shape) != tuple(dw.shape):
            raise ValueError("noise must have the shape of dw")
    N, K = dw.shape
    if N and K:
        with torch.cuda.device(dw.device):
            _C.call("lq_gradq8_quant", dw.data_ptr(), q.data_ptr(), scale.data_ptr(), int(bool(accumulate)), N, K,
                    None if noise is None else noise.data_ptr(), seed & (2**64 - 1), offset & (2**64 - 1), _stream(dw))
    return q


def transpose_bf16(x):
    """Contiguous transpose of a 2-D bf16 matrix whose sides are multiples of 8."""
    _chk(x, torch.bfloat16, "x")
    if x.dim() != 2 or x.shape[0] % 8 or x.shape[1] % 8:
        raise ValueError("x must be 2-D with both sides multiples of 8")
    R, C = x.shape
    out = torch.empty((C, R), dtype=torch.bfloat16, device=x.device)
    with torch.cuda.device(x.device):
        _C.call("lq_transpose_bf16", x.data_ptr(), out.data_ptr(), R, C, _stream(x))
    return out


def _weight_grad_native_ok(dy, x, k_mult=8):
    return (dy.is_cuda and x.is_cuda and dy.dtype == torch.bfloat16 and x.dtype == torch.bfloat16 and dy.dim() == 2
            and x.dim() == 2 and dy.is_contiguous() and x.is_contiguous() and dy.shape[0] == x.shape[0]
            and dy.shape[0] > 0 and dy.shape[0] % 64 == 0 and dy.shape[1] % 8 == 0 and x.shape[1] % k_mult == 0
            and dy.data_ptr() % 16 == 0 and x.data_ptr() % 16 == 0)


def weight_grad(dy, x):
    """dW = dY^T X for 2-D operands: the library's own GEMM (lq_weight_grad: both operands read as they lie in
    memory) for bf16 GPU operands with a multiple of 64 tokens, the tensor library's product otherwise."""
    if _weight_grad_native_ok(dy, x):
        N, K = dy.shape[1], x.shape[1]
        dw = torch.empty((N, K), dtype=torch.bfloat16, device=dy.device)
        with torch.cuda.device(dy.device):
            _C.call("lq_weight_grad", dy.data_ptr(), x.data_ptr(), dw.data_ptr(), dy.shape[0], N, K, _stream(dy))
        return dw
    if (dy.is_cuda and dy.dtype == torch.bfloat16 and x.dtype == torch.bfloat16 and dy.dim() == 2 and dy.is_contiguous()
            and dy.shape[0] % 8 == 0 and dy.shape[1] % 8 == 0 and dy.shape[0] >= 256):
        return transpose_bf16(dy).mm(x)
    return dy.t().mm(x)


def weight_grad_acc_ok(dy, x, g) -> bool:
    """Whether weight_grad_acc can add dY^T X onto the gradient tensor g in place."""
    return (_weight_grad_native_ok(dy, x) and torch.is_tensor(g) and g.is_cuda and g.device == dy.device
            and g.dtype == torch.bfloat16 and g.is_contiguous() and tuple(g.shape) == (dy.shape[1], x.shape[1])
            and g.data_ptr() % 16 == 0)


def weight_grad_acc(dy, x, g):
    """g = bf16(g + bf16(dY^T X)) in place (lq_weight_grad_acc): the weight-gradient GEMM with the bf16 ``add_`` of the
    gradient accumulation as its epilogue; the same bits as ``g.add_(weight_grad(dy, x))``."""
    if not weight_grad_acc_ok(dy, x, g):
        raise ValueError("weight_grad_acc needs contiguous bf16 GPU operands, M % 64 == 0, N % 8 == 0, K % 8 == 0 and g [N, K]")
    N, K = dy.shape[1], x.shape[1]
    with torch.cuda.device(dy.device):
        _C.call("lq_weight_grad_acc", dy.data_ptr(), x.data_ptr(), g.data_ptr(), dy.shape[0], N, K, _stream(dy))
    return g


def weight_grad_acc8(dy, x, q, scale, noise=None, seed: int = 0, offset: int = 0):
    """q = quant(dequant(q) + dY^T X) in place (lq_weight_grad_acc8): the weight-gradient GEMM with the add_ form of
    the 8-bit gradient accumulator as its epilogue. dy bf16 [M,N], x bf16 [M,K], q int8 [N,K], scale bf16 [N,1]."""
    if not _weight_grad_native_ok(dy, x, 16):
        raise ValueError("weight_grad_acc8 needs contiguous bf16 GPU operands, M % 64 == 0, N % 8 == 0, K % 16 == 0")
    N, K = dy.shape[1], x.shape[1]
    _chk(q, torch.int8, "q")
    _chk(scale, torch.bfloat16, "scale")
    if tuple(q.shape) != (N, K) or scale.numel() != N:
        raise ValueError("q must be [N, K] and scale hold N entries")
    if noise is not None:
        _chk(noise, torch.bfloat16, "noise")
        if tuple(noise.shape) != (N, K):
            raise ValueError("noise must be [N, K]")
    with torch.cuda.device(dy.device):
        _C.call("lq_weight_grad_acc8", dy.data_ptr(), x.data_ptr(), q.data_ptr(), scale.data_ptr(), dy.shape[0], N, K,
                None if noise is None else noise.data_ptr(), seed & (2**64 - 1), offset & (2**64 - 1), _stream(dy))
    return q


def repack_gptq_to_native(qweight, shape):
    N, K = shape
    _chk(qweight, torch.int32, "qweight")
    out = torch.empty(N * K // 2, dtype=torch.int8, device=qweight.device)
    with torch.cuda.device(qweight.device):
        _C.call("lq_repack_gptq_to_native", qweight.data_ptr(), out.data_ptr(), N, K, _stream(qweight))
    return out


def repack_native_to_gptq(codes, shape):
    N, K = shape
    _codes_ok(codes, N, K)
    out = torch.empty((K // 8, N), dtype=torch.int32, device=codes.device)
    with torch.cuda.device(codes.device):
        _C.call("lq_repack_native_to_gptq", codes.data_ptr(), out.data_ptr(), N, K, _stream(codes))
    return out


def residual_quant(x, q, mode: int, k1=0, b1=0.0, k2=0, b2=0.0, k3=0):
    """4-bit residual codec, quantise: writes the packed words into q (int32[n/8]) and overwrites the
    bf16 tensor x with the carry flags (1.0 / 0.0). mode 0 = three-segment companding, 1 = uniform."""
    _chk(x, torch.bfloat16, "x")
    _chk(q, torch.int32, "q")
    if x.numel() != 8 * q.numel():
        raise ValueError("x must have 8 elements per word of q")
    with torch.cuda.device(x.device):
        _C.call("lq_residual_quant", x.data_ptr(), q.data_ptr(), q.numel(), mode, k1, float(b1), k2, float(b2), k3,
                _stream(x))
    return x


_QUANT_S_DTYPES = {torch.float32: 0, torch.float16: 1, torch.float64: 2, torch.bfloat16: 3}


def residual_quant_s(x, q):
    """Deterministic uniform 4-bit quantiser (round(x * 8), no dither): packed words into q, carries over x."""
    if x.dtype not in _QUANT_S_DTYPES:
        raise TypeError(f"x must be float32, float16, float64 or bfloat16, got {x.dtype}")
    _chk(x, x.dtype, "x")
    _chk(q, torch.int32, "q")
    if x.numel() != 8 * q.numel():
        raise ValueError("x must have 8 elements per word of q")
    with torch.cuda.device(x.device):
        _C.call("lq_residual_quant_s", x.data_ptr(), q.data_ptr(), q.numel(), _QUANT_S_DTYPES[x.dtype], _stream(x))
    return x


def residual_dequant(q, mode: int, k1=0, b1=0.0, k2=0, b2=0.0, k3=0):
    """4-bit residual codec, dequantise: int32[n_words] -> bf16[n_words, 8]."""
    _chk(q, torch.int32, "q")
    x = torch.empty((q.numel(), 8), dtype=torch.bfloat16, device=q.device)
    with torch.cuda.device(q.device):
        _C.call("lq_residual_dequant", q.data_ptr(), x.data_ptr(), q.numel(), mode, k1, float(b1), k2, float(b2), k3,
                _stream(q))
    return x


def latent_w4_reconstruct(codes, scales, zeros, residual_int, shape, k1, b1, k2, b2, k3):
    """Latent weight of an A16W4 layer with a 4-bit residual: dequantised codes + dequantised residual * scale,
    with the bf16 rounding points of the reference's tensor-op chain. Returns bf16 [N, K]."""
    N, K = shape
    _codes_ok(codes, N, K)
    _qparam_ok(scales, zeros, N, K)
    _chk(residual_int, torch.int32, "residual_int")
    if residual_int.numel() != N * K // 8:
        raise ValueError("residual_int must hold N*K/8 words")
    out = torch.empty((N, K), dtype=torch.bfloat16, device=codes.device)
    with torch.cuda.device(codes.device):
        _C.call("lq_latent_w4_reconstruct", codes.data_ptr(), scales.data_ptr(), zeros.data_ptr(), residual_int.data_ptr(),
                out.data_ptr(), N, K, 128, int(k1), float(b1), int(k2), float(b2), int(k3), _stream(codes))
    return out


def latent_w4_requant(latent, scales, zeros, residual_int, shape, k1, b1, k2, b2, k3):
    """Re-quantise a bf16 latent weight: returns the packed codes and overwrites residual_int (int32[N*K/8])."""
    N, K = shape
    _chk(latent, torch.bfloat16, "latent")
    if latent.numel() != N * K:
        raise ValueError("latent must hold N*K elements")
    _qparam_ok(scales, zeros, N, K)
    _chk(residual_int, torch.int32, "residual_int")
    if residual_int.numel() != N * K // 8:
        raise ValueError("residual_int must hold N*K/8 words")
    codes = torch.empty(N * K // 2, dtype=torch.int8, device=latent.device)
    with torch.cuda.device(latent.device):
        _C.call("lq_latent_w4_requant", latent.data_ptr(), scales.data_ptr(), zeros.data_ptr(), codes.data_ptr(),
                residual_int.data_ptr(), N, K, 128, int(k1), float(b1), int(k2), float(b2), int(k3), _stream(latent))
    return codes


def latent_w8_reconstruct(codes, qscales, residual_int, k1, b1, k2, b2, k3):
    """Latent weight of an 8-bit-weight layer with a 4-bit residual (lq_latent_w8_reconstruct): bf16 [N, K] from the
    int8 codes [N, K], the bf16 row scales and the residual words."""
    _chk(codes, torch.int8, "codes")
    _chk(qscales, torch.bfloat16, "qscales")
    _chk(residual_int, torch.int32, "residual_int")
    if codes.dim() != 2 or qscales.numel() != codes.shape[0] or residual_int.numel() != codes.numel() // 8:
        raise ValueError("codes must be [N, K], qscales hold N entries and residual_int N*K/8 words")
    N, K = codes.shape
    out = torch.empty((N, K), dtype=torch.bfloat16, device=codes.device)
    with torch.cuda.device(codes.device):
        _C.call("lq_latent_w8_reconstruct", codes.data_ptr(), qscales.data_ptr(), residual_int.data_ptr(), out.data_ptr(), N, K,
                int(k1), float(b1), int(k2), float(b2), int(k3), _stream(codes))
    return out


def latent_w8_requant(latent, qscales, residual_int, k1, b1, k2, b2, k3):
    """Re-quantise the bf16 latent of an 8-bit-weight layer: returns the int8 codes and overwrites residual_int."""
    _chk(latent, torch.bfloat16, "latent")
    _chk(qscales, torch.bfloat16, "qscales")
    _chk(residual_int, torch.int32, "residual_int")
    if latent.dim() != 2 or qscales.numel() != latent.shape[0] or residual_int.numel() != latent.numel() // 8:
        raise ValueError("latent must be [N, K], qscales hold N entries and residual_int N*K/8 words")
    N, K = latent.shape
    codes = torch.empty((N, K), dtype=torch.int8, device=latent.device)
    with torch.cuda.device(latent.device):
        _C.call("lq_latent_w8_requant", latent.data_ptr(), qscales.data_ptr(), codes.data_ptr(), residual_int.data_ptr(), N, K,
                int(k1), float(b1), int(k2), float(b2), int(k3), _stream(latent))
    return codes
