"""ctypes front end to oracle/lq_oracle.c. bf16 data travels as numpy uint16 bit patterns."""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liblq_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE] + (["-B"] if force else []), check=True, capture_output=True)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.lqo_bf16_to_f32.restype = C.c_float
        _lib.lqo_bf16_to_f32.argtypes = [C.c_uint16]
        _lib.lqo_f32_to_bf16.restype = C.c_uint16
        _lib.lqo_f32_to_bf16.argtypes = [C.c_float]
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dtype):
    a = np.ascontiguousarray(a)
    assert a.dtype == dtype, (a.dtype, dtype)
    return a


def f32_to_bf16_bits(a: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even fp32 -> bf16 bit patterns (vectorised, same rule as the C helper)."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    r = np.where(nan, (u >> 16) | 0x40, r)
    return r.astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def pack(codes: np.ndarray) -> np.ndarray:
    codes = _c(codes.reshape(-1), np.uint8)
    out = np.empty(codes.size // 2, np.uint8)
    lib().lqo_pack(_p(codes), _p(out), C.c_int64(codes.size))
    return out


def unpack(packed: np.ndarray) -> np.ndarray:
    packed = _c(packed.reshape(-1).view(np.uint8), np.uint8)
    out = np.empty(packed.size * 2, np.uint8)
    lib().lqo_unpack(_p(packed), _p(out), C.c_int64(out.size))
    return out


def dequant(packed, scales, zeros, N, K, group=128) -> np.ndarray:
    packed = _c(packed.reshape(-1).view(np.uint8), np.uint8)
    scales = _c(scales.reshape(-1), np.uint16)
    zeros = _c(zeros.reshape(-1), np.uint16)
    out = np.empty((N, K), np.uint16)
    lib().lqo_dequant(_p(packed), _p(scales), _p(zeros), _p(out), C.c_int64(N), C.c_int64(K), C.c_int(group))
    return out


def a16w4_fwd(x, packed, scales, zeros, bias, M, N, K, group=128, want_f64=False):
    x = _c(x.reshape(-1), np.uint16)
    packed = _c(packed.reshape(-1).view(np.uint8), np.uint8)
    scales = _c(scales.reshape(-1), np.uint16)
    zeros = _c(zeros.reshape(-1), np.uint16)
    bias = None if bias is None else _c(bias.reshape(-1), np.uint16)
    y = np.empty((M, N), np.uint16)
    y64 = np.empty((M, N), np.float64) if want_f64 else None
    rc = lib().lqo_a16w4_fwd(_p(x), _p(packed), _p(scales), _p(zeros), _p(bias), _p(y), _p(y64), C.c_int64(M),
                             C.c_int64(N), C.c_int64(K), C.c_int(group))
    assert rc == 0
    return (y, y64) if want_f64 else y


def a16w4_dx(dy, packed, scales, zeros, M, N, K, group=128, want_f64=False):
    dy = _c(dy.reshape(-1), np.uint16)
    packed = _c(packed.reshape(-1).view(np.uint8), np.uint8)
    scales = _c(scales.reshape(-1), np.uint16)
    zeros = _c(zeros.reshape(-1), np.uint16)
    dx = np.empty((M, K), np.uint16)
    d64 = np.empty((M, K), np.float64) if want_f64 else None
    rc = lib().lqo_a16w4_dx(_p(dy), _p(packed), _p(scales), _p(zeros), _p(dx), _p(d64), C.c_int64(M), C.c_int64(N),
                            C.c_int64(K), C.c_int(group))
    assert rc == 0
    return (dx, d64) if want_f64 else dx


def philox4x32_10(ctr, key):
    ctr = np.asarray(ctr, np.uint32)
    key = np.asarray(key, np.uint32)
    out = np.empty(4, np.uint32)
    lib().lqo_philox4x32_10(_p(ctr), _p(key), _p(out))
    return out


def philox_uniform(n, seed, offset=0) -> np.ndarray:
    out = np.empty(n, np.float32)
    lib().lqo_philox_uniform(_p(out), C.c_int64(n), C.c_uint64(seed), C.c_uint64(offset))
    return out


def requant(packed, scales, zeros, grad, lr, N, K, group=128, u=None, seed=0, offset=0) -> np.ndarray:
    packed = _c(packed.reshape(-1).view(np.uint8), np.uint8)
    scales = _c(scales.reshape(-1), np.uint16)
    zeros = _c(zeros.reshape(-1), np.uint16)
    grad = _c(grad.reshape(-1), np.uint16)
    u = None if u is None else _c(u.reshape(-1), np.float32)
    out = np.empty_like(packed)
    lib().lqo_requant(_p(packed), _p(out), _p(scales), _p(zeros), _p(grad), C.c_float(lr), C.c_int64(N),
                      C.c_int64(K), C.c_int(group), _p(u), C.c_uint64(seed), C.c_uint64(offset))
    return out


def w8_requant(latent_bits, qscale_bits, N, K):
    lat = _c(latent_bits.reshape(-1), np.uint16)
    qs = _c(qscale_bits.reshape(-1), np.uint16)
    out = np.empty(N * K, np.int8)
    lib().lqo_w8_requant(_p(lat), _p(qs), _p(out), C.c_int64(N), C.c_int64(K))
    return out


def gradq8_noise(n, seed, offset=0):
    """The noise lqo_gradq8 draws for flat elements 0..n-1 when none is injected (float32)."""
    out = np.empty(n, np.float32)
    lib().lqo_gradq8_noise(_p(out), C.c_int64(n), C.c_uint64(seed), C.c_uint64(offset))
    return out


def gradq8(dw, q, scale, accumulate, N, K, noise=None, seed=0, offset=0):
    """GradientQTensor (bit = 8) set_value / add_: returns (new int8 q [N*K], bf16 scale bits [N]).
    dw, noise: bf16 bit patterns; q: int8 or None (set); scale: bf16 bits or None (set)."""
    dw = _c(dw.reshape(-1), np.uint16)
    qo = np.zeros(N * K, np.int8) if q is None else _c(q.reshape(-1), np.int8).copy()
    so = np.zeros(N, np.uint16) if scale is None else _c(scale.reshape(-1), np.uint16).copy()
    noise = None if noise is None else _c(noise.reshape(-1), np.uint16)
    lib().lqo_gradq8(_p(dw), _p(qo), _p(so), C.c_int(1 if accumulate else 0), C.c_int64(N), C.c_int64(K), _p(noise),
                     C.c_uint64(seed), C.c_uint64(offset))
    return qo, so


def a8w8(x, w, sx, sw, bias, M, N, K, want_y=True):
    x = _c(x.reshape(-1), np.int8)
    w = _c(w.reshape(-1), np.int8)
    sx = _c(sx.reshape(-1), np.float32)
    sw = _c(sw.reshape(-1), np.float32)
    bias = None if bias is None else _c(bias.reshape(-1), np.uint16)
    y = np.empty((M, N), np.uint16) if want_y else None
    acc = np.empty((M, N), np.int32)
    lib().lqo_a8w8(_p(x), _p(w), _p(sx), _p(sw), _p(bias), _p(y), _p(acc), C.c_int64(M), C.c_int64(N), C.c_int64(K))
    return y, acc


def act_quant_i8(x, clampv: float) -> np.ndarray:
    x = _c(x.reshape(-1), np.uint16)
    out = np.empty(x.size, np.int8)
    lib().lqo_act_quant_i8(_p(x), C.c_float(clampv), _p(out), C.c_int64(x.size))
    return out


def act_quant_i8_dynamic(x, M, K, alpha_bf16: bool):
    """-> (x8 int8[M*K], sx float32[M], clampv, alpha)"""
    x = _c(x.reshape(-1), np.uint16)
    x8 = np.empty(M * K, np.int8)
    sx = np.empty(M, np.float32)
    out2 = np.empty(2, np.float32)
    lib().lqo_act_quant_i8_dynamic(_p(x), _p(x8), _p(sx), _p(out2), C.c_int64(M), C.c_int64(K), C.c_int(1 if alpha_bf16 else 0))
    return x8, sx, out2[0], out2[1]


def act_quant_i8_per_token(x, M, K):
    """-> (x8 int8[M*K], sx float32[M])"""
    x = _c(x.reshape(-1), np.uint16)
    x8 = np.empty(M * K, np.int8)
    sx = np.empty(M, np.float32)
    lib().lqo_act_quant_i8_per_token(_p(x), _p(x8), _p(sx), C.c_int64(M), C.c_int64(K))
    return x8, sx


def gptq_to_native(qweight, N, K) -> np.ndarray:
    qweight = _c(qweight.reshape(-1), np.int32)
    out = np.empty(N * K // 2, np.uint8)
    lib().lqo_gptq_to_native(_p(qweight), _p(out), C.c_int64(N), C.c_int64(K))
    return out


def native_to_gptq(packed, N, K) -> np.ndarray:
    packed = _c(packed.reshape(-1).view(np.uint8), np.uint8)
    out = np.empty((K // 8, N), np.int32)
    lib().lqo_native_to_gptq(_p(packed), _p(out), C.c_int64(N), C.c_int64(K))
    return out


def markstein_check(seed: int, per_scale: int):
    """(quotient mismatches, code mismatches, cases) of the reciprocal-based divide; see lq_oracle.c."""
    qm, cm, n = C.c_int64(0), C.c_int64(0), C.c_int64(0)
    lib().lqo_markstein_check(C.c_uint32(seed), C.c_int(per_scale), C.byref(qm), C.byref(cm), C.byref(n))
    return qm.value, cm.value, n.value


def residual_quant(x_bits, mode, k1=0, b1=0.0, k2=0, b2=0.0, k3=0):
    """-> (words uint32[n/8], carries as bf16 bits); the input array is not modified."""
    x = _c(x_bits.reshape(-1), np.uint16).copy()
    q = np.empty(x.size // 8, np.uint32)
    lib().lqo_residual_quant(_p(x), _p(q), C.c_int64(q.size), C.c_int(mode), C.c_int(k1), C.c_float(b1), C.c_int(k2),
                             C.c_float(b2), C.c_int(k3))
    return q, x


def residual_quant_s(x_f32):
    """Deterministic uniform quantiser on float32 values -> (words uint32[n/8], carries uint8[n])."""
    x = _c(x_f32.reshape(-1), np.float32)
    q = np.empty(x.size // 8, np.uint32)
    carry = np.empty(x.size, np.uint8)
    lib().lqo_residual_quant_s(_p(x), _p(q), _p(carry), C.c_int64(q.size))
    return q, carry


def residual_dequant(q, mode, k1=0, b1=0.0, k2=0, b2=0.0, k3=0):
    q = _c(q.reshape(-1).view(np.uint32), np.uint32)
    x = np.empty(q.size * 8, np.uint16)
    lib().lqo_residual_dequant(_p(q), _p(x), C.c_int64(q.size), C.c_int(mode), C.c_int(k1), C.c_float(b1), C.c_int(k2),
                               C.c_float(b2), C.c_int(k3))
    return x
