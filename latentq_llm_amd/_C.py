"""ctypes binding of liblatentq_hip.so (the C ABI declared in include/latentq.h).

The library is mandatory: there is no CPU or eager fallback. Loading fails loudly
when the shared object has not been built (python -m latentq_llm_amd.build).
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liblatentq_hip.so")

ABI_VERSION = 2

_vp, _i64, _i32, _u64, _f32, _f64 = C.c_void_p, C.c_int64, C.c_int, C.c_uint64, C.c_float, C.c_double

# name -> argtypes; every function returns int except lq_last_error.
SIGNATURES = {
    "lq_abi_version": [],
    "lq_requant_sr": [_vp, _vp, _vp, _vp, _vp, _f32, _i64, _i64, _i32, _vp, _u64, _u64, _vp],
    "lq_philox_uniform": [_vp, _i64, _u64, _u64, _vp],
    "lq_a16w4_fwd": [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _vp],
    "lq_a16w4_fwd_ws": [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _vp, _i64, _vp],
    "lq_a16w4_fwd_static": [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _vp],
    "lq_a16w4_dx": [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _vp],
    "lq_a16w4_dx_ws": [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _vp, _i64, _vp],
    "lq_a16w4_plan": [_i32, _i64, _i64, _i64, _i64, _i32, _vp, _vp, _vp],
    "lq_a16w4_dequant": [_vp, _vp, _vp, _vp, _i64, _i64, _i32, _vp],
    "lq_a8w8_fwd": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp],
    "lq_a8w8_dx": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp],
    "lq_act_quant_i8": [_vp, _vp, _vp, _i64, _vp],
    "lq_act_quant_i8_dynamic": [_vp, _vp, _vp, _vp, _i64, _i64, _i32, _vp],
    "lq_act_quant_i8_per_token": [_vp, _vp, _vp, _i64, _i64, _vp],
    "lq_act_dequant_i8": [_vp, _vp, _i32, _vp, _i64, _i64, _vp],
    "lq_act_fake_quant": [_vp, _vp, _vp, _i64, _vp],
    "lq_a8w8_fwd_qs": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp],
    "lq_residual_quant": [_vp, _vp, _i64, _i32, _i32, _f32, _i32, _f32, _i32, _vp],
    "lq_residual_dequant": [_vp, _vp, _i64, _i32, _i32, _f32, _i32, _f32, _i32, _vp],
    "lq_a16w4_gate_up_silu": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _vp],
    "lq_a16w4_gate_up_silu_save": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _vp],
    "lq_a16w4_dx_silu_bwd": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _vp],
    "lq_a16w4_dx_acc": [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _vp],
    "lq_a16w4_dx_pair": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _vp],
    "lq_w8_requant": [_vp, _vp, _vp, _i64, _i64, _vp],
    "lq_residual_quant_s": [_vp, _vp, _i64, _i32, _vp],
    "lq_gradq8_quant": [_vp, _vp, _vp, _i32, _i64, _i64, _vp, _u64, _u64, _vp],
    "lq_weight_grad": [_vp, _vp, _vp, _i64, _i64, _i64, _vp],
    "lq_weight_grad_acc": [_vp, _vp, _vp, _i64, _i64, _i64, _vp],
    "lq_weight_grad_acc8": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _u64, _u64, _vp],
    "lq_repack_gptq_to_native": [_vp, _vp, _i64, _i64, _vp],
    "lq_repack_native_to_gptq": [_vp, _vp, _i64, _i64, _vp],
    "lq_calib_copy": [_vp, _vp, _i64, _vp],
    "lq_calib_read": [_vp, _i64, _i32, _vp, _vp],
    "lq_calib_mfma_loop": [_vp, _vp, _i64, _i64, _i32, _vp, _i64, _vp, _vp, _vp],
    "lq_calib_mfma_loop_i8": [_vp, _vp, _i64, _i64, _i32, _vp, _i64, _vp, _vp, _vp],
    "lq_calib_gemm_clocks": [_i32, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _vp, _i64, _vp, _vp],
    "lq_transpose_bf16": [_vp, _vp, _i64, _i64, _vp],
    "lq_latent_w4_reconstruct": [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i32, _i32, _f32, _i32, _f32, _i32, _vp],
    "lq_latent_w4_requant": [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i32, _i32, _f32, _i32, _f32, _i32, _vp],
    "lq_latent_w8_reconstruct": [_vp, _vp, _vp, _vp, _i64, _i64, _i32, _f32, _i32, _f32, _i32, _vp],
    "lq_latent_w8_requant": [_vp, _vp, _vp, _vp, _i64, _i64, _i32, _f32, _i32, _f32, _i32, _vp],
    "lq_adam8_update": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i32, _f64, _f64, _f64, _f64, _vp],
    "lq_adam8_latent_w4_step": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i32, _i32,
                                _i32, _f32, _i32, _f32, _i32, _i32, _f32, _i32, _f32, _i32, _f64, _f64, _f64, _f64, _vp],
    "lq_adam8_latent_w8_step": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i32,
                                _i32, _f32, _i32, _f32, _i32, _i32, _f32, _i32, _f32, _i32, _f64, _f64, _f64, _f64, _vp],
}

_lib = None


class LatentQError(RuntimeError):
    pass


def load():
    """Load the shared library once and type its entry points."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise LatentQError(
            f"{LIB_PATH} is missing: build it with `python -m latentq_llm_amd.build` "
            "(there is no fallback path without the HIP library)")
    lib = C.CDLL(LIB_PATH)
    for name, args in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError here = library older than this binding
        fn.argtypes = args
        fn.restype = C.c_int
    lib.lq_last_error.argtypes = []
    lib.lq_last_error.restype = C.c_char_p
    got = lib.lq_abi_version()
    if got != ABI_VERSION:
        raise LatentQError(f"liblatentq_hip.so has ABI {got}, binding expects {ABI_VERSION}; rebuild")
    _lib = lib
    return lib


def call(name: str, *args) -> None:
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise LatentQError(f"{name} failed ({rc}): {lib.lq_last_error().decode()}")
