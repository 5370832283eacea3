// Per-element arithmetic of the lbit = 4 latent weight (codes + 4-bit residual), shared by the
// latent passes (lq_latent.hip) and the fused optimizer step (lq_adam8.hip). Every line is one
// tensor operation of the reference's chains (utils/quant.py:45-72, 803-837) with its bf16 rounding.
#pragma once
#include "lq_common.h"
#include "lq_residual_codec.h"

__device__ __forceinline__ float lq_bf16r(float v) { return lq_bf16_bits_to_f32(lq_f32_to_bf16_bits(v)); }

// The dequantised value of a residual nibble depends on nothing but the nibble, so a workgroup keeps
// the 16 values bf16(value(n - 8)) in LDS and an element costs one LDS read instead of the curve's
// dozen selects and operations. Threads 0..15 fill the table; the caller synchronises before use.
__device__ __forceinline__ void lq_latent_fill_value_table(float *tab, const CodecParams &pd) {
    if (threadIdx.x < 16) tab[threadIdx.x] = lq_bf16r(value_3fold((int)threadIdx.x - 8, pd));
}

// latent = bf16(bf16(bf16(value(nibble)) * s) + bf16(bf16(q - z) * s)) with value_bf16 =
// bf16(value(nibble)) from the table; the caller applies the last rounding
__device__ __forceinline__ float lq_latent_value(unsigned code, float value_bf16, float s, float z) {
    const float wq = lq_bf16r(lq_bf16r((float)code - z) * s);
    const float r = lq_bf16r(value_bf16 * s);
    return r + wq;
}

// One element of the re-quantiser: Z = bf16(bf16(t / s) + z), q = rint(Z), residual nibble and
// carry from bf16(Z - q), code = clamp(bf16(q + carry), 0, 15).
// Only bf16(t / s) is needed, and t and s are bf16 numbers: their quotient keeps a relative distance of at
// least 2^-17 from every bf16 rounding tie (a tie has a 9-bit odd significand, and s * tie = t has no solution
// with t below 2^8), so for 2^-40 <= s <= 2^40 (kFast; the caller branches once per group) the product
// t * RN(1/s), which is within 2^-23 of the quotient, rounds to the same bf16 number. Where the quotient is a
// bf16 subnormal that argument fails, and there q = rint(Z) and the residual level (0) are the same either way;
// infinities and NaN go the same way through the product as through the quotient.
template <bool kFast>
__device__ __forceinline__ void lq_latent_requant_elem(float t, float s, float z, float r, const CodecParams &pq,
                                                       unsigned &nib, unsigned &code) {
    const float quo = kFast ? t * r : t / s;
    const float Z = lq_bf16r(lq_bf16r(quo) + z);
    const float q = rintf(Z);  // round half to even, as torch.round
    const float f = lq_bf16r(Z - q);
    bool carry;
    nib = nibble_of(level_3fold(f, pq), carry);
    // clamp(bf16(q + carry), 0, 15): q + carry is an integer, bf16 keeps every integer up to 256 and is
    // monotonic, so the rounding cannot change what the clamp returns; a NaN ends as code 0
    const float c = __builtin_amdgcn_fmed3f(fmaxf(q + (carry ? 1.0f : 0.0f), 0.0f), 0.0f, 15.0f);
    code = (unsigned)c;
}

// ---- 8-bit weights (int8 codes, one bf16 scale per row; utils/quant.py:88-103, 826-837, 1069-1070) ----
// latent = bf16(bf16(value(nibble)) * s) + bf16(q * s); the caller applies the last rounding
__device__ __forceinline__ float lq_latent_w8_value(unsigned byte, float value_bf16, float s) {
    const float q = (float)(int)(signed char)(byte & 0xFFu);
    return lq_bf16r(value_bf16 * s) + lq_bf16r(q * s);
}

// One element of the 8-bit re-quantiser: Z = bf16(t / s), q = rint(Z), residual nibble and carry from
// bf16(Z - q), code byte = clamp(q + carry, -128, 127) (NaN -> 0). kFast: the quotient as the product with
// r = 1 / s, valid for 2^-40 <= |s| <= 2^40 (see lq_latent_requant_elem).
template <bool kFast>
__device__ __forceinline__ void lq_latent_w8_requant_elem(float t, float s, float r, const CodecParams &pq, unsigned &nib,
                                                          unsigned &byte) {
    const float quo = kFast ? t * r : t / s;
    const float Z = lq_bf16r(quo);
    const float q = rintf(Z);  // round half to even, as torch.round
    const float f = lq_bf16r(Z - q);
    bool carry;
    nib = nibble_of(level_3fold(f, pq), carry);
    // q + carry is an integer (bf16 holds it exactly wherever the clamp does not decide); NaN -> 0
    const float c = q + (carry ? 1.0f : 0.0f);
    const float cc = c == c ? __builtin_amdgcn_fmed3f(c, -128.0f, 127.0f) : 0.0f;
    byte = (unsigned)(int)cc & 0xFFu;
}
