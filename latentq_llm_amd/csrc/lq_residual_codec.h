// Device-side pieces of the 4-bit residual codec shared by the codec kernels (lq_residual.hip)
// and the fused latent-weight kernels (lq_latent.hip). See lq_residual.hip for the semantics.
#pragma once
#include "lq_common.h"

namespace {

struct CodecParams {
    float c1, c2, c3;  // forward slopes (quant) or inverse slopes (dequant)
    float b1, b2;
    int t1, t2;
};

// roundf (halves away from zero) as trunc(x + copysign(pred(0.5), x)): the sum cannot reach the next integer
// unless x is at or past the half (pred(0.5) = 0.5 - 2^-25 is the largest float below 0.5), a half itself rounds
// up to the integer in the addition, and from 2^23 on x is an integer and the sum rounds back to it. Three
// instructions instead of six; checked against roundf on 2^26 floats around every kind of boundary by the CPU tests
// (the same expression in numpy) and through the kernels on every bf16 input.
__device__ __forceinline__ float lq_round_half_away(float x) {
    return truncf(x + __builtin_copysignf(0.49999997f, x));
}
// the same for x >= 0 (or NaN)
__device__ __forceinline__ float lq_round_half_up_nonneg(float x) { return truncf(x + 0.49999997f); }

// Branch-free: the segment only selects the operands of one fused multiply-add and one rounding.
__device__ __forceinline__ float level_3fold(float x, const CodecParams &p) {
    const float S = fabsf(x);
    float v = fmaf(S, 499.0f, 0.0f);
    v -= lq_round_half_up_nonneg(v);
    const bool in1 = S < p.b1, in2 = S < p.b2;
    const float arg = in1 ? x : (S - (in2 ? p.b1 : p.b2));
    const float slope = in1 ? p.c1 : (in2 ? p.c2 : p.c3);
    const float lv = lq_round_half_away(fmaf(arg, slope, v));
    const float r = lv + (float)(in2 ? p.t1 : p.t2);
    return in1 ? lv : (x < 0.0f ? -r : r);
}

__device__ __forceinline__ float level_uniform(float x) {
    const float S = fabsf(x);
    float v = fmaf(S, 499.0f, 0.0f);
    v = lq_round_half_up_nonneg(v) - v;
    return lq_round_half_away(fmaf(x, 8.0f, v));
}

// float level -> (nibble, carry). Levels below -8 (and NaN) give nibble 0: v_cvt_u32_f32 saturates negative
// inputs to 0 and converts NaN to 0, which is what the float->unsigned conversion of the reference's target does
// as well. Without a carry the level is at most 7, so level + 8 fits the nibble; the mask keeps wild inputs in it.
__device__ __forceinline__ unsigned nibble_of(float lv, bool &carry) {
    carry = lv > 7.5f;
    unsigned t;
    asm("v_cvt_u32_f32 %0, %1" : "=v"(t) : "v"(lv + 8.0f));
    return carry ? 1u : (t & 0xFu);
}

// nibble - 8 -> value of the three-segment curve (inverse slopes in p), branch-free
__device__ __forceinline__ float value_3fold(int s, const CodecParams &p) {
    const int a = s < 0 ? -s : s;
    const bool in1 = a <= p.t1, in2 = a <= p.t2;
    // |s| <= t1: s * c1;  else sign(s) * (b + (|s| - t) * c), written as fma((s -+ t), c, +-b)
    const int t = in2 ? p.t1 : p.t2;
    const float c = in1 ? p.c1 : (in2 ? p.c2 : p.c3);
    const float b = in2 ? p.b1 : p.b2;
    const float mid = (float)s * c;
    const float out = fmaf((float)(s < 0 ? s + t : s - t), c, s < 0 ? -b : b);
    return in1 ? mid : out;
}

inline CodecParams lq_codec_quant_params(int k1, float b1, int k2, float b2, int k3) {
    CodecParams p = {};
    p.c1 = (float)k1 / b1;
    p.c2 = (float)k2 / (b2 - b1);
    p.c3 = (float)((double)k3 / (0.5 - (double)b2));
    p.b1 = b1; p.b2 = b2; p.t1 = k1; p.t2 = k1 + k2;
    return p;
}

inline CodecParams lq_codec_dequant_params(int k1, float b1, int k2, float b2, int k3) {
    CodecParams p = {};
    p.c1 = b1 / (float)k1;
    p.c2 = (b2 - b1) / (float)k2;
    p.c3 = (float)((0.5 - (double)b2) / (double)k3);
    p.b1 = b1; p.b2 = b2; p.t1 = k1; p.t2 = k1 + k2;
    return p;
}

}  // namespace
