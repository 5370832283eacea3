// The 8-bit gradient accumulator's arithmetic on 16 consecutive elements, shared by the stand-alone pass
// (lq_gradq8.hip) and the weight-gradient GEMM's accumulate epilogue (lq_gemm_dw.hip).
#pragma once
#include "lq_common.h"

namespace {

__device__ __forceinline__ float bf16r(float v) { return lq_bf16_bits_to_f32(lq_f32_to_bf16_bits(v)); }

__device__ __forceinline__ float bf16_of(const u32x4_t v, int j) { return (j & 1) ? lq_bf16_hi(v[j >> 1]) : lq_bf16_lo(v[j >> 1]); }

// 16 consecutive elements (two 16-byte pieces of dW, 16 old int8, one Philox block or two pieces of noise).
//
// kFast (2^-40 <= s <= 2^40): only bf16(x / s) is needed, x and s are bf16 numbers, and the quotient of two
// 8-bit significands is never closer than 2^-17 (relative) to a bf16 rounding tie (a tie has a 9-bit odd
// significand t, and s t = x has no solution with x below 2^8), while x RN(1/s) is within 2^-23 of it: the
// product rounds to the same bf16 number as the IEEE quotient. Where the quotient is a bf16 subnormal that
// argument fails, and there the sum with the noise and the final code are the same for both anyway. Infinities
// and NaN go the same way through the product as through the quotient.
// clamp(rint(y), -128, 127) is taken as sat_u8(rne(y + 128)) - 128: y is a bf16 number, so y + 128 is exact
// in fp32 whenever |y| >= 2^-8, below that both forms give 0, and ties keep their parity. NaN -> -128.
template <bool kPhilox, bool kAcc, bool kFast>
__device__ __forceinline__ u32x4_t quant16(const u32x4_t v0, const u32x4_t v1, const u32x4_t old, const u32x4_t n0,
                                           const u32x4_t n1, float s, float r, unsigned long long counter,
                                           unsigned long long seed) {
    unsigned w[4] = {0u, 0u, 0u, 0u};
    if (kPhilox) {
        const lq_u4 A = lq_philox4x32_10((unsigned)counter, (unsigned)(counter >> 32), 0u, 0u, (unsigned)seed,
                                         (unsigned)(seed >> 32));
        w[0] = A.x; w[1] = A.y; w[2] = A.z; w[3] = A.w;
    }
    unsigned o[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        float x = j < 8 ? bf16_of(v0, j) : bf16_of(v1, j - 8);
        if (kAcc) {
            const int qi = (int)(signed char)((old[j >> 2] >> (8 * (j & 3))) & 0xFFu);
            x = bf16r(bf16r((float)qi * s) + x);
        }
        float nz;
        if (kPhilox) nz = fmaf((float)((w[j >> 2] >> (8 * (j & 3))) & 0xFFu), 0x1p-8f, 0x1p-9f - 0.5f);  // (2b - 255) / 512
        else nz = j < 8 ? bf16_of(n0, j) : bf16_of(n1, j - 8);
        const float q = kFast ? x * r : x / s;
        const float y = bf16r(bf16r(q) + nz) + 128.0f;
        switch (j & 3) {
            case 0: o[j >> 2] = act_cvt_pk_u8<0>(y, o[j >> 2]); break;
            case 1: o[j >> 2] = act_cvt_pk_u8<1>(y, o[j >> 2]); break;
            case 2: o[j >> 2] = act_cvt_pk_u8<2>(y, o[j >> 2]); break;
            default: o[j >> 2] = act_cvt_pk_u8<3>(y, o[j >> 2]); break;
        }
    }
    return u32x4_t{o[0] ^ 0x80808080u, o[1] ^ 0x80808080u, o[2] ^ 0x80808080u, o[3] ^ 0x80808080u};
}

}  // namespace
