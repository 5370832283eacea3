// Shared device/host helpers for the gfx950 kernels of liblatentq_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/latentq.h"

// ---- error plumbing (defined in lq_api.hip) --------------------------------
int lq_fail(int code, const char *fmt, ...);
int lq_check_launch(const char *what);
int lq_device_cu_count();  // compute units of the current device (cached)

#define LQ_REQUIRE(cond, ...)                          \
    do {                                               \
        if (!(cond)) return lq_fail(LQ_ERR_BAD_ARG, __VA_ARGS__); \
    } while (0)

static inline bool lq_aligned(const void *p, size_t a) { return ((uintptr_t)p & (a - 1)) == 0; }

// ---- vector types ----------------------------------------------------------
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) int i32x4_t;
typedef __attribute__((ext_vector_type(16))) int i32x16_t;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4_t;
typedef __attribute__((ext_vector_type(2))) unsigned u32x2_t;

// ---- bf16 <-> fp32 on raw bits ---------------------------------------------
__device__ __forceinline__ float lq_bf16_lo(unsigned packed) { return __uint_as_float(packed << 16); }
__device__ __forceinline__ float lq_bf16_hi(unsigned packed) { return __uint_as_float(packed & 0xFFFF0000u); }
__device__ __forceinline__ float lq_bf16_bits_to_f32(unsigned short b) { return __uint_as_float(((unsigned)b) << 16); }

// Two fp32 -> packed bf16 pair, round-to-nearest-even (v_cvt_pk_bf16_f32): lo = a, hi = b.
__device__ __forceinline__ unsigned lq_pack_bf16(float a, float b) {
    bf16x2_t r;
    r[0] = (__bf16)a;
    r[1] = (__bf16)b;
    return __builtin_bit_cast(unsigned, r);
}
__device__ __forceinline__ unsigned short lq_f32_to_bf16_bits(float a) {
    __bf16 r = (__bf16)a;
    return __builtin_bit_cast(unsigned short, r);
}

// byte SEL of `old` replaced by sat_u8(rne(v)) (v_cvt_pk_u8_f32: saturates to 0..255, NaN -> 0)
template <int SEL>
__device__ __forceinline__ unsigned act_cvt_pk_u8(float v, unsigned old) {
    unsigned r;
    asm("v_cvt_pk_u8_f32 %0, %1, %2, %3" : "=v"(r) : "v"(v), "n"(SEL), "v"(old));
    return r;
}

// ---- native int4 layout ----------------------------------------------------
// A little-endian 32-bit word of the native layout holds the codes of 8
// consecutive k: code j sits at bit 4*(j^1)  (even index = high nibble of its byte).
__device__ __forceinline__ unsigned lq_code(unsigned word, int j) { return (word >> (4 * (j ^ 1))) & 0xFu; }

// Two adjacent bytes holding 0..15 -> two floats q/512, one instruction (v_cvt_pk_f32_fp8): read
// as OCP FP8 E4M3, the bit patterns 0..15 are exactly q * 2^-9 (the first normal binade continues
// the subnormals linearly). hi = false: bytes 0 and 1 of x, true: bytes 2 and 3.
typedef float lq_f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ lq_f32x2_t lq_nibbles_lo(unsigned x) { return __builtin_amdgcn_cvt_pk_f32_fp8((int)x, false); }
__device__ __forceinline__ lq_f32x2_t lq_nibbles_hi(unsigned x) { return __builtin_amdgcn_cvt_pk_f32_fp8((int)x, true); }

// 8 codes of a native word -> 8 floats in k order, f = (q - z) * s rounded once:
// nzs = -(z*s) is exact for bf16 z and s, s512 = 512*s is exact, and fma(q/512, s512, nzs) rounds
// the exact (q - z) * s (scales of 2^118 and more, for which 512*s overflows, are not supported).
__device__ __forceinline__ void lq_dequant_word_f32(unsigned word, float s512, float nzs, float f[8]) {
    const unsigned lo4 = word & 0x0F0F0F0Fu;         // odd k
    const unsigned hi4 = (word >> 4) & 0x0F0F0F0Fu;  // even k
    const lq_f32x2_t e0 = lq_nibbles_lo(hi4), e1 = lq_nibbles_hi(hi4);  // k = 0, 2 and 4, 6
    const lq_f32x2_t o0 = lq_nibbles_lo(lo4), o1 = lq_nibbles_hi(lo4);  // k = 1, 3 and 5, 7
    f[0] = fmaf(e0[0], s512, nzs); f[1] = fmaf(o0[0], s512, nzs);
    f[2] = fmaf(e0[1], s512, nzs); f[3] = fmaf(o0[1], s512, nzs);
    f[4] = fmaf(e1[0], s512, nzs); f[5] = fmaf(o1[0], s512, nzs);
    f[6] = fmaf(e1[1], s512, nzs); f[7] = fmaf(o1[1], s512, nzs);
}

// ---- Philox4x32-10 ---------------------------------------------------------
#define LQ_PHILOX_M0 0xD2511F53u
#define LQ_PHILOX_M1 0xCD9E8D57u
#define LQ_PHILOX_W0 0x9E3779B9u
#define LQ_PHILOX_W1 0xBB67AE85u

struct lq_u4 {
    unsigned x, y, z, w;
};

__host__ __device__ __forceinline__ lq_u4 lq_philox4x32_10(unsigned c0, unsigned c1, unsigned c2, unsigned c3,
                                                          unsigned k0, unsigned k1) {
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        unsigned long long p0 = (unsigned long long)LQ_PHILOX_M0 * c0;
        unsigned long long p1 = (unsigned long long)LQ_PHILOX_M1 * c2;
#if defined(__HIP_DEVICE_COMPILE__)
        // three-input XOR in one instruction (v_bitop3_b32, truth table 0x96)
        unsigned n0 = __builtin_amdgcn_bitop3_b32((unsigned)(p1 >> 32), c1, k0, 0x96);
        unsigned n2 = __builtin_amdgcn_bitop3_b32((unsigned)(p0 >> 32), c3, k1, 0x96);
#else
        unsigned n0 = (unsigned)(p1 >> 32) ^ c1 ^ k0;
        unsigned n2 = (unsigned)(p0 >> 32) ^ c3 ^ k1;
#endif
        unsigned n1 = (unsigned)p1;
        unsigned n3 = (unsigned)p0;
        c0 = n0; c1 = n1; c2 = n2; c3 = n3;
        k0 += LQ_PHILOX_W0;
        k1 += LQ_PHILOX_W1;
    }
    lq_u4 o = {c0, c1, c2, c3};
    return o;
}
