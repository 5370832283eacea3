// Fused Adam step on 8-bit block-wise moments for gfx950.
//
// The reference's optimizer (utils/quant.py:1081-1134 with Qfunc_8bit_opt / DeQfunc_8bit_opt,
// :22-41) keeps both moments as uint8 with one fp32 (scale, max) pair per block of 2048 (or 128)
// elements, the second one as sqrt(v) + eps, and runs one step as a chain of ~25 elementwise
// tensor operations per parameter:
//     m  = bf16(max1 - q1 * scale1)                      s2 = max2 - q2 * scale2,  v = bf16(s2 * s2)
//     m  = bf16(m * beta1);  m = bf16(m + (1 - beta1) * g)
//     v  = bf16(v * beta2);  v = bf16(v + (1 - beta2) * g * g)
//     d  = bf16(sqrt(v));    d = bf16(d + eps)
//     p  = bf16(p - step * (m / d))                      (or, for the stochastic-rounding
//                                                         requantizer, direction = bf16(m / d))
//     per block: max = max(x), scale = (max - min(x)) * (1/255) + 1e-10,
//                q = clamp(rint((max - x) / scale), 0, 255)        for x = m and for x = d
// Every tensor operation computes in fp32 and rounds its result to the tensor's type; an
// operation of the form a + alpha * b is a fused multiply-add inside the tensor library's
// kernels. This kernel is that chain in one pass with the same rounding points, so its results
// equal the chain's bit for bit: 8 elements per thread (16 bytes of gradient and parameter, 8
// bytes of each moment), the block's minimum and maximum found by a reduction over the BS/8
// threads of the block, 6 bytes read and 4 written per element instead of ~120.
//
// In its latent mode the kernel also takes over the two passes around the step in the exact
// 4-bit-residual mode of the A16W4 layer: the parameter is rebuilt from codes and residual words
// (as lq_latent_w4_reconstruct does) and the updated value goes straight back to codes and
// residual words (as lq_latent_w4_requant does); a thread's 8 elements are one code word and one
// residual word. The whole optimizer step of a layer is then one pass over 4 + 4 bytes of codes
// and residual, 16 of gradient and 16 of moments per 8 elements.
#include "lq_latent_math.h"

namespace {

__device__ __forceinline__ float bf16r(float v) { return lq_bf16r(v); }

struct Adam8Params {
    const u32x4_t *grad;     // bf16
    u32x4_t *param;          // bf16, updated in place, or null
    u32x4_t *direction;      // bf16 m / d, or null
    u32x2_t *state1, *state2;  // uint8 moments, updated in place
    float *scale1, *max1, *scale2, *max2;  // per block, updated in place
    long long n_threads;     // elements / 8
    float beta1, one_minus_beta1, beta2, one_minus_beta2, eps, neg_step;
    // latent mode: the parameter lives as codes + residual words (one of each per thread)
    unsigned *codes, *residual;
    const unsigned short *wscales, *wzeros;  // per group of 128 elements
    CodecParams dequant_curve, quant_curve;
    // latent mode of an 8-bit-weight layer: int8 codes (8 per thread), one bf16 scale per row of K elements
    u32x2_t *codes8;
    const unsigned short *qscales;
    long long threads_per_row;  // K / 8
};

enum { LATENT_NONE = 0, LATENT_W4 = 1, LATENT_W8 = 2 };

// minimum and maximum over the W threads that share a block (W = 16: one 16-lane row of the
// wave, by cross-lane shuffles; W = 256: the whole workgroup, through LDS)
template <int W>
__device__ __forceinline__ void block_minmax(float &lo, float &hi, float (*red)[2]) {
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) {
        lo = fminf(lo, __shfl_xor(lo, off, 64));
        hi = fmaxf(hi, __shfl_xor(hi, off, 64));
    }
    if constexpr (W == 256) {
#pragma unroll
        for (int off = 16; off < 64; off <<= 1) {
            lo = fminf(lo, __shfl_xor(lo, off, 64));
            hi = fmaxf(hi, __shfl_xor(hi, off, 64));
        }
        const int wave = threadIdx.x >> 6;
        __syncthreads();  // the previous use of red has been read
        if ((threadIdx.x & 63) == 0) { red[wave][0] = lo; red[wave][1] = hi; }
        __syncthreads();
        lo = fminf(fminf(red[0][0], red[1][0]), fminf(red[2][0], red[3][0]));
        hi = fmaxf(fmaxf(red[0][1], red[1][1]), fmaxf(red[2][1], red[3][1]));
    }
}

// byte SEL of `old` replaced by sat_u8(rne(v)) (v_cvt_pk_u8_f32)
template <int SEL>
__device__ __forceinline__ unsigned cvt_pk_u8(float v, unsigned old) {
    unsigned r;
    asm("v_cvt_pk_u8_f32 %0, %1, %2, %3" : "=v"(r) : "v"(v), "n"(SEL), "v"(old));
    return r;
}

// m / d, correctly rounded, for two bf16 numbers. The quotient of two 8-bit significands keeps a relative
// distance of at least 2^-33 from every midpoint of two fp32 numbers (m = d * mid has no solution: mid has 25
// significant bits), and q0 = m r with the hardware reciprocal r (one ulp), corrected once by the exact residual
// (q0 + (m - q0 d) r, one rounding), is within 2^-45 of the quotient: it rounds to the same fp32 number as the
// IEEE division (every significand pair and every one-ulp variant of r is checked on the CPU). Quotients or
// divisors outside [2^-40, 2^40] (residual underflow, overflow, zero, NaN) take the division (div_bf16_operands
// names this sequence in the comments below; it is written out in the kernel).

// x[8] -> uint8 codes with the block's (scale, max); returns them packed, 8 bytes.
// The quotient (hi - x) / scale must be the correctly rounded one (a quotient one ulp off can fall
// on the other side of a rounding tie). The divisor is shared by the whole block, so the division
// is done with its correctly rounded reciprocal r = RN(1 / scale) and two residual corrections:
// q0 = t*r; q1 = q0 + (t - q0*scale)*r is within one ulp of t/scale, and one more correction of a
// quotient within one ulp returns RN(t / scale) exactly (Markstein's theorem; the residuals are
// exact as long as they do not underflow, and a numerator below 2^-100 gives code 0 either way
// because scale >= 1e-10). Half the instructions of an IEEE division. A scale above 2^60 (or NaN)
// takes the plain division.
__device__ __forceinline__ u32x2_t quantize8(const float x[8], float scale, float hi) {
    unsigned w[2] = {0u, 0u};
    const bool fast = scale <= 0x1p60f;
    const float r = 1.0f / scale;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const float t = hi - x[k];
        float q;
        if (fast) {
            const float q0 = t * r;
            const float q1 = fmaf(fmaf(-q0, scale, t), r, q0);
            q = fmaf(fmaf(-q1, scale, t), r, q1);
        } else {
            q = t / scale;
        }
        // clamp(rint(q), 0, 255) and the byte insertion in one instruction (round to nearest even, saturating,
        // NaN -> 0 like fmaxf(NaN, 0))
        switch (k & 3) {
            case 0: w[k >> 2] = cvt_pk_u8<0>(q, w[k >> 2]); break;
            case 1: w[k >> 2] = cvt_pk_u8<1>(q, w[k >> 2]); break;
            case 2: w[k >> 2] = cvt_pk_u8<2>(q, w[k >> 2]); break;
            default: w[k >> 2] = cvt_pk_u8<3>(q, w[k >> 2]); break;
        }
    }
    return u32x2_t{w[0], w[1]};
}

// bf16(sqrt(v)) for a bf16 value v. The square root of a number with 8 significant bits never
// comes closer than 2^-19 (relative) to the midpoint of two bf16 values, so any fp32 square root
// within two ulps rounds to the same bf16 value as the correctly rounded one (checked for every
// bf16 input by the CPU tests); the hardware's v_sqrt_f32 (one ulp) replaces the ~12-instruction
// correctly rounded sequence. Inputs below 2^-100 (the instruction does not take denormals) go
// through the exact one.
__device__ __forceinline__ float sqrt_bf16_to_bf16(float v) {
    if (v >= 0x1p-100f) return bf16r(__builtin_amdgcn_sqrtf(v));
    return bf16r(__builtin_sqrtf(v));
}

// A thread's 8 updated latent values back to one code word and one residual word (codec parameters by value)
template <bool kFast>
__device__ __forceinline__ void requant8(const float (&out)[8], float ws, float wz, float wr, const CodecParams pq,
                                         unsigned &cnew, unsigned &rnew) {
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        unsigned nib, code;
        lq_latent_requant_elem<kFast>(out[k], ws, wz, wr, pq, nib, code);
        rnew = (rnew << 4) | nib;
        cnew |= code << (4 * (k ^ 1));
    }
}

// The same for an 8-bit-weight layer: 8 code bytes and one residual word per thread
template <bool kFast>
__device__ __forceinline__ void requant8_w8(const float (&out)[8], float ws, float wr, const CodecParams pq, u32x2_t &cnew,
                                            unsigned &rnew) {
    unsigned cw[2] = {0u, 0u};
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        unsigned nib, byte;
        lq_latent_w8_requant_elem<kFast>(out[k], ws, wr, pq, nib, byte);
        rnew = (rnew << 4) | nib;
        cw[k >> 2] |= byte << (8 * (k & 3));
    }
    cnew = u32x2_t{cw[0], cw[1]};
}

template <int BS, int LATENT>
__global__ __launch_bounds__(256) void adam8_update_kernel(Adam8Params a) {
    constexpr int W = BS / 8;  // threads per block of the moments
    __shared__ float red[4][2];
    __shared__ float vtab[16];  // latent mode: dequantised values of the 16 residual nibbles
    if constexpr (LATENT != LATENT_NONE) {
        lq_latent_fill_value_table(vtab, a.dequant_curve);
        __syncthreads();
    }
    const long long T = (long long)blockIdx.x * 256 + threadIdx.x;
    const bool live = T < a.n_threads;  // n is a multiple of BS: a block is all-live or all-dead
    const long long Tc = live ? T : 0;
    const long long blk = Tc / W;
    const u32x4_t g4 = a.grad[Tc];
    const u32x2_t q1 = a.state1[Tc], q2 = a.state2[Tc];
    const float sc1 = a.scale1[blk], mx1 = a.max1[blk], sc2 = a.scale2[blk], mx2 = a.max2[blk];
    u32x4_t p4 = {0u, 0u, 0u, 0u};
    unsigned cword = 0, rword = 0;
    float ws = 0.0f, wz = 0.0f;
    u32x2_t c8 = {0u, 0u};
    if constexpr (LATENT == LATENT_W4) {
        cword = a.codes[Tc];
        rword = a.residual[Tc];
        ws = lq_bf16_bits_to_f32(a.wscales[Tc >> 4]);
        wz = lq_bf16_bits_to_f32(a.wzeros[Tc >> 4]);
    } else if constexpr (LATENT == LATENT_W8) {
        c8 = a.codes8[Tc];
        rword = a.residual[Tc];
        ws = lq_bf16_bits_to_f32(a.qscales[Tc / a.threads_per_row]);
    } else if (a.param) {
        p4 = a.param[Tc];
    }

    // Phase 1: the moments. The square root and the quotient use short sequences that are exact on all but
    // extreme operands; whether any of a thread's 8 elements is such an operand is collected in one flag per
    // sequence, and the (cold) exact sequences then redo all 8: one branch per thread instead of one per element.
    float m[8], d[8], v[8], out[8];
    bool odd_sqrt = false;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const float g = (k & 1) ? lq_bf16_hi(g4[k >> 1]) : lq_bf16_lo(g4[k >> 1]);
        const float c1 = (float)((q1[k >> 2] >> (8 * (k & 3))) & 0xFFu);
        const float c2 = (float)((q2[k >> 2] >> (8 * (k & 3))) & 0xFFu);
        float mk = bf16r(mx1 - c1 * sc1);
        const float s2 = mx2 - c2 * sc2;
        float vk = bf16r(s2 * s2);
        mk = bf16r(mk * a.beta1);
        mk = bf16r(fmaf(a.one_minus_beta1, g, mk));
        vk = bf16r(vk * a.beta2);
        vk = bf16r(fmaf(a.one_minus_beta2 * g, g, vk));
        m[k] = mk;
        v[k] = vk;
        // bf16(sqrt(v)) from the hardware's one-ulp square root (see sqrt_bf16_to_bf16); it does not take
        // denormals, so nonzero inputs below 2^-100 go through the exact one (zero, negative and NaN inputs give
        // the same result either way)
        d[k] = bf16r(__builtin_amdgcn_sqrtf(vk));
        odd_sqrt |= vk < 0x1p-100f && vk > 0.0f;
    }
    if (odd_sqrt) {
#pragma unroll
        for (int k = 0; k < 8; ++k) d[k] = sqrt_bf16_to_bf16(v[k]);
    }
    float ratio[8];
    bool odd_div = false;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        d[k] = bf16r(d[k] + a.eps);
        const float r = __builtin_amdgcn_rcpf(d[k]);
        const float q0 = m[k] * r;
        if (LATENT == LATENT_NONE && !a.param) {
            // Only bf16(m / d) is stored here, and the quotient of two bf16 numbers never comes closer
            // than 2^-17 (relative) to the midpoint of two bf16 values (256 m_a = (2j+1) m_b has no
            // solution with 8-bit significands), so any fp32 quotient within a few ulps rounds to the
            // same bf16 value as the correctly rounded one (every significand pair is checked by the
            // CPU tests): reciprocal and product instead of the division sequence. Results outside
            // [2^-100, 2^100] (bf16 subnormals, overflow, NaN; zero numerators excepted) take the division.
            ratio[k] = q0;
            const float ar = fabsf(q0);
            odd_div |= !(ar <= 0x1p100f && (ar >= 0x1p-100f || m[k] == 0.0f));
        } else {
            // The fp32 quotient itself enters the update: one residual correction of q0 gives the IEEE
            // quotient of two bf16 numbers (div_bf16_operands) unless quotient or divisor leave [2^-40, 2^40].
            ratio[k] = fmaf(fmaf(-q0, d[k], m[k]), r, q0);
            const float aq = fabsf(ratio[k]), ad = fabsf(d[k]);
            odd_div |= !(aq >= 0x1p-40f && aq <= 0x1p40f && ad >= 0x1p-40f && ad <= 0x1p40f);
        }
    }
    if (odd_div) {
#pragma unroll
        for (int k = 0; k < 8; ++k) ratio[k] = m[k] / d[k];
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        if constexpr (LATENT == LATENT_W4) {
            const float p = bf16r(lq_latent_value(lq_code(cword, k), vtab[(rword >> (28 - 4 * k)) & 0xFu], ws, wz));
            out[k] = bf16r(fmaf(a.neg_step, ratio[k], p));
        } else if constexpr (LATENT == LATENT_W8) {
            const float p = bf16r(lq_latent_w8_value(c8[k >> 2] >> (8 * (k & 3)), vtab[(rword >> (28 - 4 * k)) & 0xFu], ws));
            out[k] = bf16r(fmaf(a.neg_step, ratio[k], p));
        } else if (a.param) {
            const float p = (k & 1) ? lq_bf16_hi(p4[k >> 1]) : lq_bf16_lo(p4[k >> 1]);
            out[k] = fmaf(a.neg_step, ratio[k], p);
        } else {
            out[k] = ratio[k];
        }
    }
    if constexpr (LATENT == LATENT_W4) {
        const bool fast = (ws >= 0x1p-40f) && (ws <= 0x1p40f);
        const float wr = 1.0f / ws;
        unsigned cnew = 0, rnew = 0;
        if (fast) requant8<true>(out, ws, wz, wr, a.quant_curve, cnew, rnew);
        else requant8<false>(out, ws, wz, wr, a.quant_curve, cnew, rnew);
        if (live) {
            a.codes[T] = cnew;
            a.residual[T] = rnew;
        }
    } else if constexpr (LATENT == LATENT_W8) {
        const bool fast = (fabsf(ws) >= 0x1p-40f) && (fabsf(ws) <= 0x1p40f);
        const float wr = 1.0f / ws;
        u32x2_t cnew;
        unsigned rnew = 0;
        if (fast) requant8_w8<true>(out, ws, wr, a.quant_curve, cnew, rnew);
        else requant8_w8<false>(out, ws, wr, a.quant_curve, cnew, rnew);
        if (live) {
            a.codes8[T] = cnew;
            a.residual[T] = rnew;
        }
    } else if (live) {
        const u32x4_t o = {lq_pack_bf16(out[0], out[1]), lq_pack_bf16(out[2], out[3]), lq_pack_bf16(out[4], out[5]),
                           lq_pack_bf16(out[6], out[7])};
        if (a.param) a.param[T] = o;
        else a.direction[T] = o;
    }

    // the moments back to uint8 with the block's new (scale, max)
    float lo1 = m[0], hi1 = m[0], lo2 = d[0], hi2 = d[0];
#pragma unroll
    for (int k = 1; k < 8; ++k) {
        lo1 = fminf(lo1, m[k]); hi1 = fmaxf(hi1, m[k]);
        lo2 = fminf(lo2, d[k]); hi2 = fmaxf(hi2, d[k]);
    }
    block_minmax<W>(lo1, hi1, red);
    block_minmax<W>(lo2, hi2, red);
    const float inv255 = 1.0f / 255.0f;  // the tensor library divides by a scalar as a multiplication by its reciprocal
    const float ns1 = (hi1 - lo1) * inv255 + 1e-10f;
    const float ns2 = (hi2 - lo2) * inv255 + 1e-10f;
    if (live) {
        a.state1[T] = quantize8(m, ns1, hi1);
        a.state2[T] = quantize8(d, ns2, hi2);
        if (T % W == 0) {
            a.scale1[blk] = ns1; a.max1[blk] = hi1;
            a.scale2[blk] = ns2; a.max2[blk] = hi2;
        }
    }
}

}  // namespace

static int adam8_check(const char *who, const void *grad, const void *state1, const void *state2, const void *scale1,
                       const void *max1, const void *scale2, const void *max2, int64_t n, int block_elems) {
    LQ_REQUIRE(grad && state1 && state2 && scale1 && max1 && scale2 && max2, "%s: null pointer argument", who);
    LQ_REQUIRE(block_elems == 2048 || block_elems == 128, "%s: block must be 2048 or 128 elements, got %d", who, block_elems);
    LQ_REQUIRE(n > 0 && n % block_elems == 0, "%s: n=%lld must be a positive multiple of the block (%d)", who, (long long)n,
               block_elems);
    LQ_REQUIRE(n / 8 / 256 < 0x7FFFFFFFll, "%s: tensor too large", who);
    LQ_REQUIRE(lq_aligned(grad, 16) && lq_aligned(state1, 8) && lq_aligned(state2, 8) && lq_aligned(scale1, 4) &&
                   lq_aligned(max1, 4) && lq_aligned(scale2, 4) && lq_aligned(max2, 4),
               "%s: grad must be 16-byte, the moments 8-byte aligned", who);
    return LQ_OK;
}

static void adam8_scalars(Adam8Params &a, double beta1, double beta2, double eps, double step_size) {
    // the optimizer computes its scalars in double precision and the tensor library's kernels take them as fp32
    a.beta1 = (float)beta1; a.one_minus_beta1 = (float)(1.0 - beta1);
    a.beta2 = (float)beta2; a.one_minus_beta2 = (float)(1.0 - beta2);
    a.eps = (float)eps; a.neg_step = (float)(-step_size);
}

extern "C" int lq_adam8_update(const void *grad, void *param_or_null, void *direction_or_null, uint8_t *state1,
                               uint8_t *state2, float *scale1, float *max1, float *scale2, float *max2, int64_t n,
                               int block_elems, double beta1, double beta2, double eps, double step_size, void *stream) {
    int rc = adam8_check("lq_adam8_update", grad, state1, state2, scale1, max1, scale2, max2, n, block_elems);
    if (rc) return rc;
    LQ_REQUIRE((param_or_null != nullptr) != (direction_or_null != nullptr),
               "lq_adam8_update: exactly one of param and direction must be given");
    LQ_REQUIRE((!param_or_null || lq_aligned(param_or_null, 16)) && (!direction_or_null || lq_aligned(direction_or_null, 16)),
               "lq_adam8_update: param and direction must be 16-byte aligned");
    Adam8Params a = {};
    a.grad = (const u32x4_t *)grad;
    a.param = (u32x4_t *)param_or_null;
    a.direction = (u32x4_t *)direction_or_null;
    a.state1 = (u32x2_t *)state1; a.state2 = (u32x2_t *)state2;
    a.scale1 = scale1; a.max1 = max1; a.scale2 = scale2; a.max2 = max2;
    a.n_threads = n / 8;
    adam8_scalars(a, beta1, beta2, eps, step_size);
    const unsigned blocks = (unsigned)((a.n_threads + 255) / 256);
    if (block_elems == 2048)
        hipLaunchKernelGGL((adam8_update_kernel<2048, LATENT_NONE>), dim3(blocks), dim3(256), 0, (hipStream_t)stream, a);
    else
        hipLaunchKernelGGL((adam8_update_kernel<128, LATENT_NONE>), dim3(blocks), dim3(256), 0, (hipStream_t)stream, a);
    return lq_check_launch("lq_adam8_update");
}

extern "C" int lq_adam8_latent_w4_step(const void *grad, void *codes, int32_t *residual, const void *scales,
                                       const void *zeros, uint8_t *state1, uint8_t *state2, float *scale1, float *max1,
                                       float *scale2, float *max2, int64_t N, int64_t K, int group, int block_elems,
                                       int dk1, float db1, int dk2, float db2, int dk3, int qk1, float qb1, int qk2,
                                       float qb2, int qk3, double beta1, double beta2, double eps, double step_size,
                                       void *stream) {
    LQ_REQUIRE(N > 0 && K > 0 && K % LQ_GROUP == 0, "lq_adam8_latent_w4_step: need N > 0, K a positive multiple of %d",
               LQ_GROUP);
    LQ_REQUIRE(group == LQ_GROUP, "lq_adam8_latent_w4_step: group must be %d", LQ_GROUP);
    const int64_t n = N * K;
    int rc = adam8_check("lq_adam8_latent_w4_step", grad, state1, state2, scale1, max1, scale2, max2, n, block_elems);
    if (rc) return rc;
    LQ_REQUIRE(codes && residual && scales && zeros, "lq_adam8_latent_w4_step: null pointer argument");
    LQ_REQUIRE(lq_aligned(codes, 4) && lq_aligned(residual, 4), "lq_adam8_latent_w4_step: codes and residual must be 4-byte aligned");
    LQ_REQUIRE(dk1 > 0 && dk2 > 0 && dk3 > 0 && db1 > 0.0f && db2 > db1 && db2 < 0.5f && qk1 > 0 && qk2 > 0 && qk3 > 0 &&
                   qb1 > 0.0f && qb2 > qb1 && qb2 < 0.5f,
               "lq_adam8_latent_w4_step: need k1,k2,k3 > 0 and 0 < b1 < b2 < 0.5 for both curves");
    Adam8Params a = {};
    a.grad = (const u32x4_t *)grad;
    a.state1 = (u32x2_t *)state1; a.state2 = (u32x2_t *)state2;
    a.scale1 = scale1; a.max1 = max1; a.scale2 = scale2; a.max2 = max2;
    a.n_threads = n / 8;
    a.codes = (unsigned *)codes; a.residual = (unsigned *)residual;
    a.wscales = (const unsigned short *)scales; a.wzeros = (const unsigned short *)zeros;
    a.dequant_curve = lq_codec_dequant_params(dk1, db1, dk2, db2, dk3);
    a.quant_curve = lq_codec_quant_params(qk1, qb1, qk2, qb2, qk3);
    adam8_scalars(a, beta1, beta2, eps, step_size);
    const unsigned blocks = (unsigned)((a.n_threads + 255) / 256);
    if (block_elems == 2048)
        hipLaunchKernelGGL((adam8_update_kernel<2048, LATENT_W4>), dim3(blocks), dim3(256), 0, (hipStream_t)stream, a);
    else
        hipLaunchKernelGGL((adam8_update_kernel<128, LATENT_W4>), dim3(blocks), dim3(256), 0, (hipStream_t)stream, a);
    return lq_check_launch("lq_adam8_latent_w4_step");
}

extern "C" int lq_adam8_latent_w8_step(const void *grad, int8_t *codes, int32_t *residual, const void *qscales, uint8_t *state1,
                                       uint8_t *state2, float *scale1, float *max1, float *scale2, float *max2, int64_t N,
                                       int64_t K, int block_elems, int dk1, float db1, int dk2, float db2, int dk3, int qk1,
                                       float qb1, int qk2, float qb2, int qk3, double beta1, double beta2, double eps,
                                       double step_size, void *stream) {
    LQ_REQUIRE(N > 0 && K > 0 && K % 8 == 0, "lq_adam8_latent_w8_step: need N > 0, K a positive multiple of 8");
    const int64_t n = N * K;
    int rc = adam8_check("lq_adam8_latent_w8_step", grad, state1, state2, scale1, max1, scale2, max2, n, block_elems);
    if (rc) return rc;
    LQ_REQUIRE(codes && residual && qscales, "lq_adam8_latent_w8_step: null pointer argument");
    LQ_REQUIRE(lq_aligned(codes, 8) && lq_aligned(residual, 4) && lq_aligned(qscales, 2),
               "lq_adam8_latent_w8_step: codes must be 8-byte, residual 4-byte aligned");
    LQ_REQUIRE(dk1 > 0 && dk2 > 0 && dk3 > 0 && db1 > 0.0f && db2 > db1 && db2 < 0.5f && qk1 > 0 && qk2 > 0 && qk3 > 0 &&
                   qb1 > 0.0f && qb2 > qb1 && qb2 < 0.5f,
               "lq_adam8_latent_w8_step: need k1,k2,k3 > 0 and 0 < b1 < b2 < 0.5 for both curves");
    Adam8Params a = {};
    a.grad = (const u32x4_t *)grad;
    a.state1 = (u32x2_t *)state1; a.state2 = (u32x2_t *)state2;
    a.scale1 = scale1; a.max1 = max1; a.scale2 = scale2; a.max2 = max2;
    a.n_threads = n / 8;
    a.codes8 = (u32x2_t *)codes; a.residual = (unsigned *)residual;
    a.qscales = (const unsigned short *)qscales;
    a.threads_per_row = K / 8;
    a.dequant_curve = lq_codec_dequant_params(dk1, db1, dk2, db2, dk3);
    a.quant_curve = lq_codec_quant_params(qk1, qb1, qk2, qb2, qk3);
    adam8_scalars(a, beta1, beta2, eps, step_size);
    const unsigned blocks = (unsigned)((a.n_threads + 255) / 256);
    if (block_elems == 2048)
        hipLaunchKernelGGL((adam8_update_kernel<2048, LATENT_W8>), dim3(blocks), dim3(256), 0, (hipStream_t)stream, a);
    else
        hipLaunchKernelGGL((adam8_update_kernel<128, LATENT_W8>), dim3(blocks), dim3(256), 0, (hipStream_t)stream, a);
    return lq_check_launch("lq_adam8_latent_w8_step");
}
