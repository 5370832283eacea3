// Kernel (1): single-pass stochastic-rounding latent requantizer for gfx950.
//
// A thread owns 4 consecutive 32-bit words of packed codes (32 consecutive k of
// one row): they never straddle a 128-element quantisation group, so scale,
// zero and the reciprocal of the scale are per-thread constants, the codes
// move as one 16-byte load and one 16-byte store, and the 8 Philox blocks of
// the thread have consecutive counters. The kernel is bound by vector-ALU
// instruction issue (Philox4x32-10 alone is ~10 instructions per element), so
// everything per element is kept to the minimum number of instructions.
//
// This translation unit is compiled with -ffp-contract=off: every rounding
// below is written out explicitly (fmaf where a fused operation is meant).
#include "lq_common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWordsPerThread = 4;  // 4 consecutive words = 32 elements of one quantisation group

// Exact restatement of the update rule for one element (any inputs).
__device__ __forceinline__ unsigned requant_elem_exact(unsigned q, float s, float z, float g, float lr, float u) {
    float d = lq_bf16_bits_to_f32(lq_f32_to_bf16_bits((float)q - z));
    float w = lq_bf16_bits_to_f32(lq_f32_to_bf16_bits(d * s));
    float t = fmaf(-lr, g, w);
    float v = t / s;
    v = v + z;
    v = v + u;
    float c = __builtin_amdgcn_fmed3f(v, 0.0f, 15.0f);  // NaN -> 0
    return (unsigned)c;                                  // trunc == floor on [0,15]
}

// One word (8 codes) on the fast path. Preconditions (checked per lane by the caller): z is an
// integer with |z| <= 240, so q - z is exact in bf16; 2^-40 <= s <= 2^40; r = RN(1/s).
// m[] holds the noise: in Philox mode the 24-bit integer draw as a float (u = m * 2^-24 is exact,
// so fmaf(m, 2^-24, a) == a + u with a single rounding, as the definition asks), else u itself.
template <bool kPhilox>
__device__ __forceinline__ unsigned requant_word_fast(unsigned codes, const unsigned gp[4], float s, float z, float r,
                                                      float lr, const float m[8]) {
    const float nzs = -(z * s);
    const unsigned lo4 = codes & 0x0F0F0F0Fu;         // odd elements
    const unsigned hi4 = (codes >> 4) & 0x0F0F0F0Fu;  // even elements
    // the codes as q/512, two per conversion; s512 = 512*s is exact (s <= 2^40 here)
    const lq_f32x2_t e0 = lq_nibbles_lo(hi4), e1 = lq_nibbles_hi(hi4), o0 = lq_nibbles_lo(lo4), o1 = lq_nibbles_hi(lo4);
    const float qf[8] = {e0[0], o0[0], e0[1], o0[1], e1[0], o1[0], e1[1], o1[1]};
    const float s512 = s * 512.0f;
    unsigned out = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        // (q - z) * s as fma(q/512, 512*s, -(z*s)): z*s and q*s are exact (8-bit significands), the sum has at
        // most 16 significant bits, so the fma returns (q - z) * s exactly; then the bf16 rounding of
        // the dequantised weight, two elements per v_cvt_pk_bf16_f32
        const unsigned pk = lq_pack_bf16(fmaf(qf[2 * i], s512, nzs), fmaf(qf[2 * i + 1], s512, nzs));
        float t[2] = {fmaf(-lr, lq_bf16_lo(gp[i]), lq_bf16_lo(pk)), fmaf(-lr, lq_bf16_hi(gp[i]), lq_bf16_hi(pk))};
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int j = 2 * i + h;
            // |t| >= 2^60 already saturates the code (|t/s| >= 2^20), so clamping t changes nothing but
            // keeps t*r finite; a NaN t becomes -2^60 and ends as code 0, as the definition asks.
            const float tc = __builtin_amdgcn_fmed3f(t[h], -0x1p60f, 0x1p60f);
            // correctly rounded tc/s from the correctly rounded reciprocal (Markstein):
            // q0 = t*r, e = t - q0*s (exact residual), q = q0 + e*r
            const float q0 = tc * r;
            const float e = fmaf(-q0, s, tc);
            float v = fmaf(e, r, q0);
            v = v + z;
            v = kPhilox ? fmaf(m[j], 0x1p-24f, v) : (v + m[j]);
            const float c = __builtin_amdgcn_fmed3f(v, 0.0f, 15.0f);
            out |= ((unsigned)c) << (4 * (j ^ 1));
        }
    }
    return out;
}

template <bool kPhilox>
__device__ __forceinline__ unsigned requant_word_exact(unsigned codes, const unsigned gp[4], float s, float z, float lr,
                                                       const float m[8]) {
    unsigned out = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float g = (j & 1) ? lq_bf16_hi(gp[j >> 1]) : lq_bf16_lo(gp[j >> 1]);
        const float u = kPhilox ? (m[j] * 0x1p-24f) : m[j];
        out |= requant_elem_exact(lq_code(codes, j), s, z, g, lr, u) << (4 * (j ^ 1));
    }
    return out;
}

// A thread owns 4 consecutive code words (16 bytes in, 16 bytes out, 64 bytes of gradient): they
// share one scale, zero and reciprocal, and their 8 Philox blocks have consecutive counters.
template <bool kPhilox>
__global__ __launch_bounds__(kThreads) void requant_kernel(const u32x4_t *__restrict__ codes_in,
                                                           u32x4_t *__restrict__ codes_out,
                                                           const unsigned short *__restrict__ scales,
                                                           const unsigned short *__restrict__ zeros,
                                                           const u32x4_t *__restrict__ grad, const f32x4_t *__restrict__ u,
                                                           float lr, long long n_chunks, unsigned long long seed,
                                                           unsigned long long offset) {
    const long long L = (long long)blockIdx.x * kThreads + threadIdx.x;
    if (L >= n_chunks) return;
    const u32x4_t codes = codes_in[L];
    u32x4_t g[kWordsPerThread];
#pragma unroll
    for (int i = 0; i < kWordsPerThread; ++i) g[i] = grad[L * kWordsPerThread + i];
    const float s = lq_bf16_bits_to_f32(scales[L >> 2]);
    const float z = lq_bf16_bits_to_f32(zeros[L >> 2]);

    // (a negative scale takes the exact path: the NaN handling of the clamp below assumes s > 0)
    const bool fast = (z == floorf(z)) && (fabsf(z) <= 240.0f) && (s >= 0x1p-40f) && (s <= 0x1p40f);
    const float r = 1.0f / s;  // correctly rounded (IEEE division)
    const unsigned long long cbase = offset + 8ull * (unsigned long long)L;  // element i uses block i/4

    u32x4_t out;
#pragma unroll
    for (int i = 0; i < kWordsPerThread; ++i) {
        float m[8];
        if (kPhilox) {
            const unsigned long long ca = cbase + 2 * i, cb = ca + 1;
            const lq_u4 ra = lq_philox4x32_10((unsigned)ca, (unsigned)(ca >> 32), 0u, 0u, (unsigned)seed, (unsigned)(seed >> 32));
            const lq_u4 rb = lq_philox4x32_10((unsigned)cb, (unsigned)(cb >> 32), 0u, 0u, (unsigned)seed, (unsigned)(seed >> 32));
            m[0] = (float)(ra.x >> 8); m[1] = (float)(ra.y >> 8); m[2] = (float)(ra.z >> 8); m[3] = (float)(ra.w >> 8);
            m[4] = (float)(rb.x >> 8); m[5] = (float)(rb.y >> 8); m[6] = (float)(rb.z >> 8); m[7] = (float)(rb.w >> 8);
        } else {
            const f32x4_t ua = u[(L * kWordsPerThread + i) * 2], ub = u[(L * kWordsPerThread + i) * 2 + 1];
            m[0] = ua[0]; m[1] = ua[1]; m[2] = ua[2]; m[3] = ua[3];
            m[4] = ub[0]; m[5] = ub[1]; m[6] = ub[2]; m[7] = ub[3];
        }
        const unsigned gp[4] = {g[i][0], g[i][1], g[i][2], g[i][3]};
        out[i] = fast ? requant_word_fast<kPhilox>(codes[i], gp, s, z, r, lr, m)
                      : requant_word_exact<kPhilox>(codes[i], gp, s, z, lr, m);
    }
    codes_out[L] = out;
}

__global__ __launch_bounds__(256) void philox_uniform_kernel(float *__restrict__ out, long long n,
                                                             unsigned long long seed, unsigned long long offset) {
    const long long q = (long long)blockIdx.x * 256 + threadIdx.x;  // one Philox block = 4 outputs
    const long long i = q * 4;
    if (i >= n) return;
    const unsigned long long c = offset + (unsigned long long)q;
    lq_u4 r = lq_philox4x32_10((unsigned)c, (unsigned)(c >> 32), 0u, 0u, (unsigned)seed, (unsigned)(seed >> 32));
    float v[4] = {(float)(r.x >> 8) * 0x1p-24f, (float)(r.y >> 8) * 0x1p-24f, (float)(r.z >> 8) * 0x1p-24f,
                  (float)(r.w >> 8) * 0x1p-24f};
    if (i + 4 <= n) {
        f32x4_t o = {v[0], v[1], v[2], v[3]};
        *reinterpret_cast<f32x4_t *>(out + i) = o;
    } else {
        for (int j = 0; j < 4 && i + j < n; ++j) out[i + j] = v[j];
    }
}

}  // namespace

extern "C" int lq_requant_sr(const void *codes_in, void *codes_out, const void *scales, const void *zeros,
                             const void *grad, float lr, int64_t N, int64_t K, int group, const float *u_or_null,
                             uint64_t philox_seed, uint64_t philox_offset, void *stream) {
    LQ_REQUIRE(codes_in && codes_out && scales && zeros && grad, "lq_requant_sr: null pointer argument");
    LQ_REQUIRE(group == LQ_GROUP, "lq_requant_sr: group must be %d, got %d", LQ_GROUP, group);
    LQ_REQUIRE(N > 0 && K > 0 && K % LQ_GROUP == 0, "lq_requant_sr: need N > 0 and K a positive multiple of %d (N=%lld K=%lld)",
               LQ_GROUP, (long long)N, (long long)K);
    LQ_REQUIRE(lq_aligned(codes_in, 16) && lq_aligned(codes_out, 16) && lq_aligned(grad, 16) && lq_aligned(scales, 2) &&
                   lq_aligned(zeros, 2) && (!u_or_null || lq_aligned(u_or_null, 16)),
               "lq_requant_sr: misaligned buffer (codes, grad and u need 16-byte alignment)");
    const long long n_chunks = (long long)N * K / (8 * kWordsPerThread);  // K % 128 == 0: no remainder
    const long long blocks = (n_chunks + kThreads - 1) / kThreads;
    LQ_REQUIRE(blocks <= 0x7FFFFFFFll, "lq_requant_sr: tensor too large");
    hipStream_t st = (hipStream_t)stream;
    if (u_or_null) {
        hipLaunchKernelGGL(requant_kernel<false>, dim3((unsigned)blocks), dim3(kThreads), 0, st,
                           (const u32x4_t *)codes_in, (u32x4_t *)codes_out, (const unsigned short *)scales,
                           (const unsigned short *)zeros, (const u32x4_t *)grad, (const f32x4_t *)u_or_null, lr, n_chunks,
                           (unsigned long long)philox_seed, (unsigned long long)philox_offset);
    } else {
        hipLaunchKernelGGL(requant_kernel<true>, dim3((unsigned)blocks), dim3(kThreads), 0, st,
                           (const u32x4_t *)codes_in, (u32x4_t *)codes_out, (const unsigned short *)scales,
                           (const unsigned short *)zeros, (const u32x4_t *)grad, (const f32x4_t *)nullptr, lr, n_chunks,
                           (unsigned long long)philox_seed, (unsigned long long)philox_offset);
    }
    return lq_check_launch("lq_requant_sr");
}

extern "C" int lq_philox_uniform(float *out, int64_t n, uint64_t philox_seed, uint64_t philox_offset, void *stream) {
    LQ_REQUIRE(out && n >= 0, "lq_philox_uniform: bad argument");
    LQ_REQUIRE(lq_aligned(out, 16), "lq_philox_uniform: out must be 16-byte aligned");
    if (n == 0) return LQ_OK;
    const long long blocks = ((n + 3) / 4 + 255) / 256;
    LQ_REQUIRE(blocks <= 0x7FFFFFFFll, "lq_philox_uniform: n too large");
    hipLaunchKernelGGL(philox_uniform_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, out,
                       (long long)n, (unsigned long long)philox_seed, (unsigned long long)philox_offset);
    return lq_check_launch("lq_philox_uniform");
}
