// Kernel (1): single-pass stochastic-rounding latent requantizer for gfx950.
//
// One 32-bit word of packed codes (8 consecutive k of one row) is the unit of
// work; a word never straddles a 128-element quantisation group, so scale,
// zero and the reciprocal of the scale are per-word constants. All loads of a
// thread's words are issued before any arithmetic so that a wave keeps
// 4 x (4 B codes + 16 B gradient) per lane in flight.
//
// This translation unit is compiled with -ffp-contract=off: every rounding
// below is written out explicitly (fmaf where a fused operation is meant).
#include "lq_common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWordsPerThread = 4;

struct WordIn {
    unsigned codes;
    u32x4_t g;  // 8 bf16 gradients, element j in half (j&1) of dword j/2
    unsigned short s_bits, z_bits;
};

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

template <bool kPhilox>
__device__ __forceinline__ unsigned requant_word(const WordIn &in, float lr, const float *u8,
                                                 unsigned c0a, unsigned c1a, unsigned c0b, unsigned c1b,
                                                 unsigned k0, unsigned k1) {
    const float s = lq_bf16_bits_to_f32(in.s_bits);
    const float z = lq_bf16_bits_to_f32(in.z_bits);

    float g[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        g[2 * i] = lq_bf16_lo(in.g[i]);
        g[2 * i + 1] = lq_bf16_hi(in.g[i]);
    }

    // Noise. Philox mode keeps the 24-bit integer draw as a float m; u = m * 2^-24 is exact,
    // so fmaf(m, 2^-24, a) == a + u with a single rounding, as the definition asks.
    float m[8];
    if (kPhilox) {
        lq_u4 ra = lq_philox4x32_10(c0a, c1a, 0u, 0u, k0, k1);
        lq_u4 rb = lq_philox4x32_10(c0b, c1b, 0u, 0u, k0, k1);
        m[0] = (float)(ra.x >> 8); m[1] = (float)(ra.y >> 8); m[2] = (float)(ra.z >> 8); m[3] = (float)(ra.w >> 8);
        m[4] = (float)(rb.x >> 8); m[5] = (float)(rb.y >> 8); m[6] = (float)(rb.z >> 8); m[7] = (float)(rb.w >> 8);
    } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) m[j] = u8[j];
    }

    // Codes as floats: low nibbles are the odd elements, high nibbles the even ones.
    const unsigned lo4 = in.codes & 0x0F0F0F0Fu;
    const unsigned hi4 = (in.codes >> 4) & 0x0F0F0F0Fu;
    float qf[8];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        qf[2 * b] = (float)((hi4 >> (8 * b)) & 0xFFu);
        qf[2 * b + 1] = (float)((lo4 >> (8 * b)) & 0xFFu);
    }

    // Fast path preconditions: q - z exact in bf16 (integer zero of small magnitude) and a
    // scale whose reciprocal, products and residuals stay far from overflow/underflow.
    const float az = fabsf(z), as = fabsf(s);
    bool fast = (z == floorf(z)) && (az <= 240.0f) && (as >= 0x1p-40f) && (as <= 0x1p40f);

    unsigned out = 0;
    float t[8];
    if (fast) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            float p = (qf[j] - z) * s;  // exact difference, one fp32 rounding (exact: <= 16 significant bits)
            t[j] = p;
        }
        // bf16 rounding of the dequantised weight, two elements per v_cvt_pk_bf16_f32.
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            unsigned pk = lq_pack_bf16(t[2 * i], t[2 * i + 1]);
            t[2 * i] = fmaf(-lr, g[2 * i], lq_bf16_lo(pk));
            t[2 * i + 1] = fmaf(-lr, g[2 * i + 1], lq_bf16_hi(pk));
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) fast = fast && (fabsf(t[j]) < 0x1p60f);
    }
    if (fast) {
        // Correctly rounded t/s from the correctly rounded reciprocal (Markstein): q0 = t*r,
        // e = t - q0*s (exact residual), q = q0 + e*r.
        const float r = 1.0f / s;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            float q0 = t[j] * r;
            float e = fmaf(-q0, s, t[j]);
            float v = fmaf(e, r, q0);
            v = v + z;
            v = kPhilox ? fmaf(m[j], 0x1p-24f, v) : (v + m[j]);
            float c = __builtin_amdgcn_fmed3f(v, 0.0f, 15.0f);
            out |= ((unsigned)c) << (4 * (j ^ 1));
        }
    } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            float u = kPhilox ? (m[j] * 0x1p-24f) : m[j];
            out |= requant_elem_exact((unsigned)qf[j], s, z, g[j], lr, u) << (4 * (j ^ 1));
        }
    }
    return out;
}

template <bool kPhilox>
__global__ __launch_bounds__(kThreads) void requant_kernel(const unsigned *__restrict__ codes_in,
                                                           unsigned *__restrict__ codes_out,
                                                           const unsigned short *__restrict__ scales,
                                                           const unsigned short *__restrict__ zeros,
                                                           const u32x4_t *__restrict__ grad, const float *__restrict__ u,
                                                           float lr, long long n_words, unsigned long long seed,
                                                           unsigned long long offset) {
    const long long base = (long long)blockIdx.x * (kThreads * kWordsPerThread) + threadIdx.x;
    WordIn in[kWordsPerThread];
#pragma unroll
    for (int i = 0; i < kWordsPerThread; ++i) {
        const long long w = base + (long long)i * kThreads;
        if (w < n_words) {
            in[i].codes = codes_in[w];
            in[i].g = grad[w];
            in[i].s_bits = scales[w >> 4];
            in[i].z_bits = zeros[w >> 4];
        }
    }
#pragma unroll
    for (int i = 0; i < kWordsPerThread; ++i) {
        const long long w = base + (long long)i * kThreads;
        if (w < n_words) {
            float u8[8];
            unsigned c0a = 0, c1a = 0, c0b = 0, c1b = 0;
            if (kPhilox) {
                const unsigned long long ca = offset + 2ull * (unsigned long long)w;
                const unsigned long long cb = ca + 1ull;
                c0a = (unsigned)ca; c1a = (unsigned)(ca >> 32);
                c0b = (unsigned)cb; c1b = (unsigned)(cb >> 32);
            } else {
                const f32x4_t *up = reinterpret_cast<const f32x4_t *>(u) + 2 * w;
                f32x4_t ua = up[0], ub = up[1];
                u8[0] = ua[0]; u8[1] = ua[1]; u8[2] = ua[2]; u8[3] = ua[3];
                u8[4] = ub[0]; u8[5] = ub[1]; u8[6] = ub[2]; u8[7] = ub[3];
            }
            codes_out[w] = requant_word<kPhilox>(in[i], lr, u8, c0a, c1a, c0b, c1b, (unsigned)seed,
                                                 (unsigned)(seed >> 32));
        }
    }
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
    LQ_REQUIRE(lq_aligned(codes_in, 4) && lq_aligned(codes_out, 4) && lq_aligned(grad, 16) && lq_aligned(scales, 2) &&
                   lq_aligned(zeros, 2) && (!u_or_null || lq_aligned(u_or_null, 16)),
               "lq_requant_sr: misaligned buffer (codes 4 B, grad 16 B, u 16 B)");
    const long long n_words = (long long)N * K / 8;
    const long long per_block = kThreads * kWordsPerThread;
    const long long blocks = (n_words + per_block - 1) / per_block;
    LQ_REQUIRE(blocks <= 0x7FFFFFFFll, "lq_requant_sr: tensor too large");
    hipStream_t st = (hipStream_t)stream;
    if (u_or_null) {
        hipLaunchKernelGGL(requant_kernel<false>, dim3((unsigned)blocks), dim3(kThreads), 0, st,
                           (const unsigned *)codes_in, (unsigned *)codes_out, (const unsigned short *)scales,
                           (const unsigned short *)zeros, (const u32x4_t *)grad, u_or_null, lr, n_words,
                           (unsigned long long)philox_seed, (unsigned long long)philox_offset);
    } else {
        hipLaunchKernelGGL(requant_kernel<true>, dim3((unsigned)blocks), dim3(kThreads), 0, st,
                           (const unsigned *)codes_in, (unsigned *)codes_out, (const unsigned short *)scales,
                           (const unsigned short *)zeros, (const u32x4_t *)grad, (const float *)nullptr, lr, n_words,
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
