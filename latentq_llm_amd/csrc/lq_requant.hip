// Kernel (1): single-pass stochastic-rounding latent requantizer for gfx950.
//
// Update rule per element (s, z: the group's scale and zero; q: the code; g: the gradient):
//     w     = bf16(bf16(q - z) * s)                       the reference's dequantised weight
//     t     = fma(-lr, g, w)
//     y     = fma(t, (1/s) * 2^16, fma(z, 2^16, 0.5))     (t/s + z) in 16.16 fixed point, + 1/2
//     X     = y as a saturated unsigned integer            NaN and negatives -> 0, >= 2^32 -> 2^32 - 1
//     S     = min(X + a, 2^32 - 1)                          a: 16-bit uniform draw
//     code' = min(S >> 16, 15)                              = clamp(floor(x + (a + 1/2) 2^-16), 0, 15)
// i.e. the noise is uniform on the centred 2^-16 grid and the sum x + u is formed exactly in integer
// arithmetic. 1/s is the correctly rounded quotient, so every step is reproducible on a CPU.
//
// A thread owns 4 consecutive 32-bit words of packed codes (32 consecutive k of one row): they never
// straddle a 128-element quantisation group, so scale, zero and reciprocal are per-thread constants,
// the codes move as one 16-byte load and one 16-byte store, and the 4 Philox blocks of the thread
// (one per word: 8 draws of 16 bits) have consecutive counters. The kernel is bound by vector-ALU
// issue (about 16 instructions per element, 5 of them Philox4x32-10), so the tail is written to
// keep that count down:
//   - (q - z) * s comes from one fma on the code read as an FP8 number (exact for an integer zero,
//     see below) and is rounded to bf16 as the high half of a packed conversion whose low half is 0;
//   - the float -> fixed conversion saturates in hardware (v_cvt_u32_f32), the 16-bit draw is added
//     straight from its half of the Philox word with a saturating v_mad_u32_u16, and the eight codes
//     of a word are gathered from byte 2 of the eight sums with v_perm_b32.
// Threads whose (scale, zero) do not allow the one-fma dequantisation (non-integer zero, extreme
// scale) redo their 32 elements on a rolled cold path with the operations written out one by one.
//
// This translation unit is compiled with -ffp-contract=off: every rounding below is written out
// explicitly (fmaf where a fused operation is meant).
#include "lq_common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWordsPerThread = 4;  // 4 consecutive words = 32 elements of one quantisation group

// float -> uint32, truncating, saturating: NaN and negatives give 0, values >= 2^32 give 2^32 - 1
__device__ __forceinline__ unsigned cvt_u32_sat(float x) {
    unsigned r;
    asm("v_cvt_u32_f32 %0, %1" : "=v"(r) : "v"(x));
    return r;
}
// acc + (low or high 16 bits of word), saturating at 2^32 - 1
template <int HI>
__device__ __forceinline__ unsigned add_half_sat(unsigned word, unsigned acc) {
    unsigned r;
    if (HI) asm("v_mad_u32_u16 %0, %1, 1, %2 op_sel:[1,0,0,0] clamp" : "=v"(r) : "v"(word), "v"(acc));
    else asm("v_mad_u32_u16 %0, %1, 1, %2 clamp" : "=v"(r) : "v"(word), "v"(acc));
    return r;
}

// The definition, one operation per line (any inputs). a < 65536.
__device__ __forceinline__ unsigned requant_elem(unsigned q, float s, float z, float g, float lr, unsigned a) {
    const float d = lq_bf16_bits_to_f32(lq_f32_to_bf16_bits((float)q - z));
    const float w = lq_bf16_bits_to_f32(lq_f32_to_bf16_bits(d * s));
    const float t = fmaf(-lr, g, w);
    const float r16 = (1.0f / s) * 65536.0f;
    const float c16 = fmaf(z, 65536.0f, 0.5f);
    const unsigned S = add_half_sat<0>(a, cvt_u32_sat(fmaf(t, r16, c16)));
    const unsigned c = S >> 16;
    return c > 15u ? 15u : c;
}

// 16-bit draw from an injected uniform: floor(u * 2^16), NaN and negatives -> 0, u >= 1 -> 65535
__device__ __forceinline__ unsigned draw_of_uniform(float u) {
    const unsigned a = cvt_u32_sat(u * 65536.0f);
    return a > 65535u ? 65535u : a;
}

// Cold path: the 32 elements of thread L, one at a time, operands re-read from memory.
template <bool kPhilox>
__device__ __noinline__ void requant_thread_general(const unsigned *__restrict__ codes_in, unsigned *__restrict__ codes_out,
                                                    const unsigned short *__restrict__ grad, const float *__restrict__ u,
                                                    float s, float z, float lr, long long L, unsigned long long cbase,
                                                    unsigned k0, unsigned k1) {
#pragma unroll 1
    for (int i = 0; i < kWordsPerThread; ++i) {
        const long long wi = L * kWordsPerThread + i;
        const unsigned cw = codes_in[wi];
        unsigned aw[4] = {0u, 0u, 0u, 0u};
        if (kPhilox) {
            const unsigned long long c = cbase + i;
            const lq_u4 A = lq_philox4x32_10((unsigned)c, (unsigned)(c >> 32), 0u, 0u, k0, k1);
            aw[0] = A.x; aw[1] = A.y; aw[2] = A.z; aw[3] = A.w;
        }
        unsigned o = 0;
#pragma unroll 1
        for (int j = 0; j < 8; ++j) {
            const float g = lq_bf16_bits_to_f32(grad[wi * 8 + j]);
            const unsigned k = (unsigned)j >> 1;
            const unsigned word = k == 0 ? aw[0] : k == 1 ? aw[1] : k == 2 ? aw[2] : aw[3];
            const unsigned a = kPhilox ? ((word >> (16 * (j & 1))) & 0xFFFFu) : draw_of_uniform(u[wi * 8 + j]);
            o |= requant_elem(lq_code(cw, j), s, z, g, lr, a) << (4 * (j ^ 1));
        }
        codes_out[wi] = o;
    }
}

// kPre: the four Philox blocks are computed right after the loads are issued, before anything waits
// for them. Pays when the whole grid is resident at once (every wave then waits for its first bytes
// with nothing else to do); with several rounds of workgroups it only delays the loads of younger
// waves behind the arithmetic of older ones.
template <bool kPhilox, bool kPre>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(8))) void requant_kernel(
    const unsigned *__restrict__ codes_in, unsigned *__restrict__ codes_out, const unsigned short *__restrict__ scales,
    const unsigned short *__restrict__ zeros, const u32x4_t *__restrict__ grad, const f32x4_t *__restrict__ u, float lr,
    long long n_threads, unsigned long long seed, unsigned long long offset) {
    const long long L = (long long)blockIdx.x * kThreads + threadIdx.x;
    if (L >= n_threads) return;
    unsigned sbits = scales[L >> 2], zbits = zeros[L >> 2];
    const u32x4_t codes = *reinterpret_cast<const u32x4_t *>(codes_in + L * kWordsPerThread);
    u32x4_t g[kWordsPerThread];
#pragma unroll
    for (int i = 0; i < kWordsPerThread; ++i) g[i] = grad[L * kWordsPerThread + i];
    const unsigned long long cbase = offset + (unsigned long long)kWordsPerThread * (unsigned long long)L;  // word w uses block w
    const unsigned k0 = (unsigned)seed, k1 = (unsigned)(seed >> 32);

    unsigned aw[kWordsPerThread][4];
    if (kPhilox && kPre) {
#pragma unroll
        for (int i = 0; i < kWordsPerThread; ++i) {
            const unsigned long long c = cbase + i;
            const lq_u4 A = lq_philox4x32_10((unsigned)c, (unsigned)(c >> 32), 0u, 0u, k0, k1);
            aw[i][0] = A.x; aw[i][1] = A.y; aw[i][2] = A.z; aw[i][3] = A.w;
        }
        // the draws are complete here, and nothing below starts before this point
#pragma unroll
        for (int i = 0; i < kWordsPerThread; ++i) asm volatile("" : "+v"(aw[i][0]), "+v"(aw[i][1]), "+v"(aw[i][2]), "+v"(aw[i][3]));
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("" : "+v"(sbits), "+v"(zbits));
    }
    const float s = __uint_as_float(sbits << 16), z = __uint_as_float(zbits << 16);
    // One-fma dequantisation: z*s and q*s are exact in fp32 (8-bit significands) and for an integer zero
    // with |q - z| <= 255 the difference q - z is exact in bf16, so fma(q/512, 512*s, -(z*s)) is the
    // exact (q - z) * s and one rounding to bf16 gives what the two roundings of the definition give.
    const bool fast = (z == floorf(z)) && (fabsf(z) <= 240.0f) && (s >= 0x1p-100f) && (s <= 0x1p100f);
    const float r16 = (1.0f / s) * 65536.0f;
    const float nzs = -(z * s), s512 = s * 512.0f, c16 = fmaf(z, 65536.0f, 0.5f);

    u32x4_t out;
#pragma unroll
    for (int i = 0; i < kWordsPerThread; ++i) {
        if (kPhilox && !kPre) {
            const unsigned long long c = cbase + i;
            const lq_u4 A = lq_philox4x32_10((unsigned)c, (unsigned)(c >> 32), 0u, 0u, k0, k1);
            aw[i][0] = A.x; aw[i][1] = A.y; aw[i][2] = A.z; aw[i][3] = A.w;
        }
        if (!kPhilox) {
            const f32x4_t ua = u[(L * kWordsPerThread + i) * 2], ub = u[(L * kWordsPerThread + i) * 2 + 1];
            aw[i][0] = draw_of_uniform(ua[0]) | (draw_of_uniform(ua[1]) << 16);
            aw[i][1] = draw_of_uniform(ua[2]) | (draw_of_uniform(ua[3]) << 16);
            aw[i][2] = draw_of_uniform(ub[0]) | (draw_of_uniform(ub[1]) << 16);
            aw[i][3] = draw_of_uniform(ub[2]) | (draw_of_uniform(ub[3]) << 16);
        }
        const unsigned cw = codes[i];
        const unsigned lo4 = cw & 0x0F0F0F0Fu;         // odd elements
        const unsigned hi4 = (cw >> 4) & 0x0F0F0F0Fu;  // even elements
        // the codes as q/512, two per conversion
        const lq_f32x2_t e0 = lq_nibbles_lo(hi4), e1 = lq_nibbles_hi(hi4), o0 = lq_nibbles_lo(lo4), o1 = lq_nibbles_hi(lo4);
        const float qf[8] = {e0[0], o0[0], e0[1], o0[1], e1[0], o1[0], e1[1], o1[1]};
        unsigned S[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const unsigned gw = g[i][j >> 1];
            const float gv = (j & 1) ? lq_bf16_hi(gw) : lq_bf16_lo(gw);
            // bf16-rounded weight as a float: the high half of a packed pair whose low half is zero
            const float w = __uint_as_float(lq_pack_bf16(0.0f, fmaf(qf[j], s512, nzs)));
            const float t = fmaf(-lr, gv, w);
            const unsigned X = cvt_u32_sat(fmaf(t, r16, c16));
            const unsigned Sj = (j & 1) ? add_half_sat<1>(aw[i][j >> 1], X) : add_half_sat<0>(aw[i][j >> 1], X);
            S[j] = Sj < 0xFFFFFu ? Sj : 0xFFFFFu;  // code <= 15
        }
        // code of element j = byte 2 of S[j]; even elements go to the high nibbles, odd ones to the low
        const unsigned sel = 0x0C0C0602u;  // bytes (S1.b2, S0.b2, 0, 0) of v_perm_b32(S0, S1)
        const unsigned ev = (__builtin_amdgcn_perm(S[6], S[4], sel) << 16) | __builtin_amdgcn_perm(S[2], S[0], sel);
        const unsigned od = (__builtin_amdgcn_perm(S[7], S[5], sel) << 16) | __builtin_amdgcn_perm(S[3], S[1], sel);
        out[i] = (ev << 4) | od;
    }
    if (fast) *reinterpret_cast<u32x4_t *>(codes_out + L * kWordsPerThread) = out;
    else requant_thread_general<kPhilox>(codes_in, codes_out, (const unsigned short *)grad, (const float *)u, s, z, lr, L, cbase, k0, k1);
}

// out[i] = (a_i + 1/2) * 2^-16: the uniform the requantizer adds for element i
__global__ __launch_bounds__(256) void philox_uniform_kernel(float *__restrict__ out, long long n,
                                                             unsigned long long seed, unsigned long long offset) {
    const long long b = (long long)blockIdx.x * 256 + threadIdx.x;  // one Philox block = 8 outputs
    const long long i = b * 8;
    if (i >= n) return;
    const unsigned long long c = offset + (unsigned long long)b;
    const lq_u4 r = lq_philox4x32_10((unsigned)c, (unsigned)(c >> 32), 0u, 0u, (unsigned)seed, (unsigned)(seed >> 32));
    const unsigned w[4] = {r.x, r.y, r.z, r.w};
    float v[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = ((float)((w[j >> 1] >> (16 * (j & 1))) & 0xFFFFu) + 0.5f) * 0x1p-16f;
    if (i + 8 <= n) {
        *reinterpret_cast<f32x4_t *>(out + i) = f32x4_t{v[0], v[1], v[2], v[3]};
        *reinterpret_cast<f32x4_t *>(out + i + 4) = f32x4_t{v[4], v[5], v[6], v[7]};
    } else {
        for (int j = 0; j < 8 && i + j < n; ++j) out[i + j] = v[j];
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
    const long long n_threads = (long long)N * K / (8 * kWordsPerThread);  // K % 128 == 0: no remainder
    const long long blocks = (n_threads + kThreads - 1) / kThreads;
    LQ_REQUIRE(blocks <= 0x7FFFFFFFll, "lq_requant_sr: tensor too large");
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid((unsigned)blocks), block(kThreads);
    const unsigned *ci = (const unsigned *)codes_in;
    unsigned *co = (unsigned *)codes_out;
    const unsigned short *sc = (const unsigned short *)scales, *zr = (const unsigned short *)zeros;
    const u32x4_t *gr = (const u32x4_t *)grad;
    const unsigned long long seed = philox_seed, off = philox_offset;
    if (u_or_null) {
        hipLaunchKernelGGL((requant_kernel<false, false>), grid, block, 0, st, ci, co, sc, zr, gr, (const f32x4_t *)u_or_null, lr,
                           n_threads, seed, off);
    } else if (blocks <= 8ll * lq_device_cu_count()) {
        // one round: 8 workgroups of 4 waves per compute unit are resident at once
        hipLaunchKernelGGL((requant_kernel<true, true>), grid, block, 0, st, ci, co, sc, zr, gr, (const f32x4_t *)nullptr, lr,
                           n_threads, seed, off);
    } else {
        hipLaunchKernelGGL((requant_kernel<true, false>), grid, block, 0, st, ci, co, sc, zr, gr, (const f32x4_t *)nullptr, lr,
                           n_threads, seed, off);
    }
    return lq_check_launch("lq_requant_sr");
}

extern "C" int lq_philox_uniform(float *out, int64_t n, uint64_t philox_seed, uint64_t philox_offset, void *stream) {
    LQ_REQUIRE(out && n >= 0, "lq_philox_uniform: bad argument");
    LQ_REQUIRE(lq_aligned(out, 16), "lq_philox_uniform: out must be 16-byte aligned");
    if (n == 0) return LQ_OK;
    const long long blocks = ((n + 7) / 8 + 255) / 256;
    LQ_REQUIRE(blocks <= 0x7FFFFFFFll, "lq_philox_uniform: n too large");
    hipLaunchKernelGGL(philox_uniform_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, out,
                       (long long)n, (unsigned long long)philox_seed, (unsigned long long)philox_offset);
    return lq_check_launch("lq_philox_uniform");
}
