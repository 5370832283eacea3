// Kernel (2b): A16W4 GEMV for decode-sized M (1..16 tokens) on gfx950.
//
// The weight matrix is streamed from HBM exactly once. A workgroup owns 16 consecutive
// weight rows (output features); its waves split the K dimension by quantisation group
// and combine their partial sums through LDS. Inside a wave the contraction runs on the
// 16x16x32 bf16 MFMA with the (zero-padded) token block as the 16-row operand, because at
// 0.5 byte per weight even one fp32 FMA per weight would outrun the vector ALUs before HBM.
//
// Per group g (128 k) and weight row n the kernel uses
//     sum_k x[m,k] * (q[n,k] - z) * s  =  s * ( P[m,n] - (128 + z) * S[m] )
// with P = sum_k x[m,k] * (128 + q[n,k]) and S = sum_k x[m,k], both accumulated by MFMA:
// the code nibbles become the bf16 numbers 128+q by one AND-OR (bit pattern 0x4300 | q),
// so unpacking costs < 1 VALU operation per weight. The scale is applied in fp32 to the
// per-group sums, i.e. weights are NOT rounded to bf16 first (slightly more accurate than
// the dequantise-then-multiply path).
#include "lq_common.h"

namespace {

constexpr int kUnroll = 4;  // groups in flight per wave

// k-slot order produced by the AND-OR unpack of one code word: slots (2i, 2i+1) of dword i
// hold codes (1,5), (0,4), (3,7), (2,6). The activation fragment is permuted to match.
__device__ __forceinline__ void unpack_word_128q(unsigned w, unsigned o[4]) {
    o[0] = (w & 0x000F000Fu) | 0x43004300u;
    o[1] = ((w >> 4) & 0x000F000Fu) | 0x43004300u;
    o[2] = ((w >> 8) & 0x000F000Fu) | 0x43004300u;
    o[3] = ((w >> 12) & 0x000F000Fu) | 0x43004300u;
}
__device__ __forceinline__ void permute_x(const u32x4_t &d, unsigned a[4]) {
    a[0] = __builtin_amdgcn_perm(d[2], d[0], 0x07060302u);  // (x1, x5)
    a[1] = __builtin_amdgcn_perm(d[2], d[0], 0x05040100u);  // (x0, x4)
    a[2] = __builtin_amdgcn_perm(d[3], d[1], 0x07060302u);  // (x3, x7)
    a[3] = __builtin_amdgcn_perm(d[3], d[1], 0x05040100u);  // (x2, x6)
}

template <int WAVES>
__global__ __launch_bounds__(64 * WAVES) void gemv_kernel(const unsigned short *__restrict__ x,
                                                          const unsigned char *__restrict__ codes,
                                                          const unsigned short *__restrict__ scales,
                                                          const unsigned short *__restrict__ zeros,
                                                          const unsigned short *__restrict__ bias,
                                                          unsigned short *__restrict__ y, int M, int N, int K) {
    __shared__ float red[WAVES][4][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = lane & 15, kq = lane >> 4;
    const int row = blockIdx.x * 16 + n;  // weight row of this lane's B fragment
    const int G = K / LQ_GROUP;
    const bool has_x = n < M;  // as an A-fragment lane, `n` is the token index

    const unsigned char *wrow = codes + (long long)row * (K / 2) + kq * 16;
    const unsigned short *xrow = x + (long long)(has_x ? n : 0) * K + kq * 32;
    const unsigned short *srow = scales + (long long)row * G;
    const unsigned short *zrow = zeros + (long long)row * G;

    const u32x4_t ones = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
    f32x4_t acc = {0.f, 0.f, 0.f, 0.f};

    for (int g0 = wave * kUnroll; g0 < G; g0 += WAVES * kUnroll) {
        u32x4_t wv[kUnroll];
        u32x4_t xv[kUnroll][4];
        unsigned short sb[kUnroll], zb[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const int g = g0 + u;
            if (g < G) {
                wv[u] = *reinterpret_cast<const u32x4_t *>(wrow + g * 64);
                sb[u] = srow[g];
                zb[u] = zrow[g];
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    if (has_x) {
                        xv[u][t] = *reinterpret_cast<const u32x4_t *>(xrow + g * LQ_GROUP + t * 8);
                    } else {
                        xv[u][t] = u32x4_t{0u, 0u, 0u, 0u};
                    }
                }
            }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const int g = g0 + u;
            if (g < G) {
                f32x4_t P = {0.f, 0.f, 0.f, 0.f}, S = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    unsigned b[4], a[4];
                    unpack_word_128q(wv[u][t], b);
                    permute_x(xv[u][t], a);
                    const u32x4_t av = {a[0], a[1], a[2], a[3]};
                    const u32x4_t bv = {b[0], b[1], b[2], b[3]};
                    P = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, av),
                                                                __builtin_bit_cast(bf16x8_t, bv), P, 0, 0, 0);
                    S = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, av),
                                                                __builtin_bit_cast(bf16x8_t, ones), S, 0, 0, 0);
                }
                const float s = lq_bf16_bits_to_f32(sb[u]);
                const float zz = 128.0f + lq_bf16_bits_to_f32(zb[u]);
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[r] = fmaf(s, fmaf(-zz, S[r], P[r]), acc[r]);
            }
        }
    }

#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave][r][lane] = acc[r];
    __syncthreads();
    if (wave == 0) {
        // lane holds D[m = 4*kq + r][n]
        const float b = bias ? lq_bf16_bits_to_f32(bias[row]) : 0.0f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) v += red[w][r][lane];
            const int m = 4 * kq + r;
            if (m < M) y[(long long)m * N + row] = lq_f32_to_bf16_bits(v + b);
        }
    }
}

}  // namespace

int lq_gemv_a16w4_launch(const void *x, const void *codes, const void *scales, const void *zeros, const void *bias,
                         void *y, int M, int N, int K, hipStream_t st) {
    // N % 16 == 0 and K % 128 == 0 are guaranteed by the caller.
    const int blocks = N / 16;
    const int G = K / LQ_GROUP;
    // Enough waves to keep every SIMD busy, but at least one batch of groups per wave.
    int waves = 4;
    while (waves < 16 && (long long)blocks * waves < 4096 && G >= waves * 2 * kUnroll) waves *= 2;
#define LQ_GEMV_LAUNCH(W)                                                                                         \
    hipLaunchKernelGGL(gemv_kernel<W>, dim3(blocks), dim3(64 * W), 0, st, (const unsigned short *)x,               \
                       (const unsigned char *)codes, (const unsigned short *)scales, (const unsigned short *)zeros, \
                       (const unsigned short *)bias, (unsigned short *)y, M, N, K)
    if (waves == 4) LQ_GEMV_LAUNCH(4);
    else if (waves == 8) LQ_GEMV_LAUNCH(8);
    else LQ_GEMV_LAUNCH(16);
#undef LQ_GEMV_LAUNCH
    return lq_check_launch("lq_a16w4_fwd(gemv)");
}
