// 8-bit gradient accumulator of the reference's GradientQTensor (utils/quant.py:846-922) as one pass
// over the bf16 weight gradient: per-row scale, stochastic rounding to int8, and the accumulate form
// quant(dequant() + dW). Every tensor operation of the reference's chain keeps its bf16 rounding:
//   set:  vmax = bf16(4 * max_k |dW[n,k]|);  scale[n] = bf16(max(vmax, bf16(1e-5)) * (1/127))
//         q = clamp(rint(bf16(bf16(dW / scale) + noise)), -128, 127)
//   add:  x = bf16(bf16(q * scale) + dW);   q = clamp(rint(bf16(bf16(x / scale) + noise)), -128, 127)
// (a division by a Python scalar is a multiplication by its fp32 reciprocal inside the tensor
// library's GPU kernels; tensor / tensor is the IEEE quotient). The reference draws the noise with
// uniform_(-0.5, 0.5); here it is either injected (bf16) or bf16((a + 1/2) * 2^-16 - 1/2) for the
// 16-bit Philox draw a of the element (the requantizer's stream: one block per 8 elements).
//
// One workgroup per row: the row's absolute maximum needs the whole row before its first element can
// be quantised, and a second read of an 8-22 KB row by the workgroup that just read it stays in L2.
#include "lq_common.h"

namespace {

__device__ __forceinline__ float bf16r(float v) { return lq_bf16_bits_to_f32(lq_f32_to_bf16_bits(v)); }

// IEEE x / s from the correctly rounded reciprocal r = RN(1/s) when fast (2^-40 <= s <= 2^40): q0 = x r,
// e = x - q0 s exactly, q = q0 + e r; |x| is clamped to 2^60 first (the quotient then saturates the
// int8 range anyway), a NaN takes the true division.
__device__ __forceinline__ float div_by_scale(float x, float s, float r, bool fast) {
    if (fast && x == x) {
        const float xc = __builtin_amdgcn_fmed3f(x, -0x1p60f, 0x1p60f);
        const float q0 = xc * r;
        return fmaf(fmaf(-q0, s, xc), r, q0);
    }
    return x / s;
}

template <bool kPhilox>
__global__ __launch_bounds__(256) void gradq8_kernel(const unsigned short *__restrict__ dw, signed char *__restrict__ q,
                                                     unsigned short *__restrict__ scale, const unsigned short *__restrict__ noise,
                                                     int accumulate, long long K, unsigned long long seed,
                                                     unsigned long long offset) {
    __shared__ float red[4];
    const long long n = blockIdx.x;
    const unsigned short *row = dw + n * K;
    const int tid = threadIdx.x;
    float s;
    if (!accumulate) {
        float m = 0.0f;
        for (long long k = (long long)tid * 8; k < K; k += 256 * 8) {
            const u32x4_t v = *reinterpret_cast<const u32x4_t *>(row + k);
#pragma unroll
            for (int j = 0; j < 4; ++j) m = fmaxf(m, fmaxf(fabsf(lq_bf16_lo(v[j])), fabsf(lq_bf16_hi(v[j]))));
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
        if ((tid & 63) == 0) red[tid >> 6] = m;
        __syncthreads();
        m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        const float vmax = bf16r(m * 4.0f);
        const float lo = bf16r(1e-5f);
        s = bf16r(fmaxf(vmax, lo) * (1.0f / 127.0f));
        if (tid == 0) scale[n] = lq_f32_to_bf16_bits(s);
    } else {
        s = lq_bf16_bits_to_f32(scale[n]);
    }
    const bool fast = s >= 0x1p-40f && s <= 0x1p40f;
    const float r = 1.0f / s;
    for (long long k = (long long)tid * 8; k < K; k += 256 * 8) {
        const long long e0 = n * K + k;  // flat index of the first of 8 elements
        const u32x4_t v = *reinterpret_cast<const u32x4_t *>(row + k);
        float x[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) x[j] = (j & 1) ? lq_bf16_hi(v[j >> 1]) : lq_bf16_lo(v[j >> 1]);
        if (accumulate) {
            const u32x2_t old = *reinterpret_cast<const u32x2_t *>(q + e0);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int qi = (int)(signed char)((old[j >> 2] >> (8 * (j & 3))) & 0xFFu);
                x[j] = bf16r(bf16r((float)qi * s) + x[j]);
            }
        }
        float nz[8];
        if (kPhilox) {
            const unsigned long long c = offset + (unsigned long long)(e0 >> 3);
            const lq_u4 A = lq_philox4x32_10((unsigned)c, (unsigned)(c >> 32), 0u, 0u, (unsigned)seed, (unsigned)(seed >> 32));
            const unsigned w[4] = {A.x, A.y, A.z, A.w};
#pragma unroll
            for (int j = 0; j < 8; ++j)
                nz[j] = bf16r(((float)((w[j >> 1] >> (16 * (j & 1))) & 0xFFFFu) + 0.5f) * 0x1p-16f - 0.5f);
        } else {
            const u32x4_t nv = *reinterpret_cast<const u32x4_t *>(noise + e0);
#pragma unroll
            for (int j = 0; j < 8; ++j) nz[j] = (j & 1) ? lq_bf16_hi(nv[j >> 1]) : lq_bf16_lo(nv[j >> 1]);
        }
        unsigned o[2] = {0u, 0u};
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float y = bf16r(bf16r(div_by_scale(x[j], s, r, fast)) + nz[j]);
            const float c = __builtin_amdgcn_fmed3f(rintf(y), -128.0f, 127.0f);  // NaN -> -128
            o[j >> 2] |= ((unsigned)(int)c & 0xFFu) << (8 * (j & 3));
        }
        *reinterpret_cast<u32x2_t *>(q + e0) = u32x2_t{o[0], o[1]};
    }
}

}  // namespace

extern "C" int lq_gradq8_quant(const void *dw, int8_t *q_inout, void *scale_inout, int accumulate, int64_t N, int64_t K,
                               const void *noise_or_null, uint64_t philox_seed, uint64_t philox_offset, void *stream) {
    LQ_REQUIRE(dw && q_inout && scale_inout, "lq_gradq8_quant: null pointer argument");
    LQ_REQUIRE(N > 0 && K > 0 && K % 8 == 0 && N < (1ll << 31), "lq_gradq8_quant: need N > 0 and K a positive multiple of 8 (N=%lld K=%lld)",
               (long long)N, (long long)K);
    LQ_REQUIRE(lq_aligned(dw, 16) && lq_aligned(q_inout, 8) && lq_aligned(scale_inout, 2) &&
                   (!noise_or_null || lq_aligned(noise_or_null, 16)),
               "lq_gradq8_quant: dw and noise need 16-byte alignment, q 8-byte alignment");
    const dim3 grid((unsigned)N), block(256);
    if (noise_or_null)
        hipLaunchKernelGGL((gradq8_kernel<false>), grid, block, 0, (hipStream_t)stream, (const unsigned short *)dw,
                           (signed char *)q_inout, (unsigned short *)scale_inout, (const unsigned short *)noise_or_null,
                           accumulate, (long long)K, 0ull, 0ull);
    else
        hipLaunchKernelGGL((gradq8_kernel<true>), grid, block, 0, (hipStream_t)stream, (const unsigned short *)dw,
                           (signed char *)q_inout, (unsigned short *)scale_inout, (const unsigned short *)nullptr, accumulate,
                           (long long)K, (unsigned long long)philox_seed, (unsigned long long)philox_offset);
    return lq_check_launch("lq_gradq8_quant");
}
