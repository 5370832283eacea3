// 8-bit gradient accumulator of the reference's GradientQTensor (utils/quant.py:846-922) as one pass
// over the bf16 weight gradient: per-row scale, stochastic rounding to int8, and the accumulate form
// quant(dequant() + dW). Every tensor operation of the reference's chain keeps its bf16 rounding:
//   set:  vmax = bf16(4 * max_k |dW[n,k]|);  scale[n] = bf16(max(vmax, bf16(1e-5)) * (1/127))
//         q = clamp(rint(bf16(bf16(dW / scale) + noise)), -128, 127)
//   add:  x = bf16(bf16(q * scale) + dW);   q = clamp(rint(bf16(bf16(x / scale) + noise)), -128, 127)
// (a division by a Python scalar is a multiplication by its fp32 reciprocal inside the tensor
// library's GPU kernels; tensor / tensor is the IEEE quotient). The reference draws the noise with
// uniform_(-0.5, 0.5); here it is either injected (bf16) or (2b - 255) / 512 for the 8-bit Philox
// draw b of the element: byte i & 3 of word (i >> 2) & 3 of Philox4x32-10(counter = offset + i / 16,
// key = seed), i the flat element index. The 256 values are bf16 numbers, symmetric about zero.
//
// A row belongs to one workgroup (to 64, 128 or 256 of its threads): the row's absolute maximum needs the whole
// row before its first element can be quantised; rows of up to 12 288 elements stay in registers in between,
// longer ones are read a second time (from L2).
#include "lq_common.h"
#include "lq_gradq8_math.h"

namespace {

// Largest magnitude as a bit pattern: magnitudes of bf16 numbers order like unsigned integers and every NaN pattern
// lies above infinity, so that a NaN anywhere in the row ends up in the maximum (as the tensor library's amax does).
__device__ __forceinline__ unsigned absmax8(const u32x4_t v, unsigned m) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const unsigned a = v[j] & 0x7FFF7FFFu;
        const unsigned lo = a & 0xFFFFu, hi = a >> 16;
        m = m > lo ? m : lo;
        m = m > hi ? m : hi;
    }
    return m;
}

// T threads per row (64, 128 or 256: short rows get a wave or two instead of a mostly idle workgroup, 256 / T rows
// per workgroup); a thread takes 16 consecutive elements per step of 16 T. kPieces > 0: the row has at most
// kPieces * 16 T elements and a thread keeps its pieces in registers between the maximum and the quantisation;
// 0: any K, the row is read a second time (from L2).
template <bool kPhilox, bool kAcc, int kPieces, int T>
__global__ __launch_bounds__(256) void gradq8_kernel(const unsigned short *__restrict__ dw, signed char *__restrict__ q,
                                                     unsigned short *__restrict__ scale, const unsigned short *__restrict__ noise,
                                                     long long N, long long K, unsigned long long seed,
                                                     unsigned long long offset) {
    constexpr int R = 256 / T;      // rows per workgroup
    constexpr int STEP = 16 * T;    // elements of a row the row's threads take per piece
    __shared__ unsigned red[4];
    const int tid = threadIdx.x % T;
    const long long n_raw = (long long)blockIdx.x * R + threadIdx.x / T;
    const bool live = n_raw < N;    // rows past the end still take part in the barrier
    const long long n = live ? n_raw : N - 1;
    const unsigned short *row = dw + n * K;
    const u32x4_t zero4 = {0u, 0u, 0u, 0u};
    constexpr int kHeld = kPieces > 0 ? kPieces : 1;
    u32x4_t h0[kHeld], h1[kHeld], old[kHeld], z0[kHeld], z1[kHeld];
    if (kPieces > 0) {
#pragma unroll
        for (int i = 0; i < kPieces; ++i) {
            const long long k = (long long)tid * 16 + (long long)i * STEP;
            h0[i] = h1[i] = old[i] = z0[i] = z1[i] = zero4;
            if (k < K) {
                h0[i] = *reinterpret_cast<const u32x4_t *>(row + k);
                h1[i] = *reinterpret_cast<const u32x4_t *>(row + k + 8);
                if (kAcc) old[i] = *reinterpret_cast<const u32x4_t *>(q + n * K + k);
                if (!kPhilox) {
                    z0[i] = *reinterpret_cast<const u32x4_t *>(noise + n * K + k);
                    z1[i] = *reinterpret_cast<const u32x4_t *>(noise + n * K + k + 8);
                }
            }
        }
    }
    float s;
    if (!kAcc) {
        unsigned mb = 0u;
        if (kPieces > 0) {
#pragma unroll
            for (int i = 0; i < kPieces; ++i) mb = absmax8(h1[i], absmax8(h0[i], mb));
        } else {
            for (long long k = (long long)tid * 16; k < K; k += STEP)
                mb = absmax8(*reinterpret_cast<const u32x4_t *>(row + k + 8), absmax8(*reinterpret_cast<const u32x4_t *>(row + k), mb));
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const unsigned other = (unsigned)__shfl_xor((int)mb, o);
            mb = mb > other ? mb : other;
        }
        if constexpr (T > 64) {
            // waves of one row are neighbours: wave w belongs to row group w / (T / 64)
            const int wave = threadIdx.x >> 6;
            if ((threadIdx.x & 63) == 0) red[wave] = mb;
            __syncthreads();
            if constexpr (T == 256) {
                const unsigned a = red[0] > red[1] ? red[0] : red[1], b = red[2] > red[3] ? red[2] : red[3];
                mb = a > b ? a : b;
            } else {
                mb = red[wave & ~1] > red[wave | 1] ? red[wave & ~1] : red[wave | 1];
            }
        }
        const float m = __uint_as_float(mb << 16);
        const float vmax = bf16r(m * 4.0f);
        const float lo = bf16r(1e-5f);
        // a NaN row maximum stays NaN through the floor (torch.clamp keeps it): the row's scale and with it the
        // dequantised gradient are NaN, as in the reference
        s = vmax != vmax ? vmax : bf16r(fmaxf(vmax, lo) * (1.0f / 127.0f));
        if (tid == 0 && live) scale[n] = lq_f32_to_bf16_bits(s);
    } else {
        s = lq_bf16_bits_to_f32(scale[n]);
    }
    if (!live) return;
    // the scale is the same for a whole wave (a wave never spans two rows), so this branch does not diverge
    const bool fast = __builtin_amdgcn_readfirstlane((int)(s >= 0x1p-40f && s <= 0x1p40f)) != 0;
    const float r = 1.0f / s;
    if (kPieces > 0) {
#pragma unroll
        for (int i = 0; i < kPieces; ++i) {
            const long long k = (long long)tid * 16 + (long long)i * STEP;
            if (k < K) {
                const long long e0 = n * K + k;
                const unsigned long long c = offset + (unsigned long long)(e0 >> 4);
                const u32x4_t o = fast ? quant16<kPhilox, kAcc, true>(h0[i], h1[i], old[i], z0[i], z1[i], s, r, c, seed)
                                       : quant16<kPhilox, kAcc, false>(h0[i], h1[i], old[i], z0[i], z1[i], s, r, c, seed);
                *reinterpret_cast<u32x4_t *>(q + e0) = o;
            }
        }
    } else {
        for (long long k = (long long)tid * 16; k < K; k += STEP) {
            const long long e0 = n * K + k;
            const u32x4_t v0 = *reinterpret_cast<const u32x4_t *>(row + k);
            const u32x4_t v1 = *reinterpret_cast<const u32x4_t *>(row + k + 8);
            u32x4_t ol = zero4, a0 = zero4, a1 = zero4;
            if (kAcc) ol = *reinterpret_cast<const u32x4_t *>(q + e0);
            if (!kPhilox) {
                a0 = *reinterpret_cast<const u32x4_t *>(noise + e0);
                a1 = *reinterpret_cast<const u32x4_t *>(noise + e0 + 8);
            }
            const unsigned long long c = offset + (unsigned long long)(e0 >> 4);
            const u32x4_t o = fast ? quant16<kPhilox, kAcc, true>(v0, v1, ol, a0, a1, s, r, c, seed)
                                   : quant16<kPhilox, kAcc, false>(v0, v1, ol, a0, a1, s, r, c, seed);
            *reinterpret_cast<u32x4_t *>(q + e0) = o;
        }
    }
}

template <bool kPhilox, bool kAcc>
void launch_gradq8(const void *dw, int8_t *q, void *scale, const void *noise, int64_t N, int64_t K, uint64_t seed,
                   uint64_t offset, hipStream_t st) {
#define LQ_GRADQ8_LAUNCH(P, T)                                                                                        \
    hipLaunchKernelGGL((gradq8_kernel<kPhilox, kAcc, P, T>), dim3((unsigned)((N + 256 / T - 1) / (256 / T))), dim3(256), 0, \
                       st, (const unsigned short *)dw, (signed char *)q, (unsigned short *)scale,                     \
                       (const unsigned short *)noise, (long long)N, (long long)K, (unsigned long long)seed,           \
                       (unsigned long long)offset)
    if (K <= 1024) LQ_GRADQ8_LAUNCH(1, 64);
    else if (K <= 2048) LQ_GRADQ8_LAUNCH(1, 128);
    else if (K <= 4096) LQ_GRADQ8_LAUNCH(1, 256);
    else if (K <= 3 * 4096) LQ_GRADQ8_LAUNCH(3, 256);
    else LQ_GRADQ8_LAUNCH(0, 256);
#undef LQ_GRADQ8_LAUNCH
}

}  // namespace

extern "C" int lq_gradq8_quant(const void *dw, int8_t *q_inout, void *scale_inout, int accumulate, int64_t N, int64_t K,
                               const void *noise_or_null, uint64_t philox_seed, uint64_t philox_offset, void *stream) {
    LQ_REQUIRE(dw && q_inout && scale_inout, "lq_gradq8_quant: null pointer argument");
    LQ_REQUIRE(N > 0 && K > 0 && K % 16 == 0 && N < (1ll << 31), "lq_gradq8_quant: need N > 0 and K a positive multiple of 16 (N=%lld K=%lld)",
               (long long)N, (long long)K);
    LQ_REQUIRE(lq_aligned(dw, 16) && lq_aligned(q_inout, 16) && lq_aligned(scale_inout, 2) &&
                   (!noise_or_null || lq_aligned(noise_or_null, 16)),
               "lq_gradq8_quant: dw, q and noise need 16-byte alignment");
    hipStream_t st = (hipStream_t)stream;
    if (noise_or_null) {
        if (accumulate) launch_gradq8<false, true>(dw, q_inout, scale_inout, noise_or_null, N, K, 0, 0, st);
        else launch_gradq8<false, false>(dw, q_inout, scale_inout, noise_or_null, N, K, 0, 0, st);
    } else {
        if (accumulate) launch_gradq8<true, true>(dw, q_inout, scale_inout, nullptr, N, K, philox_seed, philox_offset, st);
        else launch_gradq8<true, false>(dw, q_inout, scale_inout, nullptr, N, K, philox_seed, philox_offset, st);
    }
    return lq_check_launch("lq_gradq8_quant");
}
