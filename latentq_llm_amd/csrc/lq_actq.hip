// Activation quantisers in front of the int8 GEMM (bf16 -> int8 + the per-row scales its epilogue reads):
//   lq_act_quant_i8           per-tensor, clamp value given (a device scalar)
//   lq_act_quant_i8_dynamic   per-tensor, clamp value = the tensor's own maximum (two launches, no host sync)
//   lq_act_quant_i8_per_token one scale per token row from the row's absolute maximum (one pass over HBM)
// and, for the backward passes, lq_act_dequant_i8 (int8 -> bf16) and lq_act_fake_quant (bf16 -> bf16 on the int8 grid)
#include "lq_common.h"

namespace {

// x8 = clamp(rne(bf16(bf16(x * 127) / clampv)), -128, 127); 8 elements per thread.
// The clamp value is the maximum of a bf16 tensor in every use the reference makes of it, i.e. a bf16 number;
// the quotient of two bf16 numbers keeps 2^-17 (relative) from every bf16 rounding tie, so bf16(a / c) is
// bf16(a * RN(1/c)) (kFast: c has no bits below bf16's and 2^-40 <= |c| <= 2^40; decided once per launch's
// uniform value, any other clamp value takes the division). clamp(rint(q), -128, 127) is sat_u8(rne(q + 128)) - 128:
// q is a bf16 number, so the sum is exact wherever it matters. A NaN becomes 0 (what the tensor library's
// float -> int8 conversion makes of it); the byte conversion would make it -128, so 8 inputs with a NaN among
// them take the slow form.
template <bool kFast>
__device__ __forceinline__ u32x2_t act_quant8(const u32x4_t v, float c, float r) {
    unsigned w[2] = {0u, 0u};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float f = (j & 1) ? lq_bf16_hi(v[j >> 1]) : lq_bf16_lo(v[j >> 1]);
        const float a = lq_bf16_bits_to_f32(lq_f32_to_bf16_bits(f * 127.0f));
        if (kFast) {
            const float q = lq_bf16_bits_to_f32(lq_f32_to_bf16_bits(a * r)) + 128.0f;
            switch (j & 3) {
                case 0: w[j >> 2] = act_cvt_pk_u8<0>(q, w[j >> 2]); break;
                case 1: w[j >> 2] = act_cvt_pk_u8<1>(q, w[j >> 2]); break;
                case 2: w[j >> 2] = act_cvt_pk_u8<2>(q, w[j >> 2]); break;
                default: w[j >> 2] = act_cvt_pk_u8<3>(q, w[j >> 2]); break;
            }
        } else {
            const float q = lq_bf16_bits_to_f32(lq_f32_to_bf16_bits(a / c));
            const float rr = q == q ? __builtin_amdgcn_fmed3f(rintf(q), -128.0f, 127.0f) : 0.0f;
            w[j >> 2] |= ((unsigned)(int)rr & 0xFFu) << (8 * (j & 3));
        }
    }
    if (kFast) return u32x2_t{w[0] ^ 0x80808080u, w[1] ^ 0x80808080u};
    return u32x2_t{w[0], w[1]};
}

// The 8 elements from `base` on, for the clamp value c (uniform over the launch).
__device__ __forceinline__ void act_quant_piece(const unsigned short *__restrict__ x, signed char *__restrict__ x8, long long base,
                                                long long n, float c) {
    if (base >= n) return;
    if (base + 8 <= n && (((uintptr_t)(x + base)) & 15) == 0 && (((uintptr_t)(x8 + base)) & 7) == 0) {
        const u32x4_t v = *reinterpret_cast<const u32x4_t *>(x + base);
        const bool c_is_bf16 = (__float_as_uint(c) & 0xFFFFu) == 0u && fabsf(c) >= 0x1p-40f && fabsf(c) <= 0x1p40f;
        // a NaN among the 8 inputs: the two forms differ on it (see above)
        bool any_nan = false;
#pragma unroll
        for (int j = 0; j < 4; ++j) any_nan |= (v[j] & 0x7FFFu) > 0x7F80u || (v[j] & 0x7FFF0000u) > 0x7F800000u;
        u32x2_t o;
        if (c_is_bf16 && !any_nan) o = act_quant8<true>(v, c, 1.0f / c);
        else o = act_quant8<false>(v, c, 0.0f);
        *reinterpret_cast<u32x2_t *>(x8 + base) = o;
    } else {
        for (long long i = base; i < n && i < base + 8; ++i) {
            float f = lq_bf16_bits_to_f32(x[i]);
            float a = lq_bf16_bits_to_f32(lq_f32_to_bf16_bits(f * 127.0f));
            float q = lq_bf16_bits_to_f32(lq_f32_to_bf16_bits(a / c));
            float rr = q == q ? __builtin_amdgcn_fmed3f(rintf(q), -128.0f, 127.0f) : 0.0f;
            x8[i] = (signed char)(int)rr;
        }
    }
}

__global__ __launch_bounds__(256) void act_quant_kernel(const unsigned short *__restrict__ x,
                                                        const float *__restrict__ clampv, signed char *__restrict__ x8,
                                                        long long n) {
    act_quant_piece(x, x8, ((long long)blockIdx.x * 256 + threadIdx.x) * 8, n, clampv[0]);
}

// ---- the tensor's own maximum as clamp value ---------------------------------------------------
// Order-preserving 16-bit key of a bf16 pattern: a larger value has a larger key, -0 < +0, and every NaN has the
// largest key of all, so that an integer maximum over the keys is the tensor library's max(), which returns NaN as
// soon as one element is NaN.
__device__ __forceinline__ unsigned max_key(unsigned b) {
    const unsigned a = b & 0x7FFFu;
    const unsigned k = (b & 0x8000u) ? 0x7FFFu - a : 0x8000u | a;
    return a > 0x7F80u ? 0xFFFFu : k;
}
__device__ __forceinline__ float max_key_value(unsigned k) {
    const unsigned b = k == 0xFFFFu ? 0x7FC0u : (k & 0x8000u) ? (k & 0x7FFFu) : 0x8000u | (0x7FFFu - k);
    return __uint_as_float(b << 16);
}

__device__ __forceinline__ unsigned wave_max_u32(unsigned v) {
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
        const unsigned other = (unsigned)__shfl_xor((int)v, o, 64);
        v = v > other ? v : other;
    }
    return v;
}

// Maximum over a workgroup of 256 threads, returned to every thread.
__device__ __forceinline__ unsigned wg_max_u32(unsigned v, unsigned *red) {
    v = wave_max_u32(v);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    const unsigned a = red[0] > red[1] ? red[0] : red[1], b = red[2] > red[3] ? red[2] : red[3];
    return a > b ? a : b;
}

constexpr int kMaxPartials = LQ_ACT_WORK_FLOATS - 8;

// Phase 1: workgroup b writes the largest key of its grid-stride share of x to partial[b].
__global__ __launch_bounds__(256) void tensor_max_kernel(const unsigned short *__restrict__ x, long long n,
                                                         unsigned *__restrict__ partial) {
    __shared__ unsigned red[4];
    unsigned k = 0u;  // below every key
    const long long n8 = n / 8;
    const u32x4_t *x16 = reinterpret_cast<const u32x4_t *>(x);
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n8; i += (long long)gridDim.x * 256) {
        const u32x4_t v = x16[i];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const unsigned lo = max_key(v[j] & 0xFFFFu), hi = max_key(v[j] >> 16);
            k = k > lo ? k : lo;
            k = k > hi ? k : hi;
        }
    }
    if (blockIdx.x == 0 && (long long)threadIdx.x < n - n8 * 8) {
        const unsigned t = max_key(x[n8 * 8 + threadIdx.x]);
        k = k > t ? k : t;
    }
    k = wg_max_u32(k, red);
    if (threadIdx.x == 0) partial[blockIdx.x] = k;
}

// Phase 2: every workgroup reduces the partial keys to the clamp value, then quantises its 2048 elements;
// the first M threads of the grid also write the per-row scale alpha = clampv * fl(1/127) (the tensor library
// divides a tensor by a host scalar as a product with the scalar's fp32 reciprocal), rounded to bf16 when the
// caller's alpha is a bf16 tensor.
__global__ __launch_bounds__(256) void act_quant_dyn_kernel(const unsigned short *__restrict__ x, signed char *__restrict__ x8,
                                                            float *__restrict__ sx, float *__restrict__ work, int partials,
                                                            long long n, long long M, int alpha_bf16) {
    __shared__ unsigned red[4];
    const unsigned *partial = reinterpret_cast<const unsigned *>(work + 8);
    unsigned k = 0u;
    for (int i = threadIdx.x; i < partials; i += 256) k = k > partial[i] ? k : partial[i];
    k = wg_max_u32(k, red);
    const float c = max_key_value(k);
    float alpha = c * (1.0f / 127.0f);
    if (alpha_bf16) alpha = lq_bf16_bits_to_f32(lq_f32_to_bf16_bits(alpha));
    const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
    if (gid == 0) {
        work[0] = c;
        work[1] = alpha;
    }
    for (long long m = gid; m < M; m += (long long)gridDim.x * 256) sx[m] = alpha;
    act_quant_piece(x, x8, gid * 8, n, c);
}

// ---- one scale per token row --------------------------------------------------------------------
// A wave owns a row: the row's largest |x| (as a bit pattern: magnitudes order like unsigned integers, and a NaN
// pattern is above infinity, so a NaN in the row ends up in the scale), then
//   sx[m] = amax / 127,   x8 = clamp(rint(x * (127 / amax)), -128, 127)      (fp32, IEEE division, NaN -> 0)
// with 127 / amax replaced by 0 for an all-zero row. A lane keeps PT 16-byte pieces of the row in registers between
// the two phases (rows of up to 512 * PT elements are read from memory once); longer rows are read again.
template <int PT>
__global__ __launch_bounds__(256) void act_quant_token_kernel(const unsigned short *__restrict__ x, signed char *__restrict__ x8,
                                                              float *__restrict__ sx, int M, int K) {
    const int lane = threadIdx.x & 63;
    const int m = blockIdx.x * 4 + (int)(threadIdx.x >> 6);
    if (m >= M) return;
    const u32x4_t *row = reinterpret_cast<const u32x4_t *>(x + (long long)m * K);
    u32x2_t *out = reinterpret_cast<u32x2_t *>(x8 + (long long)m * K);
    const int n16 = K / 8, T = (n16 + 63) / 64;
    u32x4_t v[PT];
    unsigned amax = 0u;
    auto take = [&](const u32x4_t &w) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const unsigned a = w[j] & 0x7FFF7FFFu;
            const unsigned lo = a & 0xFFFFu, hi = a >> 16;
            amax = amax > lo ? amax : lo;
            amax = amax > hi ? amax : hi;
        }
    };
#pragma unroll
    for (int t = 0; t < PT; ++t) {
        const int i = lane + 64 * t;
        v[t] = u32x4_t{0u, 0u, 0u, 0u};
        if (i < n16) v[t] = row[i];
    }
#pragma unroll
    for (int t = 0; t < PT; ++t) take(v[t]);
    for (int t = PT; t < T; ++t) {
        const int i = lane + 64 * t;
        if (i < n16) take(row[i]);
    }
    amax = wave_max_u32(amax);
    const float am = __uint_as_float(amax << 16);
    const float inv = am == 0.0f ? 0.0f : 127.0f / am;
    if (lane == 0) sx[m] = am / 127.0f;
    auto quant = [&](const u32x4_t &w) {
        unsigned o[2] = {0u, 0u};
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float f = (j & 1) ? lq_bf16_hi(w[j >> 1]) : lq_bf16_lo(w[j >> 1]);
            const float r = rintf(f * inv);
            const float rr = r == r ? __builtin_amdgcn_fmed3f(r, -128.0f, 127.0f) : 0.0f;
            o[j >> 2] |= ((unsigned)(int)rr & 0xFFu) << (8 * (j & 3));
        }
        return u32x2_t{o[0], o[1]};
    };
#pragma unroll
    for (int t = 0; t < PT; ++t) {
        const int i = lane + 64 * t;
        if (i < n16) out[i] = quant(v[t]);
    }
    for (int t = PT; t < T; ++t) {
        const int i = lane + 64 * t;
        if (i < n16) out[i] = quant(row[i]);
    }
}

// The way back, for the backward pass: out = bf16(x8 * bf16(s)) with s = scale[m] (per token) or scale[0]; the values of
// `x8.to(dtype) * s.to(dtype)`. 16 elements per thread (one row: K % 16 == 0).
__global__ __launch_bounds__(256) void act_dequant_kernel(const u32x4_t *__restrict__ x8, const float *__restrict__ scale,
                                                          u32x4_t *__restrict__ out, long long n_chunks, long long chunks_per_row,
                                                          int per_token) {
    const long long L = (long long)blockIdx.x * 256 + threadIdx.x;
    if (L >= n_chunks) return;
    const float s = lq_bf16_bits_to_f32(lq_f32_to_bf16_bits(scale[per_token ? L / chunks_per_row : 0]));
    const u32x4_t c = x8[L];
    u32x4_t o[2];
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        float v[4];
#pragma unroll
        for (int b = 0; b < 4; ++b) v[b] = (float)(int)(signed char)((c[w] >> (8 * b)) & 0xFFu) * s;
        o[w >> 1][2 * (w & 1)] = lq_pack_bf16(v[0], v[1]);
        o[w >> 1][2 * (w & 1) + 1] = lq_pack_bf16(v[2], v[3]);
    }
    out[2 * L] = o[0];
    out[2 * L + 1] = o[1];
}

// Fake quantisation for the backward pass of the layers that keep the bf16 activations (utils/quant.py:200-202,
// 358-360): out = bf16(clamp(rne(bf16(x * s)), -128, 127) / s) with the bf16 scalar s = 127 / clampv, i.e. the chain
// (input * s).round_().clamp_(-128, 127).div_(s) as one pass; 8 elements per thread. The quotient of an integer of at
// most 8 bits and a bf16 number keeps 2^-17 (relative) from every bf16 rounding tie, so for 2^-40 <= |s| <= 2^40 the
// product with RN(1 / s) rounds to the same bf16 number as the quotient; other scales take the division. NaN stays NaN.
__global__ __launch_bounds__(256) void act_fake_quant_kernel(const unsigned short *__restrict__ x, const unsigned short *__restrict__ s_dev,
                                                             unsigned short *__restrict__ out, long long n) {
    const float s = lq_bf16_bits_to_f32(s_dev[0]);
    const bool fast = fabsf(s) >= 0x1p-40f && fabsf(s) <= 0x1p40f;
    const float r = 1.0f / s;
    const long long base = ((long long)blockIdx.x * 256 + threadIdx.x) * 8;
    if (base >= n) return;
    auto one = [&](float f) {
        const float a = lq_bf16_bits_to_f32(lq_f32_to_bf16_bits(f * s));
        const float q = a != a ? a : __builtin_amdgcn_fmed3f(rintf(a), -128.0f, 127.0f);
        return fast ? q * r : q / s;
    };
    if (base + 8 <= n) {
        const u32x4_t v = *reinterpret_cast<const u32x4_t *>(x + base);
        u32x4_t o;
#pragma unroll
        for (int j = 0; j < 4; ++j) o[j] = lq_pack_bf16(one(lq_bf16_lo(v[j])), one(lq_bf16_hi(v[j])));
        *reinterpret_cast<u32x4_t *>(out + base) = o;
    } else {
        for (long long i = base; i < n; ++i) out[i] = lq_f32_to_bf16_bits(one(lq_bf16_bits_to_f32(x[i])));
    }
}

}  // namespace

extern "C" int lq_act_fake_quant(const void *x, const void *s_bf16_dev, void *out, int64_t n, void *stream) {
    LQ_REQUIRE(x && s_bf16_dev && out && n >= 0, "lq_act_fake_quant: bad argument");
    LQ_REQUIRE(lq_aligned(x, 16) && lq_aligned(out, 16) && lq_aligned(s_bf16_dev, 2),
               "lq_act_fake_quant: x and out must be 16-byte aligned");
    if (n == 0) return LQ_OK;
    const long long blocks = ((n + 7) / 8 + 255) / 256;
    LQ_REQUIRE(blocks <= 0x7FFFFFFFll, "lq_act_fake_quant: n too large");
    hipLaunchKernelGGL(act_fake_quant_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const unsigned short *)x,
                       (const unsigned short *)s_bf16_dev, (unsigned short *)out, (long long)n);
    return lq_check_launch("lq_act_fake_quant");
}

extern "C" int lq_act_dequant_i8(const int8_t *x8, const float *scale, int per_token, void *out, int64_t M, int64_t K,
                                 void *stream) {
    LQ_REQUIRE(x8 && scale && out, "lq_act_dequant_i8: null pointer argument");
    LQ_REQUIRE(M > 0 && K > 0 && K % 16 == 0 && M < (1ll << 31) && K < (1ll << 31),
               "lq_act_dequant_i8: need M > 0 and K a positive multiple of 16 (M=%lld K=%lld)", (long long)M, (long long)K);
    LQ_REQUIRE(lq_aligned(x8, 16) && lq_aligned(out, 16) && lq_aligned(scale, 4),
               "lq_act_dequant_i8: x8 and out must be 16-byte aligned, scale 4-byte");
    const long long n_chunks = M * K / 16;
    const long long blocks = (n_chunks + 255) / 256;
    LQ_REQUIRE(blocks <= 0x7FFFFFFFll, "lq_act_dequant_i8: tensor too large");
    hipLaunchKernelGGL(act_dequant_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const u32x4_t *)x8, scale,
                       (u32x4_t *)out, n_chunks, (long long)(K / 16), per_token);
    return lq_check_launch("lq_act_dequant_i8");
}

extern "C" int lq_act_quant_i8(const void *x, const float *clampv_dev, int8_t *x8, int64_t n, void *stream) {
    LQ_REQUIRE(x && clampv_dev && x8 && n >= 0, "lq_act_quant_i8: bad argument");
    if (n == 0) return LQ_OK;
    const long long blocks = ((n + 7) / 8 + 255) / 256;
    LQ_REQUIRE(blocks <= 0x7FFFFFFFll, "lq_act_quant_i8: n too large");
    hipLaunchKernelGGL(act_quant_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (const unsigned short *)x, clampv_dev, (signed char *)x8, (long long)n);
    return lq_check_launch("lq_act_quant_i8");
}

extern "C" int lq_act_quant_i8_dynamic(const void *x, int8_t *x8, float *sx, float *work, int64_t M, int64_t K, int alpha_bf16,
                                       void *stream) {
    LQ_REQUIRE(x && x8 && sx && work, "lq_act_quant_i8_dynamic: null pointer argument");
    LQ_REQUIRE(M > 0 && K > 0 && M < (1ll << 31) && K < (1ll << 31), "lq_act_quant_i8_dynamic: M=%lld and K=%lld must be positive",
               (long long)M, (long long)K);
    LQ_REQUIRE(lq_aligned(x, 16) && lq_aligned(x8, 8) && lq_aligned(sx, 4) && lq_aligned(work, 4),
               "lq_act_quant_i8_dynamic: x must be 16-byte aligned, x8 8-byte, sx and work 4-byte");
    const long long n = M * K;
    const long long blocks = ((n + 7) / 8 + 255) / 256;
    LQ_REQUIRE(blocks <= 0x7FFFFFFFll, "lq_act_quant_i8_dynamic: tensor too large");
    const int partials = (int)(blocks < kMaxPartials ? blocks : kMaxPartials);
    hipLaunchKernelGGL(tensor_max_kernel, dim3((unsigned)partials), dim3(256), 0, (hipStream_t)stream, (const unsigned short *)x, n,
                       reinterpret_cast<unsigned *>(work + 8));
    int rc = lq_check_launch("lq_act_quant_i8_dynamic(max)");
    if (rc) return rc;
    hipLaunchKernelGGL(act_quant_dyn_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const unsigned short *)x,
                       (signed char *)x8, sx, work, partials, n, (long long)M, alpha_bf16);
    return lq_check_launch("lq_act_quant_i8_dynamic");
}

extern "C" int lq_act_quant_i8_per_token(const void *x, int8_t *x8, float *sx, int64_t M, int64_t K, void *stream) {
    LQ_REQUIRE(x && x8 && sx, "lq_act_quant_i8_per_token: null pointer argument");
    LQ_REQUIRE(M > 0 && K > 0 && K % 8 == 0 && M < (1ll << 31) && K < (1ll << 31),
               "lq_act_quant_i8_per_token: need M > 0 and K a positive multiple of 8 (M=%lld K=%lld)", (long long)M, (long long)K);
    LQ_REQUIRE(lq_aligned(x, 16) && lq_aligned(x8, 8) && lq_aligned(sx, 4),
               "lq_act_quant_i8_per_token: x must be 16-byte aligned, x8 8-byte, sx 4-byte");
    const unsigned blocks = (unsigned)((M + 3) / 4);
    if (K <= 2048)
        hipLaunchKernelGGL(act_quant_token_kernel<4>, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (const unsigned short *)x,
                           (signed char *)x8, sx, (int)M, (int)K);
    else
        hipLaunchKernelGGL(act_quant_token_kernel<16>, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (const unsigned short *)x,
                           (signed char *)x8, sx, (int)M, (int)K);
    return lq_check_launch("lq_act_quant_i8_per_token");
}
