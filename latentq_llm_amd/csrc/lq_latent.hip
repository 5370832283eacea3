// Fused latent-weight passes of the A16W4 layer in its exact 4-bit-residual mode (lbit = 4).
//
// The optimizer step of the reference rebuilds the latent weight of every quantized layer,
//     latent = ResidualTensor.add(DeQfunc_4bit_g(codes))            (utils/quant.py:66-72, 826-837, 1066-1079)
// applies the Adam update to it and re-quantises the result,
//     codes', residual' = Qfunc_4bit_g_res(latent')                  (utils/quant.py:45-63, 803-811)
// each as a chain of ~5 and ~10 elementwise bf16 tensor operations around the residual codec
// kernel. Here each chain is one pass: 32 elements per thread, 16 bytes of codes + 16 bytes of
// residual words in and 64 bytes of latent out, or the reverse. Every tensor operation of the chains rounds
// its result to bf16 (the operands are bf16 tensors, the arithmetic is fp32 inside an operation);
// the kernels keep exactly those rounding points, so their results equal the unfused path's bit
// for bit:
//   reconstruct:  w = bf16(bf16(q - z) * s);  r = bf16(bf16(value(nibble)) * s);  latent = bf16(r + w)
//   requant:      Z = bf16(bf16(t / s) + z);  q = rint(Z);  f = bf16(Z - q)
//                 (nibble, carry) = codec(f);  code = clamp(bf16(q + carry), 0, 15)
//
// The 8-bit-weight layer keeps its latent the same way (int8 codes, one bf16 scale per row, the same residual words):
//   reconstruct:  w = bf16(q * s);  r = bf16(bf16(value(nibble)) * s);  latent = bf16(r + w)
//                 (ResidualTensor.add((p.data * p.qparam).to(dtype)), utils/quant.py:826-837, 1069-1070)
//   requant:      Z = bf16(t / s);  q = rint(Z);  f = bf16(Z - q);  (nibble, carry) = codec(f)
//                 code = clamp(q + carry, -128, 127)                  (Qfunc_8bit_res, utils/quant.py:88-103)
#include "lq_latent_math.h"

namespace {

// A thread owns 32 consecutive elements of one quantisation group: 16 bytes of codes, 16 bytes of
// residual words, 64 bytes of latent; one scale and zero per thread.
__global__ __launch_bounds__(256) void latent_reconstruct_kernel(const u32x4_t *__restrict__ codes,
                                                                 const unsigned short *__restrict__ scales,
                                                                 const unsigned short *__restrict__ zeros,
                                                                 const u32x4_t *__restrict__ residual,
                                                                 u32x4_t *__restrict__ latent, long long n_chunks,
                                                                 CodecParams p) {
    __shared__ float vtab[16];
    lq_latent_fill_value_table(vtab, p);
    __syncthreads();
    const long long L = (long long)blockIdx.x * 256 + threadIdx.x;
    if (L >= n_chunks) return;
    const u32x4_t cw = codes[L], rw = residual[L];
    const float s = lq_bf16_bits_to_f32(scales[L >> 2]);
    const float z = lq_bf16_bits_to_f32(zeros[L >> 2]);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float v[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            v[k] = lq_latent_value(lq_code(cw[i], k), vtab[(rw[i] >> (28 - 4 * k)) & 0xFu], s, z);
        }
        latent[L * 4 + i] = u32x4_t{lq_pack_bf16(v[0], v[1]), lq_pack_bf16(v[2], v[3]), lq_pack_bf16(v[4], v[5]),
                                    lq_pack_bf16(v[6], v[7])};
    }
}

// The 32 elements of one thread through the re-quantiser (codec parameters by value: scalars)
template <bool kFast>
__device__ __forceinline__ void requant_thread(const u32x4_t (&in)[4], float s, float z, float r, const CodecParams p,
                                               u32x4_t &cout, u32x4_t &rout) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        unsigned cword = 0, rword = 0;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const float t = (k & 1) ? lq_bf16_hi(in[i][k >> 1]) : lq_bf16_lo(in[i][k >> 1]);
            unsigned nib, code;
            lq_latent_requant_elem<kFast>(t, s, z, r, p, nib, code);
            rword = (rword << 4) | nib;
            cword |= code << (4 * (k ^ 1));
        }
        cout[i] = cword;
        rout[i] = rword;
    }
}

__global__ __launch_bounds__(256) void latent_requant_kernel(const u32x4_t *__restrict__ latent,
                                                             const unsigned short *__restrict__ scales,
                                                             const unsigned short *__restrict__ zeros,
                                                             u32x4_t *__restrict__ codes, u32x4_t *__restrict__ residual,
                                                             long long n_chunks, CodecParams p) {
    const long long L = (long long)blockIdx.x * 256 + threadIdx.x;
    if (L >= n_chunks) return;
    u32x4_t in[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) in[i] = latent[L * 4 + i];
    const float s = lq_bf16_bits_to_f32(scales[L >> 2]);
    const float z = lq_bf16_bits_to_f32(zeros[L >> 2]);
    const bool fast = (s >= 0x1p-40f) && (s <= 0x1p40f);
    const float r = 1.0f / s;
    u32x4_t cout, rout;
    // one branch per thread (a thread's 32 elements share their group's scale)
    if (fast) requant_thread<true>(in, s, z, r, p, cout, rout);
    else requant_thread<false>(in, s, z, r, p, cout, rout);
    codes[L] = cout;
    residual[L] = rout;
}

// ---- 8-bit weights: a thread owns 16 consecutive elements of one row (16 code bytes, two residual words) ----
__global__ __launch_bounds__(256) void latent_w8_reconstruct_kernel(const u32x4_t *__restrict__ codes,
                                                                    const unsigned short *__restrict__ qscales,
                                                                    const u32x2_t *__restrict__ residual,
                                                                    u32x4_t *__restrict__ latent, long long n_chunks,
                                                                    long long chunks_per_row, CodecParams p) {
    __shared__ float vtab[16];
    lq_latent_fill_value_table(vtab, p);
    __syncthreads();
    const long long L = (long long)blockIdx.x * 256 + threadIdx.x;
    if (L >= n_chunks) return;
    const u32x4_t cw = codes[L];
    const u32x2_t rw = residual[L];
    const float s = lq_bf16_bits_to_f32(qscales[L / chunks_per_row]);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        float v[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const int e = 8 * i + k;
            v[k] = lq_latent_w8_value(cw[e >> 2] >> (8 * (e & 3)), vtab[(rw[i] >> (28 - 4 * k)) & 0xFu], s);
        }
        latent[L * 2 + i] = u32x4_t{lq_pack_bf16(v[0], v[1]), lq_pack_bf16(v[2], v[3]), lq_pack_bf16(v[4], v[5]),
                                    lq_pack_bf16(v[6], v[7])};
    }
}

template <bool kFast>
__device__ __forceinline__ void requant_w8_thread(const u32x4_t (&in)[2], float s, float r, const CodecParams p, u32x4_t &cout,
                                                  u32x2_t &rout) {
    unsigned cw[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        unsigned rword = 0;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const float t = (k & 1) ? lq_bf16_hi(in[i][k >> 1]) : lq_bf16_lo(in[i][k >> 1]);
            unsigned nib, byte;
            lq_latent_w8_requant_elem<kFast>(t, s, r, p, nib, byte);
            rword = (rword << 4) | nib;
            const int e = 8 * i + k;
            cw[e >> 2] |= byte << (8 * (e & 3));
        }
        rout[i] = rword;
    }
    cout = u32x4_t{cw[0], cw[1], cw[2], cw[3]};
}

__global__ __launch_bounds__(256) void latent_w8_requant_kernel(const u32x4_t *__restrict__ latent,
                                                                const unsigned short *__restrict__ qscales,
                                                                u32x4_t *__restrict__ codes, u32x2_t *__restrict__ residual,
                                                                long long n_chunks, long long chunks_per_row, CodecParams p) {
    const long long L = (long long)blockIdx.x * 256 + threadIdx.x;
    if (L >= n_chunks) return;
    u32x4_t in[2];
    in[0] = latent[L * 2];
    in[1] = latent[L * 2 + 1];
    const float s = lq_bf16_bits_to_f32(qscales[L / chunks_per_row]);
    // the quotient of two bf16 numbers as a product with the reciprocal: see lq_latent_requant_elem
    const bool fast = (fabsf(s) >= 0x1p-40f) && (fabsf(s) <= 0x1p40f);
    const float r = 1.0f / s;
    u32x4_t cout;
    u32x2_t rout;
    if (fast) requant_w8_thread<true>(in, s, r, p, cout, rout);
    else requant_w8_thread<false>(in, s, r, p, cout, rout);
    codes[L] = cout;
    residual[L] = rout;
}

int check_latent_w8(const char *who, const void *a, const void *b, const void *c, const void *d, int64_t N, int64_t K, int k1,
                    float b1, int k2, float b2, int k3) {
    LQ_REQUIRE(a && b && c && d, "%s: null pointer argument", who);
    LQ_REQUIRE(N > 0 && K > 0 && K % 16 == 0, "%s: need N > 0, K a positive multiple of 16", who);
    LQ_REQUIRE(N * K / 16 <= 0x7FFFFFFFll * 256, "%s: tensor too large", who);
    LQ_REQUIRE(k1 > 0 && k2 > 0 && k3 > 0 && b1 > 0.0f && b2 > b1 && b2 < 0.5f, "%s: need k1,k2,k3 > 0 and 0 < b1 < b2 < 0.5",
               who);
    return LQ_OK;
}

int check_latent(const char *who, const void *a, const void *b, const void *c, const void *d, const void *e, int64_t N,
                 int64_t K, int group, int k1, float b1, int k2, float b2, int k3) {
    LQ_REQUIRE(a && b && c && d && e, "%s: null pointer argument", who);
    LQ_REQUIRE(group == LQ_GROUP, "%s: group must be %d", who, LQ_GROUP);
    LQ_REQUIRE(N > 0 && K > 0 && K % LQ_GROUP == 0, "%s: need N > 0, K a positive multiple of %d", who, LQ_GROUP);
    LQ_REQUIRE(N * K / 32 <= 0x7FFFFFFFll * 256, "%s: tensor too large", who);
    LQ_REQUIRE(k1 > 0 && k2 > 0 && k3 > 0 && b1 > 0.0f && b2 > b1 && b2 < 0.5f, "%s: need k1,k2,k3 > 0 and 0 < b1 < b2 < 0.5",
               who);
    return LQ_OK;
}

}  // namespace

extern "C" int lq_latent_w4_reconstruct(const void *codes, const void *scales, const void *zeros, const int32_t *residual,
                                        void *latent_out, int64_t N, int64_t K, int group, int k1, float b1, int k2,
                                        float b2, int k3, void *stream) {
    int rc = check_latent("lq_latent_w4_reconstruct", codes, scales, zeros, residual, latent_out, N, K, group, k1, b1, k2,
                          b2, k3);
    if (rc) return rc;
    LQ_REQUIRE(lq_aligned(codes, 16) && lq_aligned(residual, 16) && lq_aligned(latent_out, 16),
               "lq_latent_w4_reconstruct: codes, residual and latent must be 16-byte aligned");
    const long long n_chunks = (long long)N * K / 32;  // K % 128 == 0: no remainder
    hipLaunchKernelGGL(latent_reconstruct_kernel, dim3((unsigned)((n_chunks + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, (const u32x4_t *)codes, (const unsigned short *)scales,
                       (const unsigned short *)zeros, (const u32x4_t *)residual, (u32x4_t *)latent_out, n_chunks,
                       lq_codec_dequant_params(k1, b1, k2, b2, k3));
    return lq_check_launch("lq_latent_w4_reconstruct");
}

extern "C" int lq_latent_w4_requant(const void *latent, const void *scales, const void *zeros, void *codes_out,
                                    int32_t *residual_out, int64_t N, int64_t K, int group, int k1, float b1, int k2,
                                    float b2, int k3, void *stream) {
    int rc = check_latent("lq_latent_w4_requant", latent, scales, zeros, codes_out, residual_out, N, K, group, k1, b1, k2,
                          b2, k3);
    if (rc) return rc;
    LQ_REQUIRE(lq_aligned(latent, 16) && lq_aligned(codes_out, 16) && lq_aligned(residual_out, 16),
               "lq_latent_w4_requant: latent, codes and residual must be 16-byte aligned");
    const long long n_chunks = (long long)N * K / 32;  // K % 128 == 0: no remainder
    hipLaunchKernelGGL(latent_requant_kernel, dim3((unsigned)((n_chunks + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const u32x4_t *)latent, (const unsigned short *)scales, (const unsigned short *)zeros,
                       (u32x4_t *)codes_out, (u32x4_t *)residual_out, n_chunks, lq_codec_quant_params(k1, b1, k2, b2, k3));
    return lq_check_launch("lq_latent_w4_requant");
}

extern "C" int lq_latent_w8_reconstruct(const int8_t *codes, const void *qscales, const int32_t *residual, void *latent_out,
                                        int64_t N, int64_t K, int k1, float b1, int k2, float b2, int k3, void *stream) {
    int rc = check_latent_w8("lq_latent_w8_reconstruct", codes, qscales, residual, latent_out, N, K, k1, b1, k2, b2, k3);
    if (rc) return rc;
    LQ_REQUIRE(lq_aligned(codes, 16) && lq_aligned(residual, 8) && lq_aligned(latent_out, 16),
               "lq_latent_w8_reconstruct: codes and latent must be 16-byte, residual 8-byte aligned");
    const long long n_chunks = (long long)N * K / 16;
    hipLaunchKernelGGL(latent_w8_reconstruct_kernel, dim3((unsigned)((n_chunks + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const u32x4_t *)codes, (const unsigned short *)qscales, (const u32x2_t *)residual, (u32x4_t *)latent_out,
                       n_chunks, (long long)(K / 16), lq_codec_dequant_params(k1, b1, k2, b2, k3));
    return lq_check_launch("lq_latent_w8_reconstruct");
}

extern "C" int lq_latent_w8_requant(const void *latent, const void *qscales, int8_t *codes_out, int32_t *residual_out, int64_t N,
                                    int64_t K, int k1, float b1, int k2, float b2, int k3, void *stream) {
    int rc = check_latent_w8("lq_latent_w8_requant", latent, qscales, codes_out, residual_out, N, K, k1, b1, k2, b2, k3);
    if (rc) return rc;
    LQ_REQUIRE(lq_aligned(latent, 16) && lq_aligned(codes_out, 16) && lq_aligned(residual_out, 8),
               "lq_latent_w8_requant: latent and codes must be 16-byte, residual 8-byte aligned");
    const long long n_chunks = (long long)N * K / 16;
    hipLaunchKernelGGL(latent_w8_requant_kernel, dim3((unsigned)((n_chunks + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const u32x4_t *)latent, (const unsigned short *)qscales, (u32x4_t *)codes_out, (u32x2_t *)residual_out,
                       n_chunks, (long long)(K / 16), lq_codec_quant_params(k1, b1, k2, b2, k3));
    return lq_check_launch("lq_latent_w8_requant");
}
