// Elementwise companions of the GEMM kernels: whole-matrix dequantise, the int8 weight
// re-quantiser, GPTQ <-> native layout converters, calibration kernels and the bf16 transpose.
#include "lq_common.h"

namespace {

// One thread = one packed word (8 codes of one row) -> 16 bytes of bf16.
// Arithmetic of the reference dequantiser: bf16(bf16(q - z) * s).
__global__ __launch_bounds__(256) void dequant_kernel(const unsigned *__restrict__ codes,
                                                      const unsigned short *__restrict__ scales,
                                                      const unsigned short *__restrict__ zeros,
                                                      u32x4_t *__restrict__ out, long long n_words) {
    const long long w = (long long)blockIdx.x * 256 + threadIdx.x;
    if (w >= n_words) return;
    const unsigned word = codes[w];
    const float s = lq_bf16_bits_to_f32(scales[w >> 4]);
    const float z = lq_bf16_bits_to_f32(zeros[w >> 4]);
    u32x4_t o;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float d0 = (float)lq_code(word, 2 * i) - z;
        float d1 = (float)lq_code(word, 2 * i + 1) - z;
        unsigned dp = lq_pack_bf16(d0, d1);
        o[i] = lq_pack_bf16(lq_bf16_lo(dp) * s, lq_bf16_hi(dp) * s);
    }
    out[w] = o;
}

// Per-channel int8 re-quantiser of an 8-bit-weight layer's latent (the reference's Qfunc_8bit_res without a
// residual codec, utils/quant.py:88-103): code = clamp(rint(bf16(t / qs[n])), -128, 127) for the bf16 latent t
// and the bf16 scale of its row. Same arithmetic as act_quant8: for 2^-40 <= |qs| <= 2^40 the quotient of the two
// bf16 numbers is their reciprocal product, and rounding, clamp and byte insertion are one instruction; rows
// with another scale, and pieces with a NaN (which becomes 0), take the written-out form.
__global__ __launch_bounds__(256) void w8_requant_kernel(const u32x4_t *__restrict__ latent,
                                                         const unsigned short *__restrict__ qscales,
                                                         u32x2_t *__restrict__ codes, long long n_pieces, long long K8) {
    const long long i = (long long)blockIdx.x * 256 + threadIdx.x;  // 8 consecutive elements of one row
    if (i >= n_pieces) return;
    const float c = lq_bf16_bits_to_f32(qscales[i / K8]);
    const u32x4_t v = latent[i];
    bool any_nan = false;
#pragma unroll
    for (int j = 0; j < 4; ++j) any_nan |= (v[j] & 0x7FFFu) > 0x7F80u || (v[j] & 0x7FFF0000u) > 0x7F800000u;
    const bool fast = fabsf(c) >= 0x1p-40f && fabsf(c) <= 0x1p40f && !any_nan;
    unsigned w[2] = {0u, 0u};
    if (fast) {
        const float r = 1.0f / c;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float t = (j & 1) ? lq_bf16_hi(v[j >> 1]) : lq_bf16_lo(v[j >> 1]);
            const float q = lq_bf16_bits_to_f32(lq_f32_to_bf16_bits(t * r)) + 128.0f;
            switch (j & 3) {
                case 0: w[j >> 2] = act_cvt_pk_u8<0>(q, w[j >> 2]); break;
                case 1: w[j >> 2] = act_cvt_pk_u8<1>(q, w[j >> 2]); break;
                case 2: w[j >> 2] = act_cvt_pk_u8<2>(q, w[j >> 2]); break;
                default: w[j >> 2] = act_cvt_pk_u8<3>(q, w[j >> 2]); break;
            }
        }
        w[0] ^= 0x80808080u;
        w[1] ^= 0x80808080u;
    } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float t = (j & 1) ? lq_bf16_hi(v[j >> 1]) : lq_bf16_lo(v[j >> 1]);
            const float q = lq_bf16_bits_to_f32(lq_f32_to_bf16_bits(t / c));
            const float rr = q == q ? __builtin_amdgcn_fmed3f(rintf(q), -128.0f, 127.0f) : 0.0f;
            w[j >> 2] |= ((unsigned)(int)rr & 0xFFu) << (8 * (j & 3));
        }
    }
    codes[i] = u32x2_t{w[0], w[1]};
}

__device__ __forceinline__ unsigned swap_nibbles(unsigned g) {
    return ((g & 0x0F0F0F0Fu) << 4) | ((g >> 4) & 0x0F0F0F0Fu);
}

// 32x32-word tile transpose through LDS: GPTQ word [kw][n] <-> native word [n][kw].
// kToNative: src is [KW][N], dst is [N][KW]; otherwise src is [N][KW], dst is [KW][N].
template <bool kToNative>
__global__ __launch_bounds__(256) void repack_kernel(const unsigned *__restrict__ src, unsigned *__restrict__ dst,
                                                     int N, int KW) {
    __shared__ unsigned tile[32][33];
    const int src_rows = kToNative ? KW : N, src_cols = kToNative ? N : KW;
    const int c0 = blockIdx.x * 32, r0 = blockIdx.y * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        int r = r0 + ty + 8 * i, c = c0 + tx;
        if (r < src_rows && c < src_cols) tile[ty + 8 * i][tx] = swap_nibbles(src[(long long)r * src_cols + c]);
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        int r = c0 + ty + 8 * i, c = r0 + tx;  // dst is [src_cols][src_rows]
        if (r < src_cols && c < src_rows) dst[(long long)r * src_rows + c] = tile[tx][ty + 8 * i];
    }
}

}  // namespace

extern "C" int lq_a16w4_dequant(const void *codes, const void *scales, const void *zeros, void *w_out, int64_t N,
                                int64_t K, int group, void *stream) {
    LQ_REQUIRE(codes && scales && zeros && w_out, "lq_a16w4_dequant: null pointer argument");
    LQ_REQUIRE(group == LQ_GROUP, "lq_a16w4_dequant: group must be %d", LQ_GROUP);
    LQ_REQUIRE(N > 0 && K > 0 && K % LQ_GROUP == 0, "lq_a16w4_dequant: need N > 0, K a positive multiple of %d", LQ_GROUP);
    LQ_REQUIRE(lq_aligned(codes, 4) && lq_aligned(w_out, 16), "lq_a16w4_dequant: misaligned buffer");
    const long long n_words = (long long)N * K / 8;
    const long long blocks = (n_words + 255) / 256;
    LQ_REQUIRE(blocks <= 0x7FFFFFFFll, "lq_a16w4_dequant: tensor too large");
    hipLaunchKernelGGL(dequant_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (const unsigned *)codes, (const unsigned short *)scales, (const unsigned short *)zeros,
                       (u32x4_t *)w_out, n_words);
    return lq_check_launch("lq_a16w4_dequant");
}

extern "C" int lq_w8_requant(const void *latent, const void *qscales, int8_t *codes, int64_t N, int64_t K, void *stream) {
    LQ_REQUIRE(latent && qscales && codes, "lq_w8_requant: null pointer argument");
    LQ_REQUIRE(N > 0 && K > 0 && K % 8 == 0 && N * K / 8 / 256 < 0x7FFFFFFFll,
               "lq_w8_requant: need N > 0 and K a positive multiple of 8 (N=%lld K=%lld)", (long long)N, (long long)K);
    LQ_REQUIRE(lq_aligned(latent, 16) && lq_aligned(codes, 8) && lq_aligned(qscales, 2),
               "lq_w8_requant: latent must be 16-byte, codes 8-byte aligned");
    const long long pieces = N * K / 8;
    hipLaunchKernelGGL(w8_requant_kernel, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       (const u32x4_t *)latent, (const unsigned short *)qscales, (u32x2_t *)codes, pieces, (long long)(K / 8));
    return lq_check_launch("lq_w8_requant");
}

static int repack_common(const void *src, void *dst, int64_t N, int64_t K, void *stream, bool to_native, const char *who) {
    LQ_REQUIRE(src && dst, "%s: null pointer argument", who);
    LQ_REQUIRE(N > 0 && K > 0 && K % 8 == 0, "%s: need N > 0 and K a positive multiple of 8", who);
    LQ_REQUIRE(lq_aligned(src, 4) && lq_aligned(dst, 4), "%s: buffers must be 4-byte aligned", who);
    LQ_REQUIRE(N < (1ll << 30) && K < (1ll << 30), "%s: dimension too large", who);
    const int KW = (int)(K / 8), n = (int)N;
    if (to_native) {
        dim3 grid((n + 31) / 32, (KW + 31) / 32);
        hipLaunchKernelGGL(repack_kernel<true>, grid, dim3(256), 0, (hipStream_t)stream, (const unsigned *)src,
                           (unsigned *)dst, n, KW);
    } else {
        dim3 grid((KW + 31) / 32, (n + 31) / 32);
        hipLaunchKernelGGL(repack_kernel<false>, grid, dim3(256), 0, (hipStream_t)stream, (const unsigned *)src,
                           (unsigned *)dst, n, KW);
    }
    return lq_check_launch(who);
}

extern "C" int lq_repack_gptq_to_native(const int32_t *qweight_gptq, void *codes_native, int64_t N, int64_t K,
                                        void *stream) {
    return repack_common(qweight_gptq, codes_native, N, K, stream, true, "lq_repack_gptq_to_native");
}

extern "C" int lq_repack_native_to_gptq(const void *codes_native, int32_t *qweight_gptq, int64_t N, int64_t K,
                                        void *stream) {
    return repack_common(codes_native, qweight_gptq, N, K, stream, false, "lq_repack_native_to_gptq");
}

// ---- calibration copy -------------------------------------------------------
// Grid-stride 16-byte copy: each workgroup streams contiguous 4 KiB pieces.
__global__ __launch_bounds__(256) void calib_copy_kernel(const u32x4_t *__restrict__ src, u32x4_t *__restrict__ dst,
                                                        long long n16) {
    const long long stride = (long long)gridDim.x * 256;
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n16; i += stride)
        __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

// Read-only counterpart of the copy: every thread XORs the 16-byte pieces of its grid-stride share and the
// workgroup's last wave writes one word, so that the loads cannot be dropped and nothing else is written.
__global__ __launch_bounds__(256) void calib_read_kernel(const u32x4_t *__restrict__ src, long long n16,
                                                        unsigned *__restrict__ sink) {
    const long long stride = (long long)gridDim.x * 256;
    u32x4_t a = {0u, 0u, 0u, 0u};
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < n16; i += stride) {
        const u32x4_t v = __builtin_nontemporal_load(src + i);
        a[0] ^= v[0]; a[1] ^= v[1]; a[2] ^= v[2]; a[3] ^= v[3];
    }
    const unsigned x = a[0] ^ a[1] ^ a[2] ^ a[3];
    if (x == 0x9E3779B9u && threadIdx.x == 255) sink[blockIdx.x & 63] = x;  // practically never taken
}

// Measurement aid: nothing but matrix instructions, in the forward GEMM's shape. A workgroup is 4 waves
// (one per SIMD), each holding 4 + 2 operand fragments loaded once from the caller's buffers and 8
// accumulator tiles of 32 x 32; an iteration issues the 8 MFMAs (32x32x16 bf16) of one reduction
// slice of that kernel. Every wave records the shader-cycle counter and the 100 MHz real-time
// counter around its loop.
__global__ __launch_bounds__(256, 2) void mfma_loop_kernel(const u32x4_t *__restrict__ a, const u32x4_t *__restrict__ b,
                                                           long long n16, long long iters, unsigned long long *__restrict__ clk,
                                                           float *__restrict__ sink) {
    const int lane = threadIdx.x & 63;
    const long long wv = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    u32x4_t af[4], bf[2];
#pragma unroll
    for (int j = 0; j < 4; ++j) af[j] = a[((wv * 4 + j) * 64 + lane) % n16];
#pragma unroll
    for (int i = 0; i < 2; ++i) bf[i] = b[((wv * 2 + i) * 64 + lane) % n16];
    f32x16_t acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int q = 0; q < 16; ++q) acc[i][j][q] = 0;
    const unsigned long long t0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
    for (long long it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, bf[i]),
                                                                   __builtin_bit_cast(bf16x8_t, af[j]), acc[i][j], 0, 0, 0);
    }
    const unsigned long long t1 = __builtin_amdgcn_s_memtime(), r1 = __builtin_amdgcn_s_memrealtime();
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int q = 0; q < 16; ++q) s += acc[i][j][q];
    if (lane == 0) {
        clk[4 * wv] = t0; clk[4 * wv + 1] = t1; clk[4 * wv + 2] = r0; clk[4 * wv + 3] = r1;
        sink[wv] = s;
    }
}

// The same loop on the int8 matrix instruction of the A8W8 kernels (32x32x32, int32 accumulators).
__global__ __launch_bounds__(256, 2) void mfma_loop_i8_kernel(const u32x4_t *__restrict__ a, const u32x4_t *__restrict__ b,
                                                              long long n16, long long iters, unsigned long long *__restrict__ clk,
                                                              int *__restrict__ sink) {
    const int lane = threadIdx.x & 63;
    const long long wv = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    u32x4_t af[4], bf[2];
#pragma unroll
    for (int j = 0; j < 4; ++j) af[j] = a[((wv * 4 + j) * 64 + lane) % n16];
#pragma unroll
    for (int i = 0; i < 2; ++i) bf[i] = b[((wv * 2 + i) * 64 + lane) % n16];
    i32x16_t acc[2][4];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int q = 0; q < 16; ++q) acc[i][j][q] = 0;
    const unsigned long long t0 = __builtin_amdgcn_s_memtime(), r0 = __builtin_amdgcn_s_memrealtime();
    for (long long it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4_t, bf[i]), __builtin_bit_cast(i32x4_t, af[j]),
                                                                 acc[i][j], 0, 0, 0);
    }
    const unsigned long long t1 = __builtin_amdgcn_s_memtime(), r1 = __builtin_amdgcn_s_memrealtime();
    int s = 0;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int q = 0; q < 16; ++q) s += acc[i][j][q];
    if (lane == 0) {
        clk[4 * wv] = t0; clk[4 * wv + 1] = t1; clk[4 * wv + 2] = r0; clk[4 * wv + 3] = r1;
        sink[wv] = s;
    }
}

extern "C" int lq_calib_mfma_loop_i8(const void *a, const void *b, int64_t n_bytes, int64_t iters, int workgroups_per_cu,
                                     uint64_t *clocks, int64_t clocks_capacity, int32_t *sink, int64_t *waves, void *stream) {
    LQ_REQUIRE(a && b && clocks && sink && waves, "lq_calib_mfma_loop_i8: null pointer argument");
    LQ_REQUIRE(n_bytes >= 8192 && n_bytes % 16 == 0 && lq_aligned(a, 16) && lq_aligned(b, 16) && lq_aligned(clocks, 8),
               "lq_calib_mfma_loop_i8: operands need at least 8192 bytes, a multiple of 16, 16-byte aligned");
    LQ_REQUIRE(iters > 0 && (workgroups_per_cu == 1 || workgroups_per_cu == 2), "lq_calib_mfma_loop_i8: iters > 0, 1 or 2 workgroups per unit");
    const long long wgs = (long long)lq_device_cu_count() * workgroups_per_cu;
    LQ_REQUIRE(16 * wgs <= clocks_capacity, "lq_calib_mfma_loop_i8: clocks must hold %lld values", 16 * wgs);
    *waves = 4 * wgs;
    hipLaunchKernelGGL(mfma_loop_i8_kernel, dim3((unsigned)wgs), dim3(256), 0, (hipStream_t)stream, (const u32x4_t *)a,
                       (const u32x4_t *)b, (long long)(n_bytes / 16), (long long)iters, (unsigned long long *)clocks, sink);
    return lq_check_launch("lq_calib_mfma_loop_i8");
}

extern "C" int lq_calib_mfma_loop(const void *a, const void *b, int64_t n_elems, int64_t iters, int workgroups_per_cu,
                                  uint64_t *clocks, int64_t clocks_capacity, float *sink, int64_t *waves, void *stream) {
    LQ_REQUIRE(a && b && clocks && sink && waves, "lq_calib_mfma_loop: null pointer argument");
    LQ_REQUIRE(n_elems >= 512 && n_elems % 8 == 0 && lq_aligned(a, 16) && lq_aligned(b, 16) && lq_aligned(clocks, 8),
               "lq_calib_mfma_loop: operands need at least 512 elements, a multiple of 8, 16-byte aligned");
    LQ_REQUIRE(iters > 0 && (workgroups_per_cu == 1 || workgroups_per_cu == 2), "lq_calib_mfma_loop: iters > 0, 1 or 2 workgroups per unit");
    const long long wgs = (long long)lq_device_cu_count() * workgroups_per_cu;
    LQ_REQUIRE(16 * wgs <= clocks_capacity, "lq_calib_mfma_loop: clocks must hold %lld values", 16 * wgs);
    *waves = 4 * wgs;
    hipLaunchKernelGGL(mfma_loop_kernel, dim3((unsigned)wgs), dim3(256), 0, (hipStream_t)stream, (const u32x4_t *)a,
                       (const u32x4_t *)b, (long long)(n_elems / 8), (long long)iters, (unsigned long long *)clocks, sink);
    return lq_check_launch("lq_calib_mfma_loop");
}

extern "C" int lq_calib_copy(const void *src, void *dst, int64_t nbytes, void *stream) {
    LQ_REQUIRE(src && dst, "lq_calib_copy: null pointer argument");
    LQ_REQUIRE(nbytes >= 0 && nbytes % 16 == 0, "lq_calib_copy: nbytes must be a non-negative multiple of 16");
    LQ_REQUIRE(lq_aligned(src, 16) && lq_aligned(dst, 16), "lq_calib_copy: buffers must be 16-byte aligned");
    if (nbytes == 0) return LQ_OK;
    const long long n16 = nbytes / 16;
    long long blocks = (n16 + 255) / 256;
    if (blocks > 256 * 16) blocks = 256 * 16;
    hipLaunchKernelGGL(calib_copy_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (const u32x4_t *)src, (u32x4_t *)dst, n16);
    return lq_check_launch("lq_calib_copy");
}

extern "C" int lq_calib_read(const void *src, int64_t nbytes, int workgroups, void *sink, void *stream) {
    LQ_REQUIRE(src && sink, "lq_calib_read: null pointer argument");
    LQ_REQUIRE(nbytes >= 0 && nbytes % 16 == 0 && lq_aligned(src, 16) && lq_aligned(sink, 4),
               "lq_calib_read: nbytes must be a non-negative multiple of 16, src 16-byte aligned");
    if (nbytes == 0) return LQ_OK;
    const long long n16 = nbytes / 16;
    long long blocks = workgroups > 0 ? workgroups : (n16 + 255) / 256;
    if (blocks > (n16 + 255) / 256) blocks = (n16 + 255) / 256;
    if (blocks > 0x7FFFFFFFll) blocks = 0x7FFFFFFFll;
    hipLaunchKernelGGL(calib_read_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const u32x4_t *)src, n16,
                       (unsigned *)sink);
    return lq_check_launch("lq_calib_read");
}

// ---- bf16 matrix transpose --------------------------------------------------
// dst[c][r] = src[r][c] for a row-major [R, C] matrix, 64 x 64 tiles through LDS, 16-byte global
// accesses on both sides. The weight gradient dW = dY^T X is a GEMM whose left operand is read
// along its strided dimension; the vendor GEMM runs 20-35 % faster on a transposed copy of dY,
// and this pass costs a tenth of that GEMM.
__global__ __launch_bounds__(256) void transpose_bf16_kernel(const unsigned short *__restrict__ src,
                                                            unsigned short *__restrict__ dst, int R, int C) {
    __shared__ unsigned short tile[64][66];  // 132-byte rows: the column gathers below spread over the banks
    const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
    const int t = threadIdx.x, sub = t >> 3, ch = (t & 7) * 8;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int r = sub + 32 * i;
        if (r0 + r < R && c0 + ch < C) {
            const u32x4_t v = *reinterpret_cast<const u32x4_t *>(src + (long long)(r0 + r) * C + c0 + ch);
#pragma unroll
            for (int j = 0; j < 4; ++j) *reinterpret_cast<unsigned *>(&tile[r][ch + 2 * j]) = v[j];
        }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int c = sub + 32 * i;  // output row
        if (c0 + c < C && r0 + ch < R) {
            u32x4_t v;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                v[j] = (unsigned)tile[ch + 2 * j][c] | ((unsigned)tile[ch + 2 * j + 1][c] << 16);
            *reinterpret_cast<u32x4_t *>(dst + (long long)(c0 + c) * R + r0 + ch) = v;
        }
    }
}

extern "C" int lq_transpose_bf16(const void *src, void *dst, int64_t R, int64_t C, void *stream) {
    LQ_REQUIRE(src && dst, "lq_transpose_bf16: null pointer argument");
    LQ_REQUIRE(R > 0 && C > 0 && R % 8 == 0 && C % 8 == 0, "lq_transpose_bf16: R=%lld and C=%lld must be positive multiples of 8",
               (long long)R, (long long)C);
    LQ_REQUIRE(R < (1ll << 31) && C < (1ll << 31) && (C + 63) / 64 < 0x7FFFFFFFll && (R + 63) / 64 <= 65535 * 64ll,
               "lq_transpose_bf16: matrix too large");
    LQ_REQUIRE(lq_aligned(src, 16) && lq_aligned(dst, 16), "lq_transpose_bf16: buffers must be 16-byte aligned");
    LQ_REQUIRE((R + 63) / 64 <= 65535, "lq_transpose_bf16: more than 65535 row tiles");
    hipLaunchKernelGGL(transpose_bf16_kernel, dim3((unsigned)((C + 63) / 64), (unsigned)((R + 63) / 64)), dim3(256), 0,
                       (hipStream_t)stream, (const unsigned short *)src, (unsigned short *)dst, (int)R, (int)C);
    return lq_check_launch("lq_transpose_bf16");
}
