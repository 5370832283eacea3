// Kernels (2a) and (3): LDS-tiled MFMA GEMMs for gfx950.
//
//   MODE_W4_FWD : Y[M,N]  = X[M,K]  . deq(W)[N,K]^T     (bf16 MFMA, int4 W dequantised into LDS)
//   MODE_W4_DX  : dX[M,K] = dY[M,N] . deq(W)[N,K]       (same, W tile transposed while staging)
//   MODE_I8     : acc     = X8[M,K] . W8[N,K]^T         (int8 MFMA, int32 accumulate, scaled epilogue)
//
// Common structure. "A" is the activation-side operand, row-major with the reduction
// dimension contiguous. "B" is the weight-side operand, presented in LDS as
// [output column][reduction] exactly like A. A tile row in LDS is 128 bytes (64 bf16 or
// 128 int8) = eight 16-byte chunks; chunk c of row r is stored at chunk position
// c ^ ((r ^ (r >> 3)) & 7), which makes the 16-byte fragment reads of 8 consecutive rows
// and the staging writes hit distinct banks. One MFMA step consumes 32 bytes of every
// row (chunks 2s and 2s+1), i.e. 4 steps per tile.
//
// The MFMA is issued with the weight fragment as the first operand and the activation
// fragment as the second, so that D[i][j] has i = output column (n), j = row (m): a
// lane then owns 4 consecutive n for one m and the epilogue stores 8-byte bf16 quads.
#include "lq_common.h"

#include <type_traits>

namespace {

enum { MODE_W4_FWD = 0, MODE_W4_DX = 1, MODE_I8 = 2 };

struct GemmParams {
    const void *a;        // activations: bf16 [M, R] or int8 [M, R]
    const void *b;        // weights: packed codes or int8 [N, K]
    const unsigned short *scales;
    const unsigned short *zeros;
    const unsigned short *bias;  // bf16 [out cols] or null
    const float *sx;             // MODE_I8: per-row scale
    const float *sw;             // MODE_I8: per-column scale
    void *c;                     // bf16 [M, C]
    int *acc_out;                // MODE_I8: optional int32 [M, C]
    int M;                       // rows of A / C
    int C;                       // output columns (N for fwd/i8, K for dx)
    int R;                       // reduction length (K for fwd/i8, N for dx)
    int Kw;                      // K of the weight matrix (row length of W in elements)
    int tiles_m, tiles_n;
};

__device__ __forceinline__ int swz(int row) { return (row ^ (row >> 3)) & 7; }

// 8 codes of a native word -> 8 bf16 (k order) = 4 packed dwords, w = bf16((q - z) * s).
// nzs = -(z*s) is exact for integer zeros, and fma(q, s, nzs) rounds the exact (q-z)*s once.
__device__ __forceinline__ void dequant_word(unsigned word, float s, float nzs, unsigned o[4]) {
    const unsigned lo4 = word & 0x0F0F0F0Fu;
    const unsigned hi4 = (word >> 4) & 0x0F0F0F0Fu;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float e = fmaf((float)((hi4 >> (8 * i)) & 0xFFu), s, nzs);
        float d = fmaf((float)((lo4 >> (8 * i)) & 0xFFu), s, nzs);
        o[i] = lq_pack_bf16(e, d);
    }
}

template <int MODE, int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(64 * WM * WN) void gemm_kernel(GemmParams p) {
    constexpr int NT = 64 * WM * WN;
    constexpr int TM = BM / WM, TN = BN / WN;  // wave tile
    constexpr int FM = TM / 32, FN = TN / 32;  // 32x32 fragments per wave tile
    constexpr int ROWB = 128;                  // bytes per LDS tile row
    constexpr int A_BYTES = BM * ROWB, B_BYTES = BN * ROWB;
    constexpr int ESZ = (MODE == MODE_I8) ? 1 : 2;
    constexpr int RT = ROWB / ESZ;  // reduction elements per tile (64 bf16 / 128 int8)
    static_assert(TM % 32 == 0 && TN % 32 == 0, "wave tile must be a multiple of 32x32");
    static_assert((BM * 8) % NT == 0, "A staging must divide evenly");

    __shared__ __attribute__((aligned(16))) unsigned char smem[2 * (A_BYTES + B_BYTES)];
    unsigned char *lds_a = smem;                // [2][BM][128]
    unsigned char *lds_b = smem + 2 * A_BYTES;  // [2][BN][128]

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave % WM, wn = wave / WM;

    // Workgroup ids are dealt round-robin over the 8 XCDs; give each XCD a contiguous range of
    // tiles (m fastest) so that the tiles resident on one XCD share weight columns in its L2.
    const int nwg = p.tiles_m * p.tiles_n;
    int id = blockIdx.x;
    {
        const int per = nwg / 8;
        if (id < per * 8) id = (id % 8) * per + id / 8;
    }
    const int tile_m = id % p.tiles_m, tile_n = id / p.tiles_m;
    const int m0 = tile_m * BM, c0 = tile_n * BN;

    // ---- staging assignments ------------------------------------------------
    constexpr int APT = BM * 8 / NT;  // 16-byte chunks of A per thread per tile
    const unsigned char *a_src[APT];
    int a_dst[APT];
    const long long lda = (long long)p.R * ESZ;
#pragma unroll
    for (int i = 0; i < APT; ++i) {
        const int c = i * NT + tid;
        const int row = c >> 3, ch = c & 7;
        int gr = m0 + row;
        gr = gr < p.M ? gr : p.M - 1;
        a_src[i] = (const unsigned char *)p.a + gr * lda + ch * 16;
        a_dst[i] = row * ROWB + ((ch ^ swz(row)) << 4);
    }

    // B staging registers
    constexpr int BPT_I8 = (MODE == MODE_I8) ? BN * 8 / NT : 1;
    constexpr int BPT_W4 = (MODE == MODE_W4_FWD) ? (BN * 2 + NT - 1) / NT : 1;
    const unsigned char *b_src[MODE == MODE_I8 ? BPT_I8 : (MODE == MODE_W4_FWD ? BPT_W4 : 4)];
    int b_dst[MODE == MODE_I8 ? BPT_I8 : (MODE == MODE_W4_FWD ? BPT_W4 : 1)];
    const unsigned short *s_src[MODE == MODE_W4_DX ? 4 : BPT_W4];
    const unsigned short *z_src[MODE == MODE_W4_DX ? 4 : BPT_W4];
    int b_row[BPT_W4];
    int b_half[BPT_W4];
    const int groups_per_row = p.Kw / LQ_GROUP;

    if (MODE == MODE_I8) {
#pragma unroll
        for (int i = 0; i < BPT_I8; ++i) {
            const int c = i * NT + tid;
            const int row = c >> 3, ch = c & 7;
            int gr = c0 + row;
            gr = gr < p.C ? gr : p.C - 1;
            b_src[i] = (const unsigned char *)p.b + (long long)gr * p.Kw + ch * 16;
            b_dst[i] = row * ROWB + ((ch ^ swz(row)) << 4);
        }
    } else if (MODE == MODE_W4_FWD) {
        // tile = BN rows x 32 bytes of codes; a thread takes 16 bytes (32 codes) of one row.
#pragma unroll
        for (int i = 0; i < BPT_W4; ++i) {
            const int c = i * NT + tid;
            const int row = (c >> 1) % BN, half = c & 1;
            int gr = c0 + row;
            gr = gr < p.C ? gr : p.C - 1;
            b_src[i] = (const unsigned char *)p.b + (long long)gr * (p.Kw / 2) + half * 16;
            s_src[i] = p.scales + (long long)gr * groups_per_row;
            z_src[i] = p.zeros + (long long)gr * groups_per_row;
            b_row[i] = row;
            b_half[i] = half;
        }
    } else {
        // dX: tile = 64 weight rows (reduction n) x BN columns (k); a thread takes one code word
        // (8 k) from each of 4 consecutive rows and emits, per k, 4 consecutive n (8 bytes).
        static_assert(MODE != MODE_W4_DX || (NT == 256 && BN == 128), "dX staging assumes 256 threads, 128 columns");
        const int kw = tid & 15, nblk = tid >> 4;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int n = nblk * 4 + r;  // + tile offset along n added per tile
            b_src[r] = (const unsigned char *)p.b + (long long)n * (p.Kw / 2) + (c0 / 8 + kw) * 4;
            const int g = (c0 + kw * 8) / LQ_GROUP;
            s_src[r] = p.scales + (long long)n * groups_per_row + g;
            z_src[r] = p.zeros + (long long)n * groups_per_row + g;
        }
        b_dst[0] = (kw * 8) * ROWB;  // row base; chunk/half resolved at write time
        b_row[0] = nblk;
        b_half[0] = 0;
    }

    // ---- register staging buffers --------------------------------------------
    u32x4_t a_reg[APT];
    u32x4_t b_reg[MODE == MODE_I8 ? BPT_I8 : BPT_W4];
    unsigned bw_reg[4];
    unsigned short s_reg[MODE == MODE_W4_DX ? 4 : BPT_W4], z_reg[MODE == MODE_W4_DX ? 4 : BPT_W4];

    auto load_tile = [&](int kt) {
#pragma unroll
        for (int i = 0; i < APT; ++i) a_reg[i] = *reinterpret_cast<const u32x4_t *>(a_src[i] + (long long)kt * ROWB);
        if (MODE == MODE_I8) {
#pragma unroll
            for (int i = 0; i < BPT_I8; ++i)
                b_reg[i] = *reinterpret_cast<const u32x4_t *>(b_src[i] + (long long)kt * ROWB);
        } else if (MODE == MODE_W4_FWD) {
#pragma unroll
            for (int i = 0; i < BPT_W4; ++i) {
                b_reg[i] = *reinterpret_cast<const u32x4_t *>(b_src[i] + (long long)kt * 32);
                s_reg[i] = s_src[i][kt >> 1];
                z_reg[i] = z_src[i][kt >> 1];
            }
        } else {
            const long long row_off = (long long)kt * 64;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                bw_reg[r] = *reinterpret_cast<const unsigned *>(b_src[r] + row_off * (p.Kw / 2));
                s_reg[r] = s_src[r][row_off * groups_per_row];
                z_reg[r] = z_src[r][row_off * groups_per_row];
            }
        }
    };

    auto store_tile = [&](int buf) {
        unsigned char *la = lds_a + buf * A_BYTES;
        unsigned char *lb = lds_b + buf * B_BYTES;
#pragma unroll
        for (int i = 0; i < APT; ++i) *reinterpret_cast<u32x4_t *>(la + a_dst[i]) = a_reg[i];
        if (MODE == MODE_I8) {
#pragma unroll
            for (int i = 0; i < BPT_I8; ++i) *reinterpret_cast<u32x4_t *>(lb + b_dst[i]) = b_reg[i];
        } else if (MODE == MODE_W4_FWD) {
#pragma unroll
            for (int i = 0; i < BPT_W4; ++i) {
                if (BN * 2 % NT == 0 || i * NT + tid < BN * 2) {
                    const float s = lq_bf16_bits_to_f32(s_reg[i]);
                    const float nzs = -(lq_bf16_bits_to_f32(z_reg[i]) * s);
                    const int row = b_row[i];
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        unsigned o[4];
                        dequant_word(b_reg[i][w], s, nzs, o);
                        const int ch = b_half[i] * 4 + w;
                        u32x4_t v = {o[0], o[1], o[2], o[3]};
                        *reinterpret_cast<u32x4_t *>(lb + row * ROWB + ((ch ^ swz(row)) << 4)) = v;
                    }
                }
            }
        } else {
            // 4 rows (n) x 8 k  ->  for each k: 4 consecutive n = 8 bytes at LDS row k.
            unsigned o[4][4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float s = lq_bf16_bits_to_f32(s_reg[r]);
                const float nzs = -(lq_bf16_bits_to_f32(z_reg[r]) * s);
                dequant_word(bw_reg[r], s, nzs, o[r]);
            }
            const int nblk = b_row[0];
            const int ch = nblk >> 1, hf = nblk & 1;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int row = (b_dst[0] / ROWB) + j;
                // element j of word r: dword j/2, half j&1
                unsigned e[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) e[r] = (j & 1) ? (o[r][j >> 1] >> 16) : (o[r][j >> 1] & 0xFFFFu);
                u32x2_t v = {e[0] | (e[1] << 16), e[2] | (e[3] << 16)};
                *reinterpret_cast<u32x2_t *>(lb + row * ROWB + ((ch ^ swz(row)) << 4) + hf * 8) = v;
            }
        }
    };

    // ---- accumulators -------------------------------------------------------
    using acc_t = typename std::conditional<MODE == MODE_I8, i32x16_t, f32x16_t>::type;
    acc_t acc[FN][FM];
#pragma unroll
    for (int i = 0; i < FN; ++i)
#pragma unroll
        for (int j = 0; j < FM; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    const int nk = p.R / RT;
    const int frag_row = lane & 31, kh = lane >> 5;

    load_tile(0);
    store_tile(0);
    __syncthreads();

    for (int kt = 0; kt < nk; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < nk) load_tile(kt + 1);

        const unsigned char *la = lds_a + buf * A_BYTES + (wm * TM) * ROWB;
        const unsigned char *lb = lds_b + buf * B_BYTES + (wn * TN) * ROWB;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const int ch = 2 * ks + kh;
            u32x4_t af[FM], bf[FN];
#pragma unroll
            for (int i = 0; i < FM; ++i) {
                const int row = i * 32 + frag_row;
                af[i] = *reinterpret_cast<const u32x4_t *>(la + row * ROWB + ((ch ^ swz(wm * TM + row)) << 4));
            }
#pragma unroll
            for (int i = 0; i < FN; ++i) {
                const int row = i * 32 + frag_row;
                bf[i] = *reinterpret_cast<const u32x4_t *>(lb + row * ROWB + ((ch ^ swz(wn * TN + row)) << 4));
            }
#pragma unroll
            for (int i = 0; i < FN; ++i)
#pragma unroll
                for (int j = 0; j < FM; ++j) {
                    if constexpr (MODE == MODE_I8) {
                        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4_t, bf[i]),
                                                                         __builtin_bit_cast(i32x4_t, af[j]),
                                                                         acc[i][j], 0, 0, 0);
                    } else {
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, bf[i]),
                                                                           __builtin_bit_cast(bf16x8_t, af[j]),
                                                                           acc[i][j], 0, 0, 0);
                    }
                }
        }
        if (kt + 1 < nk) store_tile(buf ^ 1);
        __syncthreads();
    }

    // ---- epilogue -----------------------------------------------------------
    // acc[i][j][r]: column c = c0 + wn*TN + i*32 + 8*(r/4) + 4*(lane/32) + r%4, row m = m0 + wm*TM + j*32 + lane%32.
    unsigned short *out = (unsigned short *)p.c;
#pragma unroll
    for (int j = 0; j < FM; ++j) {
        const int m = m0 + wm * TM + j * 32 + frag_row;
        if (m >= p.M) continue;
        float sxm = 1.0f;
        if (MODE == MODE_I8) sxm = p.sx[m];
#pragma unroll
        for (int i = 0; i < FN; ++i) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int c = c0 + wn * TN + i * 32 + 8 * q + 4 * kh;
                if (c >= p.C) continue;  // C is a multiple of 4: a quad is all-in or all-out
                float v[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    if (MODE == MODE_I8) {
                        v[r] = ((float)acc[i][j][4 * q + r] * sxm) * p.sw[c + r];
                    } else {
                        v[r] = acc[i][j][4 * q + r];
                    }
                    if (p.bias) v[r] += lq_bf16_bits_to_f32(p.bias[c + r]);
                }
                u32x2_t o = {lq_pack_bf16(v[0], v[1]), lq_pack_bf16(v[2], v[3])};
                *reinterpret_cast<u32x2_t *>(out + (long long)m * p.C + c) = o;
                if (MODE == MODE_I8 && p.acc_out) {
                    i32x4_t a4 = {(int)acc[i][j][4 * q], (int)acc[i][j][4 * q + 1], (int)acc[i][j][4 * q + 2],
                                  (int)acc[i][j][4 * q + 3]};
                    *reinterpret_cast<i32x4_t *>(p.acc_out + (long long)m * p.C + c) = a4;
                }
            }
        }
    }
}

template <int MODE, int BM, int BN, int WM, int WN>
int launch_gemm(GemmParams p, hipStream_t st, const char *who) {
    p.tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.C + BN - 1) / BN;
    auto kern = gemm_kernel<MODE, BM, BN, WM, WN>;
    const long long nwg = (long long)p.tiles_m * p.tiles_n;
    if (nwg > 0x7FFFFFFFll) return lq_fail(LQ_ERR_BAD_ARG, "%s: problem too large", who);
    hipLaunchKernelGGL(kern, dim3((unsigned)nwg), dim3(64 * WM * WN), 0, st, p);
    return lq_check_launch(who);
}

}  // namespace

// GEMV path (lq_gemv.hip)
int lq_gemv_a16w4_launch(const void *x, const void *codes, const void *scales, const void *zeros, const void *bias,
                         void *y, int M, int N, int K, hipStream_t st);

static int check_w4_common(const char *who, const void *a, const void *codes, const void *scales, const void *zeros,
                           const void *out, int64_t M, int64_t N, int64_t K, int group) {
    LQ_REQUIRE(a && codes && scales && zeros && out, "%s: null pointer argument", who);
    LQ_REQUIRE(group == LQ_GROUP, "%s: group must be %d, got %d", who, LQ_GROUP, group);
    LQ_REQUIRE(M > 0 && N > 0 && K > 0, "%s: M, N, K must be positive (M=%lld N=%lld K=%lld)", who, (long long)M,
               (long long)N, (long long)K);
    LQ_REQUIRE(K % LQ_GROUP == 0, "%s: K=%lld must be a multiple of %d", who, (long long)K, LQ_GROUP);
    LQ_REQUIRE(M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31) && N * K < (1ll << 40), "%s: dimension too large", who);
    LQ_REQUIRE(lq_aligned(a, 16) && lq_aligned(codes, 16) && lq_aligned(out, 16) && lq_aligned(scales, 2) &&
                   lq_aligned(zeros, 2),
               "%s: activation, code and output buffers must be 16-byte aligned", who);
    return LQ_OK;
}

extern "C" int lq_a16w4_fwd(const void *x, const void *codes, const void *scales, const void *zeros,
                            const void *bias_or_null, void *y, int64_t M, int64_t N, int64_t K, int group,
                            void *stream) {
    int rc = check_w4_common("lq_a16w4_fwd", x, codes, scales, zeros, y, M, N, K, group);
    if (rc) return rc;
    LQ_REQUIRE(N % 16 == 0, "lq_a16w4_fwd: N=%lld must be a multiple of 16", (long long)N);
    if (M <= 16)
        return lq_gemv_a16w4_launch(x, codes, scales, zeros, bias_or_null, y, (int)M, (int)N, (int)K, (hipStream_t)stream);
    GemmParams p = {};
    p.a = x; p.b = codes; p.scales = (const unsigned short *)scales; p.zeros = (const unsigned short *)zeros;
    p.bias = (const unsigned short *)bias_or_null; p.c = y;
    p.M = (int)M; p.C = (int)N; p.R = (int)K; p.Kw = (int)K;
    if (M <= 128) return launch_gemm<MODE_W4_FWD, 128, 128, 2, 2>(p, (hipStream_t)stream, "lq_a16w4_fwd");
    return launch_gemm<MODE_W4_FWD, 256, 128, 2, 2>(p, (hipStream_t)stream, "lq_a16w4_fwd");
}

extern "C" int lq_a16w4_dx(const void *dy, const void *codes, const void *scales, const void *zeros, void *dx,
                           int64_t M, int64_t N, int64_t K, int group, void *stream) {
    int rc = check_w4_common("lq_a16w4_dx", dy, codes, scales, zeros, dx, M, N, K, group);
    if (rc) return rc;
    LQ_REQUIRE(N % 64 == 0, "lq_a16w4_dx: N=%lld must be a multiple of 64", (long long)N);
    GemmParams p = {};
    p.a = dy; p.b = codes; p.scales = (const unsigned short *)scales; p.zeros = (const unsigned short *)zeros;
    p.c = dx;
    p.M = (int)M; p.C = (int)K; p.R = (int)N; p.Kw = (int)K;
    if (M <= 128) return launch_gemm<MODE_W4_DX, 128, 128, 2, 2>(p, (hipStream_t)stream, "lq_a16w4_dx");
    return launch_gemm<MODE_W4_DX, 256, 128, 2, 2>(p, (hipStream_t)stream, "lq_a16w4_dx");
}

extern "C" int lq_a8w8_fwd(const void *x, const void *w, const float *sx, const float *sw, const void *bias_or_null,
                           void *y, int32_t *acc_or_null, int64_t M, int64_t N, int64_t K, void *stream) {
    LQ_REQUIRE(x && w && sx && sw && y, "lq_a8w8_fwd: null pointer argument");
    LQ_REQUIRE(M > 0 && N > 0 && K > 0, "lq_a8w8_fwd: M, N, K must be positive");
    LQ_REQUIRE(K % 128 == 0, "lq_a8w8_fwd: K=%lld must be a multiple of 128", (long long)K);
    LQ_REQUIRE(N % 16 == 0, "lq_a8w8_fwd: N=%lld must be a multiple of 16", (long long)N);
    LQ_REQUIRE(M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31), "lq_a8w8_fwd: dimension too large");
    LQ_REQUIRE(lq_aligned(x, 16) && lq_aligned(w, 16) && lq_aligned(y, 16) && lq_aligned(sx, 4) && lq_aligned(sw, 4) &&
                   (!acc_or_null || lq_aligned(acc_or_null, 16)),
               "lq_a8w8_fwd: x, w, y, acc must be 16-byte aligned");
    GemmParams p = {};
    p.a = x; p.b = w; p.sx = sx; p.sw = sw; p.bias = (const unsigned short *)bias_or_null; p.c = y;
    p.acc_out = acc_or_null;
    p.M = (int)M; p.C = (int)N; p.R = (int)K; p.Kw = (int)K;
    if (M <= 128) return launch_gemm<MODE_I8, 128, 128, 2, 2>(p, (hipStream_t)stream, "lq_a8w8_fwd");
    return launch_gemm<MODE_I8, 256, 128, 2, 2>(p, (hipStream_t)stream, "lq_a8w8_fwd");
}
