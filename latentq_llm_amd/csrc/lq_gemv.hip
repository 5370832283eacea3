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
//
// Memory access. The MFMA wants lane 16*kq + n to hold 8 k of weight row n, which as a load
// pattern would put the 4 lanes of every quad on 4 different rows (64 separate cache-line
// requests per wave instruction). The codes are therefore loaded with lane 4*r + c reading
// 16-byte chunk c of row r (a quad reads 64 contiguous bytes) and moved to the MFMA layout
// with one ds_bpermute per dword. For the same reason the scales and zeros of a batch of 4
// consecutive groups are fetched as one 8-byte load by the 16 lanes kq = 0 only and then
// broadcast, and activation loads are limited to the lanes of live tokens: what a vector load
// costs here is cache-line look-ups per quad, not bytes.
#include "lq_common.h"

namespace {


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

typedef __attribute__((address_space(3))) void lds_void;
typedef const __attribute__((address_space(1))) void gbl_void;

constexpr int kUnroll = 4;       // groups per batch (scale/zero batches are 4 x bf16 = 8 bytes)
constexpr int kXRow = 1024 + 16;  // LDS bytes per staged token row: 4 groups x 256 B, padded against bank conflicts

// MP = number of token rows staged per wave and batch (>= M). NT = 16-row weight tiles per
// workgroup: every workgroup stages the activations of its K range again, so with many tokens two
// tiles per workgroup halve that traffic (and share the activation-sum MFMAs).
// GU (with NT = 2, no QS): gate / up mode. Tile 1 is the same 16 rows of a second matrix (codes2, scales2,
// zeros2) and the output is silu(tile 0) * tile 1 on the fp32 sums: the gate / up pair of a gated MLP in one
// pass over both matrices.
template <int WAVES, int MP, int NT, bool QS, bool GU = false>
__global__ __launch_bounds__(64 * WAVES) void gemv_kernel(const unsigned short *__restrict__ x,
                                                          const unsigned char *__restrict__ codes,
                                                          const unsigned short *__restrict__ scales,
                                                          const unsigned short *__restrict__ zeros,
                                                          const unsigned short *__restrict__ bias,
                                                          unsigned short *__restrict__ y, int M, int N, int K,
                                                          const unsigned char *__restrict__ codes2 = nullptr,
                                                          const unsigned short *__restrict__ scales2 = nullptr,
                                                          const unsigned short *__restrict__ zeros2 = nullptr) {
    static_assert(!GU || (NT == 2 && !QS), "gate / up mode: two tiles, scales and zeros straight from memory");
    constexpr int RT = GU ? 1 : NT;  // 16-row tiles of output rows per workgroup
    __shared__ float red[WAVES][NT][4][64];
    __shared__ __attribute__((aligned(16))) unsigned char xs[WAVES][MP][kXRow];
    extern __shared__ __attribute__((aligned(16))) unsigned char sq[];  // QS: scales then zeros of the workgroup's rows
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));  // scalar: uniform control flow
    const int n = lane & 15, kq = lane >> 4;
    const int row = blockIdx.x * (16 * RT) + n;  // weight row of this lane's B fragment in tile 0 (tile j: + 16 j)
    const int G = K / LQ_GROUP;

    // load layout of the codes: lane 4*r + c -> row r of this block, 16-byte chunk c of the group
    const long long wrow_off = (long long)(blockIdx.x * (16 * RT) + (lane >> 2)) * (K / 2) + (lane & 3) * 16;
    const unsigned char *wrow = codes + wrow_off;
    const unsigned char *wrow2 = GU ? codes2 + wrow_off : nullptr;  // gate / up mode: tile 1 is the second matrix
    const long long tile_stride = 16ll * (K / 2);  // bytes between the same row of consecutive tiles
    const int bperm_src = (4 * n + kq) * 4;  // ds_bpermute: take from lane 4*n + kq
    const int bcast_src = n * 4;             // ds_bpermute: take from lane n (kq = 0)
    const unsigned short *srow = scales + (long long)row * G;
    const unsigned short *zrow = zeros + (long long)row * G;
    // As an A-fragment lane, `n` is the token index; lanes of tokens >= M re-read the last staged
    // row: they only feed accumulator rows m >= M, which are never stored.
    const unsigned char *xfrag = &xs[wave][n < M ? n : M - 1][kq * 64];

    const u32x4_t ones = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
    f32x4_t acc[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j) acc[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    // QS: the scales and zeros of the workgroup's 16*NT rows are one contiguous block each; the waves
    // fetch them together with 16-byte loads (issued first, so that they return first) and every wave
    // then takes its groups from LDS
    constexpr int kQPieces = 2;  // 16-byte pieces per thread: up to 64*WAVES*2*16 bytes of scales + zeros
    const int q_bytes = 16 * NT * G * 2;
    // LDS row pitch of the staged block: rows whose length is a multiple of 16 bytes get 16 bytes of
    // padding (a 64-byte pitch would put the 16 rows a group is read from on 4 bank groups); other
    // lengths keep the block as it is (its 16-byte pieces straddle rows)
    const int q_row = G * 2, q_pitch = (q_row % 16 == 0) ? q_row + 16 : q_row;
    const int q_lds = 16 * NT * q_pitch;  // bytes per array in LDS
    u32x4_t qstage[kQPieces];
    if constexpr (QS) {
        const unsigned char *sb = (const unsigned char *)(scales + (long long)blockIdx.x * (16 * NT) * G);
        const unsigned char *zb = (const unsigned char *)(zeros + (long long)blockIdx.x * (16 * NT) * G);
#pragma unroll
        for (int i = 0; i < kQPieces; ++i) {
            const int pc = (int)threadIdx.x + i * 64 * WAVES;
            const int o = pc * 16;
            qstage[i] = u32x4_t{0u, 0u, 0u, 0u};
            if (o < 2 * q_bytes) qstage[i] = *reinterpret_cast<const u32x4_t *>(o < q_bytes ? sb + o : zb + (o - q_bytes));
        }
    }
    bool first = true;
    // every wave runs this exactly once: in its first batch, after that batch's loads are issued, or
    // after the loop when it has no batch at all (the barrier inside needs all waves)
    auto publish_q = [&]() {
#pragma unroll
        for (int i = 0; i < kQPieces; ++i) {
            const int o = ((int)threadIdx.x + i * 64 * WAVES) * 16;
            if (o < 2 * q_bytes) {
                const int oa = o < q_bytes ? o : o - q_bytes;
                const int dst = q_pitch == q_row ? oa : (oa / q_row) * q_pitch + oa % q_row;
                *reinterpret_cast<u32x4_t *>(sq + (o < q_bytes ? 0 : q_lds) + dst) = qstage[i];
            }
        }
        __syncthreads();
    };
    for (int g0 = wave * kUnroll; g0 < G; g0 += WAVES * kUnroll) {
        const bool full = g0 + kUnroll <= G;  // a short tail batch re-reads the last group with zero scale
        // ---- activations: one LDS-direct load per token row (1 KB = this batch's 512 k), coalesced.
        //      In a tail batch the lanes past the end of the row re-read its first bytes (dead groups).
        {
            const long long xoff = (long long)g0 * (LQ_GROUP * 2) + lane * 16;
            const long long lim = (long long)K * 2;
            const long long off = xoff < lim ? xoff : 0;
#pragma unroll
            for (int m = 0; m < MP; ++m)
                if (m < M)
                    __builtin_amdgcn_global_load_lds((gbl_void *)((const unsigned char *)x + (long long)m * lim + off),
                                                     (lds_void *)&xs[wave][m][0], 16, 0, 0);
        }
        // ---- codes, scales, zeros
        u32x4_t wv[NT][kUnroll];
        float sc[NT][kUnroll], zz[NT][kUnroll];
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) {
                const int g = g0 + u < G ? g0 + u : G - 1;
                const unsigned char *wt = (GU && j == 1) ? wrow2 : wrow + j * tile_stride;
                wv[j][u] = *reinterpret_cast<const u32x4_t *>(wt + g * 64);
            }
        if constexpr (QS) {
            if (first) {
                publish_q();
                first = false;
            }
#pragma unroll
            for (int j = 0; j < NT; ++j) {
                const unsigned short *ls = reinterpret_cast<const unsigned short *>(sq + (j * 16 + n) * q_pitch);
                const unsigned short *lz = reinterpret_cast<const unsigned short *>(sq + q_lds + (j * 16 + n) * q_pitch);
#pragma unroll
                for (int u = 0; u < kUnroll; ++u) {
                    const bool live = g0 + u < G;
                    const int g = live ? g0 + u : G - 1;
                    sc[j][u] = live ? lq_bf16_bits_to_f32(ls[g]) : 0.0f;
                    zz[j][u] = 128.0f + lq_bf16_bits_to_f32(lz[g]);
                }
            }
        } else
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            const unsigned short *sr = GU ? (j == 0 ? srow : scales2 + (long long)row * G) : srow + (long long)j * 16 * G;
            const unsigned short *zr = GU ? (j == 0 ? zrow : zeros2 + (long long)row * G) : zrow + (long long)j * 16 * G;
            if (full) {
                u32x2_t sraw = {0u, 0u}, zraw = {0u, 0u};
                if (kq == 0) {
                    sraw = *reinterpret_cast<const u32x2_t *>(sr + g0);
                    zraw = *reinterpret_cast<const u32x2_t *>(zr + g0);
                }
                unsigned s01 = (unsigned)__builtin_amdgcn_ds_bpermute(bcast_src, (int)sraw[0]);
                unsigned s23 = (unsigned)__builtin_amdgcn_ds_bpermute(bcast_src, (int)sraw[1]);
                unsigned z01 = (unsigned)__builtin_amdgcn_ds_bpermute(bcast_src, (int)zraw[0]);
                unsigned z23 = (unsigned)__builtin_amdgcn_ds_bpermute(bcast_src, (int)zraw[1]);
                sc[j][0] = lq_bf16_lo(s01); sc[j][1] = lq_bf16_hi(s01); sc[j][2] = lq_bf16_lo(s23); sc[j][3] = lq_bf16_hi(s23);
                zz[j][0] = 128.0f + lq_bf16_lo(z01); zz[j][1] = 128.0f + lq_bf16_hi(z01);
                zz[j][2] = 128.0f + lq_bf16_lo(z23); zz[j][3] = 128.0f + lq_bf16_hi(z23);
            } else {
#pragma unroll
                for (int u = 0; u < kUnroll; ++u) {
                    const bool live = g0 + u < G;
                    const int g = live ? g0 + u : G - 1;
                    sc[j][u] = live ? lq_bf16_bits_to_f32(sr[g]) : 0.0f;
                    zz[j][u] = 128.0f + lq_bf16_bits_to_f32(zr[g]);
                }
            }
        }
        // ---- codes to the MFMA lane layout
#pragma unroll
        for (int j = 0; j < NT; ++j)
#pragma unroll
            for (int u = 0; u < kUnroll; ++u)
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    wv[j][u][t] = (unsigned)__builtin_amdgcn_ds_bpermute(bperm_src, (int)wv[j][u][t]);
        // ---- MFMAs
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the staged rows have landed in LDS
        // One group at a time: a single pair of MFMA accumulators (plus one per extra tile) is live,
        // which keeps the kernel at <= 80 registers (6 waves per SIMD, three 8-wave workgroups per
        // CU); the unpacking between two MFMAs on the same accumulator covers their latency.
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            f32x4_t P[NT], S = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < NT; ++j) P[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                unsigned a[4];
                const u32x4_t xv = *reinterpret_cast<const u32x4_t *>(xfrag + u * 256 + t * 16);
                permute_x(xv, a);
                const u32x4_t av = {a[0], a[1], a[2], a[3]};
                S = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, av),
                                                            __builtin_bit_cast(bf16x8_t, ones), S, 0, 0, 0);
#pragma unroll
                for (int j = 0; j < NT; ++j) {
                    unsigned b[4];
                    unpack_word_128q(wv[j][u][t], b);
                    const u32x4_t bv = {b[0], b[1], b[2], b[3]};
                    P[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, av),
                                                                   __builtin_bit_cast(bf16x8_t, bv), P[j], 0, 0, 0);
                }
            }
#pragma unroll
            for (int j = 0; j < NT; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[j][r] = fmaf(sc[j][u], fmaf(-zz[j][u], S[r], P[j][r]), acc[j][r]);
            __builtin_amdgcn_sched_barrier(0);  // keeps the next group's unpacking from being hoisted (registers)
        }
        // the next batch overwrites the staged rows: all fragment reads above must have returned
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }

    if constexpr (QS) {
        if (first) publish_q();
    }
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) red[wave][j][r][lane] = acc[j][r];
    __syncthreads();
    if constexpr (GU) {
        if (wave == 0) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float g = 0.f, u = 0.f;
#pragma unroll
                for (int w = 0; w < WAVES; ++w) {
                    g += red[w][0][r][lane];
                    u += red[w][1][r][lane];
                }
                const int m = 4 * kq + r;
                if (m < M) y[(long long)m * N + row] = lq_f32_to_bf16_bits(g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)) * u);
            }
        }
    } else if (wave < NT) {
        // wave j finishes tile j; lane holds D[m = 4*kq + r][n]
        const int orow = row + 16 * wave;
        const float b = bias ? lq_bf16_bits_to_f32(bias[orow]) : 0.0f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float v = 0.f;
#pragma unroll
            for (int w = 0; w < WAVES; ++w) v += red[w][wave][r][lane];
            const int m = 4 * kq + r;
            if (m < M) y[(long long)m * N + orow] = lq_f32_to_bf16_bits(v + b);
        }
    }
}

}  // namespace

namespace {

struct GemvArgs {
    const void *x, *codes, *scales, *zeros, *bias;
    void *y;
    int M, N, K;
    hipStream_t st;
};

struct GemvGuArgs {
    const void *x, *codes, *scales, *zeros, *codes2, *scales2, *zeros2;
    void *y;
    int M, N, K;
    hipStream_t st;
};

template <int W, int MP>
void launch_gu(const GemvGuArgs &a) {
    hipLaunchKernelGGL((gemv_kernel<W, MP, 2, false, true>), dim3(a.N / 16), dim3(64 * W), 0, a.st, (const unsigned short *)a.x,
                       (const unsigned char *)a.codes, (const unsigned short *)a.scales, (const unsigned short *)a.zeros,
                       (const unsigned short *)nullptr, (unsigned short *)a.y, a.M, a.N, a.K, (const unsigned char *)a.codes2,
                       (const unsigned short *)a.scales2, (const unsigned short *)a.zeros2);
}

template <int W, int MP, int NT>
void launch_one(const GemvArgs &a) {
    // Scales and zeros through LDS: pays with many staged tokens when a wave uses them for more than one
    // batch or for two row tiles (measured: 13.5 -> 12.5 us on 11008 x 4096 at 16 tokens; with one batch
    // and one tile per wave the extra barrier costs more than the loads it saves). Both blocks must be
    // 16-byte aligned and fit two 16-byte pieces per thread.
    const size_t q_bytes = (size_t)16 * NT * (a.K / LQ_GROUP) * 2;
    const int batches = (a.K / LQ_GROUP + kUnroll - 1) / kUnroll;
    const bool qs = MP == 16 && (NT == 2 || batches > W) && lq_aligned(a.scales, 16) && lq_aligned(a.zeros, 16) &&
                    2 * q_bytes <= (size_t)64 * W * 2 * 16;
    if (qs)
        hipLaunchKernelGGL((gemv_kernel<W, MP, NT, true>), dim3(a.N / (16 * NT)), dim3(64 * W), 2 * q_bytes + 2 * 16 * NT * 16, a.st,
                           (const unsigned short *)a.x, (const unsigned char *)a.codes, (const unsigned short *)a.scales,
                           (const unsigned short *)a.zeros, (const unsigned short *)a.bias, (unsigned short *)a.y, a.M, a.N, a.K);
    else
        hipLaunchKernelGGL((gemv_kernel<W, MP, NT, false>), dim3(a.N / (16 * NT)), dim3(64 * W), 0, a.st,
                           (const unsigned short *)a.x, (const unsigned char *)a.codes, (const unsigned short *)a.scales,
                           (const unsigned short *)a.zeros, (const unsigned short *)a.bias, (unsigned short *)a.y, a.M, a.N, a.K);
}

// Waves per workgroup: as many as there are batches, up to the cap, in powers of two. More waves
// mean more of the matrix in flight at once, which matters more than an even split of the batches
// (K = 11008 = 22 batches: 16 waves, 6 of them with two batches, beat 11 waves x 2).
int pick_waves(int batches, int max_waves) {
    int w = 2;
    while (w < batches && w < max_waves) w *= 2;
    return w;
}

template <int MP, int NT, int MAXW>
void launch_waves(int w, const GemvArgs &a) {
    switch (w) {
        case 2: launch_one<2, MP, NT>(a); break;
        case 4: launch_one<4, MP, NT>(a); break;
        case 8: if constexpr (MAXW >= 8) launch_one<8, MP, NT>(a); break;
        default: launch_one<MAXW, MP, NT>(a); break;
    }
}

}  // namespace

int lq_gemv_a16w4_launch(const void *x, const void *codes, const void *scales, const void *zeros, const void *bias,
                         void *y, int M, int N, int K, hipStream_t st) {
    // N % 16 == 0, K % 128 == 0 and 1 <= M <= 16 are guaranteed by the caller.
    const GemvArgs a = {x, codes, scales, zeros, bias, y, M, N, K, st};
    const int batches = (K / LQ_GROUP + 3) / 4;  // one batch of 4 groups per wave when possible: all of a
                                                 // wave's loads are then in flight at once
    if (M <= 4) {
        launch_waves<4, 1, 16>(pick_waves(batches, 16), a);
    } else if (M <= 8) {
        // 8 staged token rows (8.1 KB of LDS per wave): 8 waves with one 16-row tile, 16 when K has more than 16
        // batches (measured on 11008 x 4096 / 4096 x 11008 / 8192^2 at 8 tokens: 11.1 / 10.9 / 14.9 us against
        // 12.1 / 11.8 / 18.5 with 16 staged rows and the two-tile workgroups below)
        launch_waves<8, 1, 16>(pick_waves(batches, batches > 16 ? 16 : 8), a);
    } else if (N % 32 == 0 && N >= 32 * 256) {
        // many tokens and enough rows for one 32-row workgroup per CU: half the activation traffic;
        // 4 waves = 65 KB of staged activations: two workgroups per CU, all of them resident at once
        launch_waves<16, 2, 4>(pick_waves(batches, 4), a);
    } else {
        // 16 staged token rows cost a wave 16.25 KB of LDS, which caps the workgroup at 8 waves
        launch_waves<16, 1, 8>(pick_waves(batches, 8), a);
    }
    return lq_check_launch("lq_a16w4_fwd(gemv)");
}

// silu(x Wgate^T) * (x Wup^T) for 1 <= M <= 16: both matrices in one pass. N % 16 == 0 and K % 128 == 0 are
// guaranteed by the caller.
int lq_gemv_a16w4_gate_up_launch(const void *x, const void *codes_g, const void *scales_g, const void *zeros_g,
                                 const void *codes_u, const void *scales_u, const void *zeros_u, void *h, int M, int N, int K,
                                 hipStream_t st) {
    const GemvGuArgs a = {x, codes_g, scales_g, zeros_g, codes_u, scales_u, zeros_u, h, M, N, K, st};
    const int batches = (K / LQ_GROUP + 3) / 4;
    if (M <= 4) {
        switch (pick_waves(batches, 16)) {
            case 2: launch_gu<2, 4>(a); break;
            case 4: launch_gu<4, 4>(a); break;
            case 8: launch_gu<8, 4>(a); break;
            default: launch_gu<16, 4>(a); break;
        }
    } else {
        // 16 staged token rows cost a wave 16.25 KB of LDS: at most 8 waves
        switch (pick_waves(batches, 8)) {
            case 2: launch_gu<2, 16>(a); break;
            case 4: launch_gu<4, 16>(a); break;
            default: launch_gu<8, 16>(a); break;
        }
    }
    return lq_check_launch("lq_a16w4_gate_up_silu(gemv)");
}
