// Kernel (2a): LDS-tiled MFMA GEMMs for gfx950.
//
//   MODE_W4_FWD : Y[M,N]  = X[M,K]  . deq(W)[N,K]^T     (bf16 MFMA, int4 W dequantised into LDS)
//   MODE_W4_DX  : dX[M,K] = dY[M,N] . deq(W)[N,K]       (same, W tile transposed on the way out of LDS)
//   MODE_W8_DX  : dX[M,K] = dY[M,N] . (W8 * qs)[N,K]    (MODE_W4_DX with int8 codes and one bf16 scale per row n)
//
// (The forward pass of large grids runs the weights-direct kernel of lq_gemm_fwd.hip instead; the int8 GEMM of the
// A8W8 layers is lq_gemm_i8.hip, dispatched from this file.)
//
// Common structure. "A" is the activation-side operand, row-major with the reduction
// dimension contiguous. "B" is the weight-side operand, presented in LDS as
// [output column][reduction] exactly like A, except in MODE_W4_DX: there the reduction runs
// over n, the tile is kept in the weights' own [n][k] order (64 rows of 256 bytes, written as
// plain 16-byte pieces) and the math waves fetch their operands with the transposing LDS read
// ds_read_b64_tr_b16, so that the weight waves do the same cheap work in both directions.
// A tile row holds 128 bytes (64 bf16) = eight 16-byte chunks; one MFMA step
// consumes 32 bytes of every row (chunks 2s and 2s+1), i.e. 4 steps per tile. Bank conflicts of
// the 16-byte fragment reads (consecutive rows, same chunk) are avoided by XOR swizzles:
//   * chunk c of A row r sits at position c ^ ((r >> 1) & 7);
//   * chunk c of B row r sits at position c ^ ((r ^ (r >> 3)) & 7) (MODE_W4_DX: see dx_slot).
//
// The MFMA is issued with the weight fragment as the first operand and the activation
// fragment as the second, so that D[i][j] has i = output column (n), j = row (m): a
// lane then owns 4 consecutive n for one m; the epilogue regroups them through LDS into 16-byte
// pieces of full output rows.
//
// Wave specialisation. A workgroup has 2 x WM x WN waves, two per SIMD.
//   * The first WM x WN ("math") waves issue the MFMAs. They also fetch the A tiles, but with
//     LDS-direct loads (global_load_lds_dwordx4): no registers, no vector-ALU work, 8
//     instructions per tile, two tiles ahead of the tile being multiplied (three A buffers).
//     An LDS-direct load writes lane l at (wave base) + 16*l, so the swizzle is applied on the
//     global side: the lane that owns 16-byte slot s fetches the chunk that belongs there.
//   * The other WM x WN ("weight") waves turn packed int4 codes into bf16 B tiles: code loads two
//     tiles ahead into registers, dequantisation on the vector ALUs, LDS writes one tile ahead
//     (two B buffers). A single wave can issue one instruction every 4 cycles, so this
//     instruction-heavy work must not sit in the waves that feed the matrix pipe.
// One s_barrier per reduction tile orders the buffers. The barrier is issued without a memory
// fence and with explicit s_waitcnt values, so that the LDS-direct loads of tile kt+2 stay in
// flight across it; the loop is unrolled 6x so that every LDS buffer is a distinct __shared__
// array addressed by a compile-time index (the compiler then knows that a pending LDS-direct
// load never aliases the fragment reads it schedules next to it).
#include "lq_common.h"

#include <atomic>

#include <type_traits>

namespace {

enum { MODE_W4_FWD = 0, MODE_W4_DX = 1, MODE_W8_DX = 3 };

struct GemmParams {
    const void *a;        // activations: bf16 [M, R]
    const void *b;        // weights: packed int4 codes, or int8 [N, K] (MODE_W8_DX)
    const unsigned short *scales;
    const unsigned short *zeros;
    const unsigned short *bias;  // bf16 [out cols] or null
    void *c;                     // bf16 [M, C]
    int M;                       // rows of A / C
    int C;                       // output columns (N for fwd, K for dx)
    int R;                       // reduction length (K for fwd, N for dx)
    int Kw;                      // K of the weight matrix (row length of W in elements)
    int tiles_m, tiles_n;
    // split reduction: workgroup (tile, blockIdx.y) covers steps_per_split reduction steps from
    // blockIdx.y * steps_per_split and writes its fp32 partial tile to partial[blockIdx.y][M][C]
    int steps_per_split;
    float *partial;
    // measurement aid (null in normal use): workgroup w writes the shader-cycle counter and the
    // 100 MHz real-time counter at its start and end to clk[4 w .. 4 w + 3]
    unsigned long long *clk;
    // MODE_W4_DX epilogue forms (on the bf16-rounded product P, 8 columns per lane):
    //   EP_STORE   c = P
    //   EP_ADD     c = bf16(c + P)                                   (the second of two products that share their output)
    //   EP_SILU_BW c  = bf16(P * u * s * (1 + g * (1 - s))),  s = 1 / (1 + exp(-g))      (gradient of the gate product)
    //              c2 = bf16(P * g * s)                                                 (gradient of the up product)
    //              for P = the gradient of h = silu(g) * u; ep_g, ep_u: bf16 [M, C]
    int ep_mode;
    const unsigned short *ep_g, *ep_u;
    unsigned short *c2;
    // MODE_W4_DX, two products into one output: c = a * deq(b) + a2 * deq(b2), both pairs of the shape (M, R) x (R, C).
    // The reduction runs over the first pair's R / 64 steps and then over the second's; a2 = null: one product.
    const void *a2, *b2;
    const unsigned short *scales2, *zeros2;
};

enum { EP_STORE = 0, EP_ADD = 1, EP_SILU_BW = 2 };

typedef __attribute__((address_space(3))) void lds_void;
typedef const __attribute__((address_space(1))) void gbl_void;
typedef short v4s_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) v4s_t lds_v4s_t;

template <int I>
using ic = std::integral_constant<int, I>;

__device__ __forceinline__ int swz(int row) { return (row ^ (row >> 3)) & 7; }
// dX tile ([n][k], 256-byte rows of eight 32-byte pieces c32 = k / 16, each two 16-byte halves).
// Byte offset within row n of half `half` of piece c32, with j = n & 3:
//   piece = ((c32 >> 1) ^ j) | (((c32 & 1) ^ (j >> 1)) << 2),  half ^= j & 1.
// Writes: a staging instruction puts lane (row, quarter q) on piece c32 = 2q + e with e and the half
// fixed. LDS takes a 16-byte write instruction 8 lanes (2 rows x 4 quarters, 128 bytes) at a time
// over 32 banks: their slots modulo 8 are 2 (q ^ j) + (half ^ (j & 1)), all different; the 16
// lanes of 4 rows also fall on 16 different slots of 256 bytes. Reads: a transposing read covers,
// per 32 lanes, rows n..n+3 at the two pieces (c, c + 1), c even: pieces (q ^ j) and (q ^ j) + 4
// for j = 0..3, every bank once. (An earlier layout spread the quarters over pieces 2q ^ f(j): two
// of the four quarters of a row then shared their slot modulo 8, and the counters showed one
// bank-conflict cycle per write cycle.)
__device__ __forceinline__ int dx_slot(int row, int c32, int half) {
    const int j = row & 3;
    const int piece = ((c32 >> 1) ^ j) | (((c32 & 1) ^ (j >> 1)) << 2);
    return (piece << 5) | ((half ^ (j & 1)) << 4);
}

template <int MODE, int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(128 * WM * WN) void gemm_kernel(GemmParams p) {
    constexpr bool kDx = MODE == MODE_W4_DX || MODE == MODE_W8_DX;  // reduction over n, weight tile kept in [n][k] order
    constexpr int NT = 64 * WM * WN;           // threads per role
    constexpr int TM = BM / WM, TN = BN / WN;  // wave tile
    constexpr int FM = TM / 32, FN = TN / 32;  // 32x32 fragments per wave tile
    constexpr int ROWB = 128;                  // bytes of data per tile row (and per LDS row of B)
    constexpr int AROW = 128;                  // bytes per LDS row of A
    constexpr int APT = BM * 8 / NT;           // 16-byte LDS slots of A filled per math thread per tile
    constexpr int A_BYTES = APT * NT * 16, B_BYTES = BN * ROWB;
    constexpr int ESZ = 2;
    constexpr int RT = ROWB / ESZ;  // reduction elements per tile: 64
    static_assert(TM % 32 == 0 && TN % 32 == 0, "wave tile must be a multiple of 32x32");
    static_assert((BN * 8) % NT == 0, "B staging must divide evenly");
    static_assert(A_BYTES == BM * AROW && (BM * 8) % NT == 0, "A staging must divide evenly");

    __shared__ __attribute__((aligned(16))) unsigned char lds_a0[A_BYTES];
    __shared__ __attribute__((aligned(16))) unsigned char lds_a1[A_BYTES];
    __shared__ __attribute__((aligned(16))) unsigned char lds_a2[A_BYTES];
    __shared__ __attribute__((aligned(16))) unsigned char lds_b0[B_BYTES];
    __shared__ __attribute__((aligned(16))) unsigned char lds_b1[B_BYTES];
    auto abuf = [&](auto i) -> unsigned char * {
        constexpr int I = decltype(i)::value;
        if constexpr (I == 0) return lds_a0;
        else if constexpr (I == 1) return lds_a1;
        else return lds_a2;
    };
    auto bbuf = [&](auto i) -> unsigned char * {
        constexpr int I = decltype(i)::value;
        if constexpr (I == 0) return lds_b0;
        else return lds_b1;
    };

    // wave index as a scalar, so that the role split is a uniform branch and LDS-direct
    // destinations are wave-uniform
    const int wave_all = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    unsigned long long clk_t0 = 0, clk_r0 = 0;
    if (p.clk) {
        clk_t0 = __builtin_amdgcn_s_memtime();
        clk_r0 = __builtin_amdgcn_s_memrealtime();
    }
    const bool is_weight_wave = wave_all >= WM * WN;
    const int wave = wave_all % (WM * WN);
    const int lane = threadIdx.x & 63;
    const int tid = wave * 64 + lane;  // index within the role
    const int wm = wave % WM, wn = wave / WM;

    // Workgroup ids are dealt round-robin over the 8 XCDs (id % 8). Give each XCD a contiguous
    // range of the tile sequence, and order that sequence in bands of GN tile columns walked
    // row by row: the ~32 workgroups resident on an XCD then form a 2 x 16 patch that shares
    // 2 A row-blocks and 16 B column-blocks in that XCD's L2.
    const int nwg = p.tiles_m * p.tiles_n;
    int id = blockIdx.x;
    {
        const int per = nwg / 8;
        if (id < per * 8) id = (id % 8) * per + id / 8;
    }
    constexpr int GN = 16;
    const int band = id / (p.tiles_m * GN);
    const int within = id - band * (p.tiles_m * GN);
    const int rest = p.tiles_n - band * GN;
    const int bw = rest < GN ? rest : GN;
    const int tile_m = within / bw, tile_n = band * GN + within % bw;
    const int m0 = tile_m * BM, c0 = tile_n * BN;
    // reduction steps of this workgroup: all of them, or one slice of a split reduction
    const int k0 = p.partial ? (int)blockIdx.y * p.steps_per_split : 0;
    const bool pair = MODE == MODE_W4_DX && p.a2 != nullptr;  // never together with a split reduction
    const int n1 = p.R / RT;                                  // steps of the first (or only) product
    const int nk = p.partial ? (n1 - k0 < p.steps_per_split ? n1 - k0 : p.steps_per_split) : pair ? 2 * n1 : n1;
    const int groups_per_row = p.Kw / LQ_GROUP;

    if (is_weight_wave) {
        // ======================= weight waves: B tiles =======================
        //   W4_FWD  : NW code words (8 k each) of one weight row -> NW 16-byte chunks of that row.
        //   W4_DX   : 4 code words (32 k) of one weight row n -> four 16-byte pieces of LDS row n. The
        //             tile stays in the weights' own [n][k] order; the math waves transpose it on
        //             the way out of LDS (ds_read_b64_tr_b16).
        constexpr int NW = (MODE == MODE_W4_FWD) ? BN * 8 / NT : 1;  // tile has BN rows x 8 words
        static_assert(MODE != MODE_W4_FWD || NW == 2 || NW == 4 || NW == 8, "bad fwd staging split");
        static_assert(!kDx || (BN == 128 && NT == 256), "dX staging: 64 rows x 4 threads");
        constexpr int NSZ = 1;
        constexpr int NWORDS = (MODE == MODE_W4_DX) ? 4 : (MODE == MODE_W8_DX) ? 8 : NW;

        const unsigned char *b_src[1];
        const unsigned short *s_src[NSZ];
        const unsigned short *z_src[NSZ];
        const unsigned char *b_src2 = nullptr;  // W4_DX: the second product's codes, scales and zeros
        const unsigned short *s_src2 = nullptr, *z_src2 = nullptr;
        int b_row = 0, b_w0 = 0;  // W4_FWD: LDS row and first word; W4_DX: LDS row (n) and quarter of the row

        if constexpr (MODE == MODE_W4_FWD) {
            constexpr int TPR = 8 / NW;  // threads per weight row
            b_row = tid / TPR;
            b_w0 = (tid % TPR) * NW;
            int gr = c0 + b_row;
            gr = gr < p.C ? gr : p.C - 1;
            b_src[0] = (const unsigned char *)p.b + (long long)gr * (p.Kw / 2) + b_w0 * 4 + (long long)k0 * 32;
            s_src[0] = p.scales + (long long)gr * groups_per_row + k0 / 2;  // k0 is even: a group is two steps
            z_src[0] = p.zeros + (long long)gr * groups_per_row + k0 / 2;
        } else if constexpr (MODE == MODE_W8_DX) {
            b_row = tid >> 2;  // n within the tile
            b_w0 = tid & 3;    // 32 of the tile's 128 output columns k = 32 code bytes
            b_src[0] = (const unsigned char *)p.b + ((long long)k0 * 64 + b_row) * p.Kw + c0 + b_w0 * 32;
            s_src[0] = p.scales + ((long long)k0 * 64 + b_row);  // one scale per weight row n
            z_src[0] = nullptr;
        } else {
            b_row = tid >> 2;  // n within the tile (the tile offset along n is added per tile)
            b_w0 = tid & 3;    // 32 of the tile's 128 output columns k
            b_src[0] = (const unsigned char *)p.b + ((long long)k0 * 64 + b_row) * (p.Kw / 2) + c0 / 2 + b_w0 * 16;
            const int g = (c0 + b_w0 * 32) / LQ_GROUP;
            s_src[0] = p.scales + ((long long)k0 * 64 + b_row) * groups_per_row + g;
            z_src[0] = p.zeros + ((long long)k0 * 64 + b_row) * groups_per_row + g;
            if (pair) {
                b_src2 = (const unsigned char *)p.b2 + (long long)b_row * (p.Kw / 2) + c0 / 2 + b_w0 * 16;
                s_src2 = p.scales2 + (long long)b_row * groups_per_row + g;
                z_src2 = p.zeros2 + (long long)b_row * groups_per_row + g;
            }
        }

        struct Stage {
            unsigned w[NWORDS];  // code words
            unsigned short s[NSZ], z[NSZ];
        };
        Stage S0, S1;

        auto load_b = [&](int kt, Stage &S) {
            if constexpr (MODE == MODE_W4_FWD) {
                const unsigned char *src = b_src[0] + (long long)kt * 32;
                if constexpr (NW == 8) {
                    u32x4_t v0 = *reinterpret_cast<const u32x4_t *>(src), v1 = *reinterpret_cast<const u32x4_t *>(src + 16);
#pragma unroll
                    for (int i = 0; i < 4; ++i) { S.w[i] = v0[i]; S.w[4 + i] = v1[i]; }
                } else if constexpr (NW == 4) {
                    u32x4_t v = *reinterpret_cast<const u32x4_t *>(src);
#pragma unroll
                    for (int i = 0; i < 4; ++i) S.w[i] = v[i];
                } else {
                    u32x2_t v = *reinterpret_cast<const u32x2_t *>(src);
                    S.w[0] = v[0]; S.w[1] = v[1];
                }
                S.s[0] = s_src[0][kt >> 1];
                S.z[0] = z_src[0][kt >> 1];
            } else if constexpr (MODE == MODE_W8_DX) {
                const long long row_off = (long long)kt * 64;
                const u32x4_t v0 = *reinterpret_cast<const u32x4_t *>(b_src[0] + row_off * p.Kw);
                const u32x4_t v1 = *reinterpret_cast<const u32x4_t *>(b_src[0] + row_off * p.Kw + 16);
#pragma unroll
                for (int i = 0; i < 4; ++i) { S.w[i] = v0[i]; S.w[4 + i] = v1[i]; }
                S.s[0] = s_src[0][row_off];
            } else {
                const bool second = kt >= n1 && pair;
                const long long row_off = (long long)(second ? kt - n1 : kt) * 64;
                u32x4_t v = *reinterpret_cast<const u32x4_t *>((second ? b_src2 : b_src[0]) + row_off * (p.Kw / 2));
#pragma unroll
                for (int i = 0; i < 4; ++i) S.w[i] = v[i];
                S.s[0] = (second ? s_src2 : s_src[0])[row_off * groups_per_row];
                S.z[0] = (second ? z_src2 : z_src[0])[row_off * groups_per_row];
            }
        };

        auto store_b = [&](unsigned char *lb, Stage &S) {
            if constexpr (MODE == MODE_W4_FWD) {
                const float s = lq_bf16_bits_to_f32(S.s[0]);
                const float nzs = -(lq_bf16_bits_to_f32(S.z[0]) * s);
                const float s512 = s * 512.0f;  // the codes come out of the conversion as q/512
#pragma unroll
                for (int w = 0; w < NW; ++w) {
                    float f[8];
                    lq_dequant_word_f32(S.w[w], s512, nzs, f);
                    const int ch = b_w0 + w;
                    u32x4_t v = {lq_pack_bf16(f[0], f[1]), lq_pack_bf16(f[2], f[3]), lq_pack_bf16(f[4], f[5]),
                                 lq_pack_bf16(f[6], f[7])};
                    *reinterpret_cast<u32x4_t *>(lb + b_row * ROWB + ((ch ^ swz(b_row)) << 4)) = v;
                }
            } else if constexpr (MODE == MODE_W8_DX) {
                // bf16(w8 * qs), the weight the reference's backward multiplies with (utils/quant.py:200-201): the
                // byte + 128 converts with one instruction, and fma(u, s, -128 s) is the exact product (16 bits)
                const float s = lq_bf16_bits_to_f32(S.s[0]);
                const float off = -128.0f * s;
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const unsigned a = S.w[2 * w] ^ 0x80808080u, b = S.w[2 * w + 1] ^ 0x80808080u;
                    u32x4_t v = {lq_pack_bf16(fmaf((float)((a >> 0) & 0xFFu), s, off), fmaf((float)((a >> 8) & 0xFFu), s, off)),
                                 lq_pack_bf16(fmaf((float)((a >> 16) & 0xFFu), s, off), fmaf((float)((a >> 24) & 0xFFu), s, off)),
                                 lq_pack_bf16(fmaf((float)((b >> 0) & 0xFFu), s, off), fmaf((float)((b >> 8) & 0xFFu), s, off)),
                                 lq_pack_bf16(fmaf((float)((b >> 16) & 0xFFu), s, off), fmaf((float)((b >> 24) & 0xFFu), s, off))};
                    const int c32 = b_w0 * 2 + (w >> 1);  // 32-byte piece of the 256-byte row
                    *reinterpret_cast<u32x4_t *>(lb + b_row * 256 + dx_slot(b_row, c32, w & 1)) = v;
                }
            } else {
                const float s = lq_bf16_bits_to_f32(S.s[0]);
                const float nzs = -(lq_bf16_bits_to_f32(S.z[0]) * s);
                const float s512 = s * 512.0f;  // the codes come out of the conversion as q/512
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    float f[8];
                    lq_dequant_word_f32(S.w[w], s512, nzs, f);
                    u32x4_t v = {lq_pack_bf16(f[0], f[1]), lq_pack_bf16(f[2], f[3]), lq_pack_bf16(f[4], f[5]),
                                 lq_pack_bf16(f[6], f[7])};
                    const int c32 = b_w0 * 2 + (w >> 1);  // 32-byte piece of the 256-byte row
                    *reinterpret_cast<u32x4_t *>(lb + b_row * 256 + dx_slot(b_row, c32, w & 1)) = v;
                }
            }
        };

        // Barrier after the LDS writes of this wave have completed (no fence: see file header).
        auto publish = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

        load_b(0, S0);
        load_b(nk > 1 ? 1 : 0, S1);
        store_b(lds_b0, S0);
        publish();
        // iteration kt: codes of tile kt+2 -> registers, tile kt+1 -> LDS buffer (kt+1)&1
        int kt = 0;
        for (; kt + 2 <= nk; kt += 2) {
            load_b(kt + 2 < nk ? kt + 2 : nk - 1, S0);
            store_b(lds_b1, S1);
            publish();
            load_b(kt + 3 < nk ? kt + 3 : nk - 1, S1);
            if (kt + 2 < nk) store_b(lds_b0, S0);
            publish();
        }
        if (kt < nk) publish();  // odd tile count: the last tile has nothing left to prepare
        return;
    }

    // =========================== math waves: A tiles + MFMA ===========================
    static_assert(APT <= 30, "vmcnt range");
    // Lane-varying 32-bit byte offsets into A; the tile offset (kt * 128 bytes) is wave-uniform.
    unsigned a_off[APT];
    const long long lda = (long long)p.R * ESZ;
#pragma unroll
    for (int i = 0; i < APT; ++i) {
        const int slot = i * NT + tid;  // LDS slot: row slot/8, position slot%8 holds chunk pos ^ swizzle
        const int row = slot >> 3;
        const int ch = (slot & 7) ^ ((row >> 1) & 7);
        int gr = m0 + row;
        gr = gr < p.M ? gr : p.M - 1;
        a_off[i] = (unsigned)((gr - m0) * lda + ch * 16);
    }
    const unsigned char *a_base = (const unsigned char *)p.a + m0 * lda + (long long)k0 * ROWB;
    const unsigned char *a_base2 = pair ? (const unsigned char *)p.a2 + m0 * lda : a_base;
    // LDS-direct load: lane l of the wave writes 16 bytes at (wave-uniform base) + 16*l. Written as
    // inline assembly (M0 = LDS base, one wait state, then the load with a scalar base and a 32-bit
    // lane offset) so that the compiler's wait-count insertion does not see an LDS write it cannot
    // tell apart from the fragment reads and park a vmcnt(0) in front of them: the explicit
    // s_waitcnt before each barrier is the only ordering these loads need.
    static_assert(APT % 4 == 0, "A loads are issued in four parts per tile");
    // part q (0..3) of a tile's loads: APT/4 of them
    auto issue_a_part = [&](int kt, unsigned char *la, int q) {
        const bool second = kt >= n1 && pair;
        const unsigned long long addr = (unsigned long long)((second ? a_base2 : a_base) + (long long)(second ? kt - n1 : kt) * ROWB);
        // the load takes its base from scalar registers
        const unsigned char *src = (const unsigned char *)(((unsigned long long)(unsigned)__builtin_amdgcn_readfirstlane((int)(addr >> 32)) << 32) |
                                                           (unsigned)__builtin_amdgcn_readfirstlane((int)addr));
#pragma unroll
        for (int i = q * (APT / 4); i < (q + 1) * (APT / 4); ++i) {
            const unsigned lds_addr = (unsigned)reinterpret_cast<size_t>((lds_void *)(la + (i * NT + wave * 64) * 16));
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                         :: "s"(lds_addr), "v"(a_off[i]), "s"(src) : "memory");
        }
    };
    auto issue_a = [&](int kt, unsigned char *la) {
#pragma unroll
        for (int q = 0; q < 4; ++q) issue_a_part(kt, la, q);
    };

    f32x16_t acc[FN][FM];
#pragma unroll
    for (int i = 0; i < FN; ++i)
#pragma unroll
        for (int j = 0; j < FM; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    const int frag_row = lane & 31, kh = lane >> 5;
    // A fragment of slice ks: row wm*TM + 32i + frag_row, chunk 2ks + kh at position chunk ^ ((row >> 1) & 7)
    int a_frag[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
        a_frag[ks] = (wm * TM + frag_row) * AROW + (((2 * ks + kh) ^ ((frag_row >> 1) & 7)) << 4);  // + i*32*AROW
    int b_frag_off[FN], b_frag_swz[FN];
#pragma unroll
    for (int i = 0; i < FN; ++i) {
        const int row = wn * TN + i * 32 + frag_row;
        b_frag_off[i] = row * ROWB;
        b_frag_swz[i] = swz(row);
    }
    // dX: the B tile is stored [n][k]; an MFMA lane needs 8 consecutive n of one k. A transposing
    // read hands lane i of each 16-lane block the column i%4 of the four 8-byte rows addressed by
    // lanes i/4, i/4 + 4, i/4 + 8, i/4 + 12 of that block. Let block lane r address row n0 + r/4
    // at columns k0 + 4*(r%4): lane i then receives W[n0 .. n0+3][k0 + i]. The four blocks of a
    // wave are (k0, n0) = (0, 0), (16, 0), (0, 8), (16, 8); a second read 4 rows further down
    // completes the 8 n of the operand.
    int dx_off[FN];
    if constexpr (kDx) {
        const int i16 = lane & 15, blk = lane >> 4;
        const int row_lane = 8 * (blk >> 1) + (i16 >> 2), colblk = blk & 1;  // row_lane & 3 is the row's j
#pragma unroll
        for (int i = 0; i < FN; ++i) {
            const int c32 = (wn * TN + i * 32) / 16 + colblk;
            dx_off[i] = row_lane * 256 + dx_slot(row_lane, c32, (i16 & 3) >> 1) + (i16 & 1) * 8;
        }
    }
    auto read_frags = [&](const unsigned char *la, const unsigned char *lb, int ks, u32x4_t *af, u32x4_t *bf) {
        const int ch = 2 * ks + kh;
#pragma unroll
        for (int i = 0; i < FM; ++i)
            af[i] = *reinterpret_cast<const u32x4_t *>(la + a_frag[ks] + i * 32 * AROW);
        if constexpr (kDx) {
#pragma unroll
            for (int i = 0; i < FN; ++i) {
                const v4s_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_t *)(lb + dx_off[i] + ks * 4096));
                const v4s_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_t *)(lb + dx_off[i] + ks * 4096 + 1024));
                const u32x2_t l2 = __builtin_bit_cast(u32x2_t, lo), h2 = __builtin_bit_cast(u32x2_t, hi);
                bf[i] = u32x4_t{l2[0], l2[1], h2[0], h2[1]};
            }
        } else {
#pragma unroll
            for (int i = 0; i < FN; ++i)
                bf[i] = *reinterpret_cast<const u32x4_t *>(lb + b_frag_off[i] + ((ch ^ b_frag_swz[i]) << 4));
        }
    };
    auto mfma_step = [&](const u32x4_t *af, const u32x4_t *bf) {
#pragma unroll
        for (int i = 0; i < FN; ++i)
#pragma unroll
            for (int j = 0; j < FM; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, bf[i]),
                                                                   __builtin_bit_cast(bf16x8_t, af[j]), acc[i][j], 0, 0, 0);
    };

    // Tile kt: A in buffer kt%3, B in buffer kt%2; the fragments of its first reduction slice are
    // already in af[0] / bf[0]. Four slices of FN*FM MFMAs; each also reads the fragments of the
    // next slice and issues a quarter of the A loads of tile kt+2 (into the buffer tile kt-1 left;
    // one burst of them would hold the wave at the memory pipeline's queue with its MFMAs behind
    // it). The tile's one synchronisation point sits before the last slice: this wave's part of
    // tile kt+1 has landed (all but the 3/4 of tile kt+2's loads issued since), its fragment reads of
    // tile kt have all returned, the weight waves have published B tile kt+1. The last slice then
    // already reads the first fragments of tile kt+1, so the MFMA stream does not drain at the
    // tile boundary. After the barrier nobody reads tile kt's buffers any more, which is what
    // lets the weight waves overwrite its B buffer and the next tile's loads its A buffer.
    u32x4_t af[2][FM], bf[2][FN];
    auto tile_step = [&](int kt, auto ai, auto bi) {
        constexpr int AI = decltype(ai)::value, BI = decltype(bi)::value;
        const unsigned char *la = abuf(ic<AI>()), *lb = bbuf(ic<BI>());
        const unsigned char *la_next = abuf(ic<(AI + 1) % 3>()), *lb_next = bbuf(ic<BI ^ 1>());
        unsigned char *la_load = abuf(ic<(AI + 2) % 3>());
        const int kt_a = kt + 2 < nk ? kt + 2 : nk - 1;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            if (t == 3) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(3 * APT / 4) : "memory");
            if (t < 3) read_frags(la, lb, t + 1, af[(t + 1) & 1], bf[(t + 1) & 1]);
            else read_frags(la_next, lb_next, 0, af[0], bf[0]);
            issue_a_part(kt_a, la_load, t);
            mfma_step(af[t & 1], bf[t & 1]);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    issue_a(0, lds_a0);
    issue_a(nk > 1 ? 1 : 0, lds_a1);
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(APT) : "memory");
    read_frags(lds_a0, lds_b0, 0, af[0], bf[0]);
    __builtin_amdgcn_sched_barrier(0);
    int kt = 0;
    for (; kt + 6 <= nk; kt += 6) {
        tile_step(kt, ic<0>(), ic<0>());
        tile_step(kt + 1, ic<1>(), ic<1>());
        tile_step(kt + 2, ic<2>(), ic<0>());
        tile_step(kt + 3, ic<0>(), ic<1>());
        tile_step(kt + 4, ic<1>(), ic<0>());
        tile_step(kt + 5, ic<2>(), ic<1>());
    }
    // remainder of 0..5 tiles; kt is a multiple of 6 here, so the buffer phases restart at 0
    const int rem = nk - kt;
    if (rem > 0) tile_step(kt, ic<0>(), ic<0>());
    if (rem > 1) tile_step(kt + 1, ic<1>(), ic<1>());
    if (rem > 2) tile_step(kt + 2, ic<2>(), ic<0>());
    if (rem > 3) tile_step(kt + 3, ic<0>(), ic<1>());
    if (rem > 4) tile_step(kt + 4, ic<1>(), ic<0>());

    // the clamped prefetches issued by the last two tiles are still writing LDS: drain them
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    // ---- epilogue -----------------------------------------------------------
    // acc[i][j][r]: column c = c0 + wn*TN + i*32 + 8*(r/4) + 4*(lane/32) + r%4, row m = m0 + wm*TM + j*32 + lane%32.
    // A lane holds 4 consecutive columns of one row; stored straight from the registers an
    // instruction would touch 32 rows with 16 bytes each. Every math wave passes its block through
    // LDS instead, 32 rows (one j) at a time, and stores 16 bytes per lane with TN/8 lanes on the
    // contiguous bytes of a row. The B buffers are free here (the weight waves wrote their last
    // tile before the final barrier, and no load is in flight into them); a wave's staging area
    // is private, row pitch TN*2 + 16 bytes.
    if (p.partial) {
        // split reduction: the fp32 accumulators as they are, 16 bytes per lane; a second kernel adds
        // the slices in a fixed order, adds the bias and rounds
        float *part = p.partial + (long long)blockIdx.y * p.M * p.C;
#pragma unroll
        for (int j = 0; j < FM; ++j) {
            const int m = m0 + wm * TM + j * 32 + frag_row;
            if (m >= p.M) continue;
#pragma unroll
            for (int i = 0; i < FN; ++i)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int c = c0 + wn * TN + i * 32 + 8 * q + 4 * kh;
                    if (c >= p.C) continue;
                    f32x4_t v = {(float)acc[i][j][4 * q], (float)acc[i][j][4 * q + 1], (float)acc[i][j][4 * q + 2],
                                 (float)acc[i][j][4 * q + 3]};
                    *reinterpret_cast<f32x4_t *>(part + (long long)m * p.C + c) = v;
                }
        }
        return;
    }
    unsigned short *out = (unsigned short *)p.c;
    constexpr int EP = TN * 2 + 16;
    constexpr int EP_WAVE = 32 * EP;
    constexpr int EP_PER_BUF = B_BYTES / EP_WAVE;
    static_assert(WM * WN <= 2 * EP_PER_BUF, "epilogue staging does not fit the B buffers");
    unsigned char *ep = (wave >= EP_PER_BUF ? lds_b1 : lds_b0) + (wave % EP_PER_BUF) * EP_WAVE;
    constexpr int LPR = TN / 8;        // lanes per staged row (16 bytes each)
    constexpr int RPI = 64 / LPR;      // rows per store instruction
    const int ep_row = lane / LPR, ep_chunk = lane % LPR;
    const int c_lane = c0 + wn * TN + ep_chunk * 8;
    float bias_v[FN][4][4];
#pragma unroll
    for (int i = 0; i < FN; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int c = c0 + wn * TN + i * 32 + 8 * q + 4 * kh;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const bool in = c + r < p.C;
                bias_v[i][q][r] = (p.bias && in) ? lq_bf16_bits_to_f32(p.bias[c + r]) : 0.0f;
            }
        }
#pragma unroll
    for (int j = 0; j < FM; ++j) {
#pragma unroll
        for (int i = 0; i < FN; ++i) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                float v[4];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    v[r] = acc[i][j][4 * q + r];
                    if (p.bias) v[r] += bias_v[i][q][r];
                }
                u32x2_t o = {lq_pack_bf16(v[0], v[1]), lq_pack_bf16(v[2], v[3])};
                *reinterpret_cast<u32x2_t *>(ep + frag_row * EP + (i * 32 + 8 * q + 4 * kh) * 2) = o;
            }
        }
#pragma unroll
        for (int it = 0; it < 32 / RPI; ++it) {
            const int row = it * RPI + ep_row;
            const u32x4_t o = *reinterpret_cast<const u32x4_t *>(ep + row * EP + ep_chunk * 16);
            const int mm = m0 + wm * TM + j * 32 + row;
            if (mm < p.M && c_lane < p.C) {
                const long long off = (long long)mm * p.C + c_lane;
                if (kDx && p.ep_mode == EP_ADD) {
                    const u32x4_t old = *reinterpret_cast<const u32x4_t *>(out + off);
                    u32x4_t sum;
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        sum[e] = lq_pack_bf16(lq_bf16_lo(old[e]) + lq_bf16_lo(o[e]), lq_bf16_hi(old[e]) + lq_bf16_hi(o[e]));
                    *reinterpret_cast<u32x4_t *>(out + off) = sum;
                } else if (kDx && p.ep_mode == EP_SILU_BW) {
                    const u32x4_t g8 = *reinterpret_cast<const u32x4_t *>(p.ep_g + off);
                    const u32x4_t u8 = *reinterpret_cast<const u32x4_t *>(p.ep_u + off);
                    u32x4_t dg, du;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        float rg[2], ru[2];
#pragma unroll
                        for (int hh = 0; hh < 2; ++hh) {
                            const float d = hh ? lq_bf16_hi(o[e]) : lq_bf16_lo(o[e]);
                            const float g = hh ? lq_bf16_hi(g8[e]) : lq_bf16_lo(g8[e]);
                            const float u = hh ? lq_bf16_hi(u8[e]) : lq_bf16_lo(u8[e]);
                            const float sg = __builtin_amdgcn_rcpf(1.0f + __expf(-g));
                            rg[hh] = d * u * (sg * (1.0f + g * (1.0f - sg)));
                            ru[hh] = d * (g * sg);
                        }
                        dg[e] = lq_pack_bf16(rg[0], rg[1]);
                        du[e] = lq_pack_bf16(ru[0], ru[1]);
                    }
                    *reinterpret_cast<u32x4_t *>(out + off) = dg;
                    *reinterpret_cast<u32x4_t *>(p.c2 + off) = du;
                } else {
                    *reinterpret_cast<u32x4_t *>(out + off) = o;
                }
            }
        }
    }
    if (p.clk && threadIdx.x == 0) {
        unsigned long long *c = p.clk + 4ll * (blockIdx.x + (long long)blockIdx.y * gridDim.x);
        c[0] = clk_t0; c[1] = __builtin_amdgcn_s_memtime(); c[2] = clk_r0; c[3] = __builtin_amdgcn_s_memrealtime();
    }
}

template <int MODE, int BM, int BN, int WM, int WN>
int launch_gemm(GemmParams p, hipStream_t st, const char *who) {
    p.tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.C + BN - 1) / BN;
    auto kern = gemm_kernel<MODE, BM, BN, WM, WN>;
    const long long nwg = (long long)p.tiles_m * p.tiles_n;
    if (nwg > 0x7FFFFFFFll) return lq_fail(LQ_ERR_BAD_ARG, "%s: problem too large", who);
    const int total_steps = p.R / 64;
    const unsigned splits = p.partial ? (unsigned)((total_steps + p.steps_per_split - 1) / p.steps_per_split) : 1u;
    hipLaunchKernelGGL(kern, dim3((unsigned)nwg, splits), dim3(128 * WM * WN), 0, st, p);
    return lq_check_launch(who);
}

// out[m][c] = bf16(sum over the slices, in order, of partial[s][m][c] (+ bias[c])); 8 columns per thread
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float *__restrict__ partial,
                                                           const unsigned short *__restrict__ bias,
                                                           unsigned short *__restrict__ out, long long MC, int C, int splits) {
    const long long e = ((long long)blockIdx.x * 256 + threadIdx.x) * 8;
    if (e >= MC) return;
    float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < splits; ++s) {
        const f32x4_t a = *reinterpret_cast<const f32x4_t *>(partial + (long long)s * MC + e);
        const f32x4_t b = *reinterpret_cast<const f32x4_t *>(partial + (long long)s * MC + e + 4);
#pragma unroll
        for (int k = 0; k < 4; ++k) { v[k] += a[k]; v[4 + k] += b[k]; }
    }
    if (bias) {
        const int c = (int)(e % C);
#pragma unroll
        for (int k = 0; k < 8; ++k) v[k] += lq_bf16_bits_to_f32(bias[c + k]);
    }
    *reinterpret_cast<u32x4_t *>(out + e) = u32x4_t{lq_pack_bf16(v[0], v[1]), lq_pack_bf16(v[2], v[3]),
                                                    lq_pack_bf16(v[4], v[5]), lq_pack_bf16(v[6], v[7])};
}

}  // namespace

// weights-direct forward GEMM (lq_gemm_fwd.hip)
long long lq_gemm_fwd_direct_workgroups(int M, int N);
long long lq_gemm_fwd_direct128_workgroups(int M, int N);
int lq_gemm_fwd_direct_launch(const void *x, const void *codes, const void *scales, const void *zeros, const void *bias,
                              void *y, int M, int N, int K, hipStream_t st, unsigned long long *clk, bool narrow);
int lq_gemm_fwd_gate_up_launch(const void *x, const void *codes_g, const void *scales_g, const void *zeros_g,
                               const void *codes_u, const void *scales_u, const void *zeros_u, void *h, void *g_out, void *u_out,
                               int M, int N, int K, hipStream_t st);

// int8 GEMM with 256 x 256 tiles (lq_gemm_i8.hip)
long long lq_gemm_i8_256_workgroups(int M, int N);
int lq_gemm_i8_tile_launch(const void *x8, const void *w8, const float *sx, const void *sw, bool sw_bf16, const void *bias, void *y,
                           int *acc_or_null, int M, int N, int K, int tile, int stages, hipStream_t st);

// GEMV path (lq_gemv.hip)
int lq_gemv_a16w4_launch(const void *x, const void *codes, const void *scales, const void *zeros, const void *bias,
                         void *y, int M, int N, int K, hipStream_t st);
int lq_gemv_a16w4_gate_up_launch(const void *x, const void *codes_g, const void *scales_g, const void *zeros_g,
                                 const void *codes_u, const void *scales_u, const void *zeros_u, void *h, int M, int N, int K,
                                 hipStream_t st);

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

// Split reduction for grids that fill less than half of the compute units: the reduction is cut
// into up to 8 slices of an even number of steps (at least 8) so that every unit gets at most one
// workgroup, fp32 partial tiles go to the caller's workspace, then a reduce kernel adds them. Both
// staged tile heights are tried (128 x 128 at ~0.56 us per step, 256 x 128 at pace_big); the plan
// with the smaller estimated time is returned (splits = 1: do not split). The estimate counts the
// partial tiles written and read back through the last-level cache at ~5 TB/s and ~3 us for the
// second launch.
struct SplitPlan {
    int splits = 1, steps_per_split = 0;
    bool big = false;
    double est_us = 1e30;
};

static SplitPlan plan_split(long long M, long long C, int total_steps, size_t ws_bytes, double pace_big, long long cus) {
    SplitPlan best;
    if (!ws_bytes) return best;
    const long long fit = (long long)(ws_bytes / ((size_t)M * C * 4));
    for (int big = 0; big < 2; ++big) {
        const long long tiles = ((M + (big ? 255 : 127)) / (big ? 256 : 128)) * ((C + 127) / 128);
        if (tiles * 2 > cus) continue;
        long long S = cus / tiles;
        if (S > 8) S = 8;
        if (S > fit) S = fit;
        if (S < 2) continue;
        int per = (int)((total_steps + S - 1) / S);
        per += per & 1;
        if (per < 8) per = 8;
        S = (total_steps + per - 1) / per;
        if (S < 2) continue;
        // with more than three quarters of the units busy the clock gives ~9 % (as for the unsplit kernels)
        const double busy = 4 * tiles * S > 3 * cus ? 1.09 : 1.0;
        const double est = busy * (big ? pace_big : 0.56) * (per + 3) * (double)((tiles * S + cus - 1) / cus) + 4.0 + 3.0 +
                           2.0 * S * M * C * 4 / 5.0e6;
        if (est < best.est_us) {
            best.splits = (int)S; best.steps_per_split = per; best.big = big != 0; best.est_us = est;
        }
    }
    return best;
}

// Which kernel runs a product, and how its reduction is cut (the values of LQ_PLAN_* in latentq.h).
struct W4Plan {
    int kernel = LQ_PLAN_STAGED_128;
    int splits = 1, steps_per_split = 0;
};

// Forward pass, M > 16. Rough time per 64-deep step of the three kernels without a split
// (microseconds, measured): the weights-direct kernel (128 x 256 tiles) takes ~0.86 with one
// workgroup on a compute unit and ~1.45 for two sharing it; the staged kernel ~0.56 per round of
// 128 x 128 tiles and ~0.88 per round of 256 x 128 tiles (one workgroup per unit and round). The
// weights-direct kernel with 128 x 128 tiles fits three workgroups on a unit: ~0.55-0.61 alone (the
// more units are busy, the lower the clock: 0.55 up to three quarters of them, 0.61 with all), ~0.74
// as soon as a few units hold two, ~1.23 for two everywhere, ~1.38 for three; a full round of the
// staged 128 x 128 tiles likewise takes ~0.66 instead of ~0.56. The weights-direct kernels load scales and zeros four groups at a time: rows
// must be 4-byte aligned, i.e. the number of groups per row even.
static W4Plan plan_fwd(long long M, long long N, long long K, size_t ws_bytes, long long cus) {
    W4Plan out;
    const long long wg_direct = lq_gemm_fwd_direct_workgroups((int)M, (int)N);
    const long long rem = wg_direct % (2 * cus);
    const double est_direct = (K / LQ_GROUP) % 2 != 0 ? 1e30
                              : 1.45 * (double)(wg_direct / (2 * cus)) + (rem == 0 ? 0.0 : rem <= cus ? 0.86 : 1.45);
    const long long cols = (N + 127) / 128;
    const long long tiles_small = ((M + 127) / 128) * cols;
    const double est_small = tiles_small <= cus && 4 * tiles_small > 3 * cus ? 0.66 : 0.56 * (double)((tiles_small + cus - 1) / cus);
    const double est_big = 0.88 * (double)((((M + 255) / 256) * cols + cus - 1) / cus);
    double est_direct128 = 1e30;
    if ((K / LQ_GROUP) % 2 == 0) {
        const long long wg = lq_gemm_fwd_direct128_workgroups((int)M, (int)N);
        const long long rem128 = wg % (3 * cus);
        const double tail = rem128 == 0 ? 0.0
                            : 4 * rem128 <= 3 * cus ? 0.55
                            : rem128 <= cus ? 0.61
                            : rem128 <= 2 * cus ? 0.74 + 0.49 * (double)(rem128 - cus) / (double)cus
                                                : 1.38;
        est_direct128 = 1.38 * (double)(wg / (3 * cus)) + tail;
    }
    double step_us = est_direct;
    out.kernel = LQ_PLAN_DIRECT;
    if (est_direct128 < step_us) { step_us = est_direct128; out.kernel = LQ_PLAN_DIRECT_128; }
    if (est_small < step_us) { step_us = est_small; out.kernel = LQ_PLAN_STAGED_128; }
    if (est_big < step_us) { step_us = est_big; out.kernel = LQ_PLAN_STAGED_256; }
    double est_gemm = step_us * (double)(K / 64 + 3) + 4.0;
    const SplitPlan sp = plan_split(M, N, (int)(K / 64), ws_bytes, 0.88, cus);
    if (sp.splits >= 2 && sp.est_us < est_gemm) {
        out.kernel = sp.big ? LQ_PLAN_STAGED_256 : LQ_PLAN_STAGED_128;
        out.splits = sp.splits;
        out.steps_per_split = sp.steps_per_split;
        est_gemm = sp.est_us;
    }
    if (M <= 128) {
        // A few more tokens than one GEMV takes: the GEMM's 128-row tiles would be mostly padding and
        // its grid (N/128 workgroups, each walking all of K) fills a fraction of the device, so
        // chunks of 16 tokens through the GEMV can be faster: the first streams the weights from
        // HBM at near memory speed, the others find them in the last-level cache. Rough costs in
        // microseconds: a GEMV chunk takes its bytes at ~1.8 TB/s the first time (at least 6) and
        // ~2.3 TB/s after (at least 5; measured).
        const long long chunks = (M + 15) / 16;
        const double bytes = (double)(N * K / 2 + N * (K / LQ_GROUP) * 4);
        const double first_us = bytes / 1.8e6 > 6.0 ? bytes / 1.8e6 : 6.0;
        const double next_us = bytes / 2.3e6 > 5.0 ? bytes / 2.3e6 : 5.0;
        if (first_us + (chunks - 1) * next_us < est_gemm) {
            out.kernel = LQ_PLAN_GEMV_CHUNKS;
            out.splits = 1;
            out.steps_per_split = 0;
        }
    }
    return out;
}

// dX: rounds of one workgroup per compute unit at ~0.54 us per 64-deep step for 128 x 128 tiles,
// ~0.75 for 256 x 128 (a second small-tile workgroup on the same unit adds its full time), or a split reduction.
static W4Plan plan_dx(long long M, long long N, long long K, size_t ws_bytes, long long cus) {
    W4Plan out;
    const long long cols = (K + 127) / 128;
    const double est_small = 0.54 * (double)((((M + 127) / 128) * cols + cus - 1) / cus);
    const double est_big = 0.75 * (double)((((M + 255) / 256) * cols + cus - 1) / cus);
    out.kernel = est_small < est_big ? LQ_PLAN_STAGED_128 : LQ_PLAN_STAGED_256;
    const double est_gemm = (est_small < est_big ? est_small : est_big) * (double)(N / 64 + 3) + 4.0;
    const SplitPlan sp = plan_split(M, K, (int)(N / 64), ws_bytes, 0.75, cus);
    if (sp.splits >= 2 && sp.est_us < est_gemm) {
        out.kernel = sp.big ? LQ_PLAN_STAGED_256 : LQ_PLAN_STAGED_128;
        out.splits = sp.splits;
        out.steps_per_split = sp.steps_per_split;
    }
    return out;
}

static int launch_split_reduce(const GemmParams &p, int splits, hipStream_t st, const char *who) {
    const long long MC = (long long)p.M * p.C;
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)((MC / 8 + 255) / 256)), dim3(256), 0, st, p.partial, p.bias,
                       (unsigned short *)p.c, MC, p.C, splits);
    return lq_check_launch(who);
}

static int a16w4_fwd_impl(const char *who, const void *x, const void *codes, const void *scales, const void *zeros,
                          const void *bias_or_null, void *y, int64_t M, int64_t N, int64_t K, int group, void *workspace,
                          size_t ws_bytes, void *stream, unsigned long long *clk = nullptr) {
    int rc = check_w4_common(who, x, codes, scales, zeros, y, M, N, K, group);
    if (rc) return rc;
    LQ_REQUIRE(N % 16 == 0, "%s: N=%lld must be a multiple of 16", who, (long long)N);
    LQ_REQUIRE(!workspace || lq_aligned(workspace, 16), "%s: the workspace must be 16-byte aligned", who);
    if (M <= 16)
        return lq_gemv_a16w4_launch(x, codes, scales, zeros, bias_or_null, y, (int)M, (int)N, (int)K, (hipStream_t)stream);
    const W4Plan plan = plan_fwd(M, N, K, workspace ? ws_bytes : 0, lq_device_cu_count());
    if (plan.kernel == LQ_PLAN_GEMV_CHUNKS) {
        const int chunks = (int)((M + 15) / 16);
        for (int c = 0; c < chunks; ++c) {
            const int rows = (int)(M - 16 * c < 16 ? M - 16 * c : 16);
            rc = lq_gemv_a16w4_launch((const unsigned short *)x + (long long)c * 16 * K, codes, scales, zeros, bias_or_null,
                                      (unsigned short *)y + (long long)c * 16 * N, rows, (int)N, (int)K, (hipStream_t)stream);
            if (rc) return rc;
        }
        return LQ_OK;
    }
    if (plan.kernel == LQ_PLAN_DIRECT || plan.kernel == LQ_PLAN_DIRECT_128)
        return lq_gemm_fwd_direct_launch(x, codes, scales, zeros, bias_or_null, y, (int)M, (int)N, (int)K, (hipStream_t)stream, clk,
                                         plan.kernel == LQ_PLAN_DIRECT_128);
    GemmParams p = {};
    p.clk = clk;
    p.a = x; p.b = codes; p.scales = (const unsigned short *)scales; p.zeros = (const unsigned short *)zeros;
    p.bias = (const unsigned short *)bias_or_null; p.c = y;
    p.M = (int)M; p.C = (int)N; p.R = (int)K; p.Kw = (int)K;
    if (plan.splits >= 2) {
        p.partial = (float *)workspace;
        p.steps_per_split = plan.steps_per_split;
    }
    rc = plan.kernel == LQ_PLAN_STAGED_256 ? launch_gemm<MODE_W4_FWD, 256, 128, 2, 2>(p, (hipStream_t)stream, who)
                                           : launch_gemm<MODE_W4_FWD, 128, 128, 2, 2>(p, (hipStream_t)stream, who);
    if (rc || plan.splits < 2) return rc;
    return launch_split_reduce(p, plan.splits, (hipStream_t)stream, who);
}

static int gate_up_impl(const char *who, const void *x, const void *codes_gate, const void *scales_gate, const void *zeros_gate,
                        const void *codes_up, const void *scales_up, const void *zeros_up, void *h, void *g_out, void *u_out,
                        int64_t M, int64_t N, int64_t K, int group, void *stream) {
    int rc = check_w4_common(who, x, codes_gate, scales_gate, zeros_gate, h, M, N, K, group);
    if (rc) return rc;
    rc = check_w4_common(who, x, codes_up, scales_up, zeros_up, h, M, N, K, group);
    if (rc) return rc;
    LQ_REQUIRE(N % 16 == 0, "%s: N=%lld must be a multiple of 16", who, (long long)N);
    LQ_REQUIRE((g_out == nullptr) == (u_out == nullptr) && lq_aligned(g_out, 16) && lq_aligned(u_out, 16),
               "%s: g_out and u_out are given together, 16-byte aligned", who);
    if (M <= 16) {
        if (g_out) {
            // the two products on their own (one GEMV pass each), then the fused pass for h
            rc = lq_gemv_a16w4_launch(x, codes_gate, scales_gate, zeros_gate, nullptr, g_out, (int)M, (int)N, (int)K, (hipStream_t)stream);
            if (rc) return rc;
            rc = lq_gemv_a16w4_launch(x, codes_up, scales_up, zeros_up, nullptr, u_out, (int)M, (int)N, (int)K, (hipStream_t)stream);
            if (rc) return rc;
        }
        return lq_gemv_a16w4_gate_up_launch(x, codes_gate, scales_gate, zeros_gate, codes_up, scales_up, zeros_up, h, (int)M, (int)N,
                                            (int)K, (hipStream_t)stream);
    }
    LQ_REQUIRE(K % 256 == 0, "%s: K=%lld must be a multiple of 256 for more than 16 tokens", who, (long long)K);
    return lq_gemm_fwd_gate_up_launch(x, codes_gate, scales_gate, zeros_gate, codes_up, scales_up, zeros_up, h, g_out, u_out, (int)M,
                                      (int)N, (int)K, (hipStream_t)stream);
}

extern "C" int lq_a16w4_gate_up_silu(const void *x, const void *codes_gate, const void *scales_gate, const void *zeros_gate,
                                     const void *codes_up, const void *scales_up, const void *zeros_up, void *h, int64_t M,
                                     int64_t N, int64_t K, int group, void *stream) {
    return gate_up_impl("lq_a16w4_gate_up_silu", x, codes_gate, scales_gate, zeros_gate, codes_up, scales_up, zeros_up, h, nullptr,
                        nullptr, M, N, K, group, stream);
}

extern "C" int lq_a16w4_gate_up_silu_save(const void *x, const void *codes_gate, const void *scales_gate, const void *zeros_gate,
                                          const void *codes_up, const void *scales_up, const void *zeros_up, void *h, void *g_out,
                                          void *u_out, int64_t M, int64_t N, int64_t K, int group, void *stream) {
    LQ_REQUIRE(g_out && u_out, "lq_a16w4_gate_up_silu_save: null pointer argument");
    return gate_up_impl("lq_a16w4_gate_up_silu_save", x, codes_gate, scales_gate, zeros_gate, codes_up, scales_up, zeros_up, h, g_out,
                        u_out, M, N, K, group, stream);
}

extern "C" int lq_a16w4_fwd(const void *x, const void *codes, const void *scales, const void *zeros,
                            const void *bias_or_null, void *y, int64_t M, int64_t N, int64_t K, int group,
                            void *stream) {
    return a16w4_fwd_impl("lq_a16w4_fwd", x, codes, scales, zeros, bias_or_null, y, M, N, K, group, nullptr, 0, stream);
}

extern "C" int lq_a16w4_fwd_ws(const void *x, const void *codes, const void *scales, const void *zeros,
                               const void *bias_or_null, void *y, int64_t M, int64_t N, int64_t K, int group,
                               void *workspace, int64_t workspace_bytes, void *stream) {
    return a16w4_fwd_impl("lq_a16w4_fwd_ws", x, codes, scales, zeros, bias_or_null, y, M, N, K, group, workspace,
                          workspace && workspace_bytes > 0 ? (size_t)workspace_bytes : 0, stream);
}

struct DxEpilogue {
    int mode = EP_STORE;
    const void *g = nullptr, *u = nullptr;
    void *c2 = nullptr;
};

static int a16w4_dx_impl(const char *who, const void *dy, const void *codes, const void *scales, const void *zeros,
                         void *dx, int64_t M, int64_t N, int64_t K, int group, void *workspace, size_t ws_bytes,
                         void *stream, unsigned long long *clk = nullptr, const DxEpilogue &ep = DxEpilogue()) {
    int rc = check_w4_common(who, dy, codes, scales, zeros, dx, M, N, K, group);
    if (rc) return rc;
    LQ_REQUIRE(N % 64 == 0, "%s: N=%lld must be a multiple of 64", who, (long long)N);
    LQ_REQUIRE(!workspace || lq_aligned(workspace, 16), "%s: the workspace must be 16-byte aligned", who);
    GemmParams p = {};
    p.clk = clk;
    p.ep_mode = ep.mode;
    p.ep_g = (const unsigned short *)ep.g; p.ep_u = (const unsigned short *)ep.u; p.c2 = (unsigned short *)ep.c2;
    // the epilogue forms other than a plain store live in the GEMM kernel only: no split reduction with them
    if (ep.mode != EP_STORE) workspace = nullptr;
    p.a = dy; p.b = codes; p.scales = (const unsigned short *)scales; p.zeros = (const unsigned short *)zeros;
    p.c = dx;
    p.M = (int)M; p.C = (int)K; p.R = (int)N; p.Kw = (int)K;
    const W4Plan plan = plan_dx(M, N, K, workspace ? ws_bytes : 0, lq_device_cu_count());
    if (plan.splits >= 2) {
        p.partial = (float *)workspace;
        p.steps_per_split = plan.steps_per_split;
    }
    rc = plan.kernel == LQ_PLAN_STAGED_256 ? launch_gemm<MODE_W4_DX, 256, 128, 2, 2>(p, (hipStream_t)stream, who)
                                           : launch_gemm<MODE_W4_DX, 128, 128, 2, 2>(p, (hipStream_t)stream, who);
    if (rc || plan.splits < 2) return rc;
    return launch_split_reduce(p, plan.splits, (hipStream_t)stream, who);
}

// Scratch of the entry point that allocates nothing: one array per device, part of the code object,
// held by every device the library runs on until the process ends.
static __device__ __align__(256) unsigned char scratch[LQ_STATIC_SCRATCH_BYTES];

// Device address of `scratch` on the current device; looked up once per device (the array's name is
// only a host-side handle: each device has its own copy at its own address).
static int lq_static_scratch(void **out) {
    static std::atomic<void *> ptrs[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
        return lq_fail(LQ_ERR_LAUNCH, "lq_a16w4_fwd_static: cannot identify the current device");
    void *p = ptrs[dev].load(std::memory_order_acquire);
    if (!p) {
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p)
            return lq_fail(LQ_ERR_LAUNCH, "lq_a16w4_fwd_static: hipGetSymbolAddress failed on device %d: %s", dev,
                           hipGetErrorString(e));
        ptrs[dev].store(p, std::memory_order_release);
    }
    *out = p;
    return LQ_OK;
}

extern "C" int lq_a16w4_fwd_static(const void *x, const void *codes, const void *scales, const void *zeros,
                                   const void *bias_or_null, void *y, int64_t M, int64_t N, int64_t K, int group,
                                   void *stream) {
    LQ_REQUIRE(M > 0 && N > 0, "lq_a16w4_fwd_static: M and N must be positive (M=%lld N=%lld)", (long long)M, (long long)N);
    // two fp32 slices of the output are the least a split reduction takes
    LQ_REQUIRE(M <= 16 || (M < (1ll << 31) && N < (1ll << 31) && 8 * M * N <= (int64_t)LQ_STATIC_SCRATCH_BYTES),
               "lq_a16w4_fwd_static: an output of %lld x %lld needs %lld bytes for two fp32 slices, the static scratch holds %lld; "
               "use lq_a16w4_fwd or lq_a16w4_fwd_ws",
               (long long)M, (long long)N, (long long)(8 * M * N), (long long)LQ_STATIC_SCRATCH_BYTES);
    void *ws = nullptr;
    if (M > 16) {
        const int rc = lq_static_scratch(&ws);
        if (rc) return rc;
    }
    return a16w4_fwd_impl("lq_a16w4_fwd_static", x, codes, scales, zeros, bias_or_null, y, M, N, K, group, ws,
                          ws ? (size_t)LQ_STATIC_SCRATCH_BYTES : 0, stream);
}

// Measurement aid: lq_a16w4_fwd / lq_a16w4_dx with every workgroup recording its start and end on the
// shader-cycle counter and on the 100 MHz real-time counter (4 values per workgroup).
extern "C" int lq_calib_gemm_clocks(int backward, const void *a, const void *codes, const void *scales, const void *zeros,
                                    void *out, int64_t M, int64_t N, int64_t K, int group, uint64_t *clocks,
                                    int64_t clocks_capacity, int64_t *workgroups, void *stream) {
    LQ_REQUIRE(clocks && workgroups && lq_aligned(clocks, 8), "lq_calib_gemm_clocks: clocks and workgroups must be given");
    LQ_REQUIRE(M > 16, "lq_calib_gemm_clocks: needs M > 16 (the GEMM kernels)");
    LQ_REQUIRE(N > 0 && K > 0 && K % LQ_GROUP == 0 && M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31) &&
                   (backward ? N % 64 == 0 : N % 16 == 0),
               "lq_calib_gemm_clocks: bad shape");
    const long long cus = lq_device_cu_count();
    const W4Plan plan = backward ? plan_dx(M, N, K, 0, cus) : plan_fwd(M, N, K, 0, cus);
    LQ_REQUIRE(plan.kernel != LQ_PLAN_GEMV_CHUNKS, "lq_calib_gemm_clocks: this shape runs as GEMV chunks");
    const long long cols = backward ? K : N;
    const long long wg = plan.kernel == LQ_PLAN_DIRECT ? lq_gemm_fwd_direct_workgroups((int)M, (int)N)
                         : plan.kernel == LQ_PLAN_DIRECT_128 ? lq_gemm_fwd_direct128_workgroups((int)M, (int)N)
                         : plan.kernel == LQ_PLAN_STAGED_256 ? ((M + 255) / 256) * ((cols + 127) / 128)
                                                             : ((M + 127) / 128) * ((cols + 127) / 128);
    LQ_REQUIRE(4 * wg <= clocks_capacity, "lq_calib_gemm_clocks: clocks must hold %lld values, holds %lld", 4 * wg,
               (long long)clocks_capacity);
    *workgroups = wg;
    if (backward)
        return a16w4_dx_impl("lq_calib_gemm_clocks", a, codes, scales, zeros, out, M, N, K, group, nullptr, 0, stream,
                             (unsigned long long *)clocks);
    return a16w4_fwd_impl("lq_calib_gemm_clocks", a, codes, scales, zeros, nullptr, out, M, N, K, group, nullptr, 0, stream,
                          (unsigned long long *)clocks);
}

// The plan the two entry points above would follow, without launching anything.
extern "C" int lq_a16w4_plan(int backward, int64_t M, int64_t N, int64_t K, int64_t workspace_bytes, int compute_units,
                             int *kernel, int *splits, int *steps_per_split) {
    LQ_REQUIRE(kernel && splits && steps_per_split, "lq_a16w4_plan: null pointer argument");
    LQ_REQUIRE(M > 0 && N > 0 && K > 0 && K % LQ_GROUP == 0 && M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31),
               "lq_a16w4_plan: need positive M, N, K with K a multiple of %d", LQ_GROUP);
    LQ_REQUIRE(backward ? N % 64 == 0 : N % 16 == 0, "lq_a16w4_plan: N=%lld must be a multiple of %d", (long long)N,
               backward ? 64 : 16);
    const long long cus = compute_units > 0 ? compute_units : lq_device_cu_count();
    const size_t ws = workspace_bytes > 0 ? (size_t)workspace_bytes : 0;
    W4Plan plan;
    if (!backward && M <= 16) plan.kernel = LQ_PLAN_GEMV;
    else plan = backward ? plan_dx(M, N, K, ws, cus) : plan_fwd(M, N, K, ws, cus);
    *kernel = plan.kernel; *splits = plan.splits; *steps_per_split = plan.steps_per_split;
    return LQ_OK;
}

extern "C" int lq_a16w4_dx(const void *dy, const void *codes, const void *scales, const void *zeros, void *dx,
                           int64_t M, int64_t N, int64_t K, int group, void *stream) {
    return a16w4_dx_impl("lq_a16w4_dx", dy, codes, scales, zeros, dx, M, N, K, group, nullptr, 0, stream);
}

extern "C" int lq_a16w4_dx_acc(const void *dy, const void *codes, const void *scales, const void *zeros, void *dx_inout,
                               int64_t M, int64_t N, int64_t K, int group, void *stream) {
    DxEpilogue ep;
    ep.mode = EP_ADD;
    return a16w4_dx_impl("lq_a16w4_dx_acc", dy, codes, scales, zeros, dx_inout, M, N, K, group, nullptr, 0, stream, nullptr, ep);
}

// dx = dy1 * deq(W1) + dy2 * deq(W2) for two layers of the same shape that share their input (gate and up of an MLP
// block): one launch whose reduction runs through the first product and on into the second, the sum kept in the fp32
// accumulators (one rounding to bf16 where lq_a16w4_dx followed by lq_a16w4_dx_acc has two).
extern "C" int lq_a16w4_dx_pair(const void *dy1, const void *codes1, const void *scales1, const void *zeros1, const void *dy2,
                                const void *codes2, const void *scales2, const void *zeros2, void *dx, int64_t M, int64_t N,
                                int64_t K, int group, void *stream) {
    const char *who = "lq_a16w4_dx_pair";
    int rc = check_w4_common(who, dy1, codes1, scales1, zeros1, dx, M, N, K, group);
    if (rc) return rc;
    rc = check_w4_common(who, dy2, codes2, scales2, zeros2, dx, M, N, K, group);
    if (rc) return rc;
    LQ_REQUIRE(N % 64 == 0, "%s: N=%lld must be a multiple of 64", who, (long long)N);
    GemmParams p = {};
    p.a = dy1; p.b = codes1; p.scales = (const unsigned short *)scales1; p.zeros = (const unsigned short *)zeros1;
    p.a2 = dy2; p.b2 = codes2; p.scales2 = (const unsigned short *)scales2; p.zeros2 = (const unsigned short *)zeros2;
    p.c = dx;
    p.M = (int)M; p.C = (int)K; p.R = (int)N; p.Kw = (int)K;
    const W4Plan plan = plan_dx(M, N, K, 0, lq_device_cu_count());
    return plan.kernel == LQ_PLAN_STAGED_256 ? launch_gemm<MODE_W4_DX, 256, 128, 2, 2>(p, (hipStream_t)stream, who)
                                             : launch_gemm<MODE_W4_DX, 128, 128, 2, 2>(p, (hipStream_t)stream, who);
}

extern "C" int lq_a16w4_dx_silu_bwd(const void *dh_dy, const void *codes, const void *scales, const void *zeros, const void *g,
                                    const void *u, void *dg_out, void *du_out, int64_t M, int64_t N, int64_t K, int group,
                                    void *stream) {
    LQ_REQUIRE(g && u && du_out && lq_aligned(g, 16) && lq_aligned(u, 16) && lq_aligned(du_out, 16),
               "lq_a16w4_dx_silu_bwd: g, u and du_out must be given, 16-byte aligned");
    DxEpilogue ep;
    ep.mode = EP_SILU_BW;
    ep.g = g; ep.u = u; ep.c2 = du_out;
    return a16w4_dx_impl("lq_a16w4_dx_silu_bwd", dh_dy, codes, scales, zeros, dg_out, M, N, K, group, nullptr, 0, stream, nullptr, ep);
}

extern "C" int lq_a16w4_dx_ws(const void *dy, const void *codes, const void *scales, const void *zeros, void *dx,
                              int64_t M, int64_t N, int64_t K, int group, void *workspace, int64_t workspace_bytes,
                              void *stream) {
    return a16w4_dx_impl("lq_a16w4_dx_ws", dy, codes, scales, zeros, dx, M, N, K, group, workspace,
                         workspace && workspace_bytes > 0 ? (size_t)workspace_bytes : 0, stream);
}

// dX of an 8-bit-weight layer straight from the int8 codes: the staged dX kernel with the weight waves forming
// bf16(w8 * qs[n]) instead of dequantising int4 groups.
extern "C" int lq_a8w8_dx(const void *dy, const void *w, const void *qscales_bf16, void *dx, int64_t M, int64_t N, int64_t K,
                          void *stream) {
    LQ_REQUIRE(dy && w && qscales_bf16 && dx, "lq_a8w8_dx: null pointer argument");
    LQ_REQUIRE(M > 0 && N > 0 && K > 0 && M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31) && N * K < (1ll << 40),
               "lq_a8w8_dx: M, N, K must be positive (M=%lld N=%lld K=%lld)", (long long)M, (long long)N, (long long)K);
    LQ_REQUIRE(N % 64 == 0 && K % 128 == 0, "lq_a8w8_dx: N=%lld must be a multiple of 64 and K=%lld of 128", (long long)N, (long long)K);
    LQ_REQUIRE(lq_aligned(dy, 16) && lq_aligned(w, 16) && lq_aligned(dx, 16) && lq_aligned(qscales_bf16, 2),
               "lq_a8w8_dx: dy, w and dx must be 16-byte aligned");
    GemmParams p = {};
    p.a = dy; p.b = w; p.scales = (const unsigned short *)qscales_bf16; p.c = dx;
    p.M = (int)M; p.C = (int)K; p.R = (int)N; p.Kw = (int)K;
    const W4Plan plan = plan_dx(M, N, K, 0, lq_device_cu_count());
    return plan.kernel == LQ_PLAN_STAGED_256 ? launch_gemm<MODE_W8_DX, 256, 128, 2, 2>(p, (hipStream_t)stream, "lq_a8w8_dx")
                                             : launch_gemm<MODE_W8_DX, 128, 128, 2, 2>(p, (hipStream_t)stream, "lq_a8w8_dx");
}

static int a8w8_fwd_impl(const void *x, const void *w, const float *sx, const void *sw, bool sw_bf16, const void *bias_or_null,
                         void *y, int32_t *acc_or_null, int64_t M, int64_t N, int64_t K, void *stream) {
    LQ_REQUIRE(x && w && sx && sw && y, "lq_a8w8_fwd: null pointer argument");
    LQ_REQUIRE(M > 0 && N > 0 && K > 0, "lq_a8w8_fwd: M, N, K must be positive");
    LQ_REQUIRE(K % 128 == 0, "lq_a8w8_fwd: K=%lld must be a multiple of 128", (long long)K);
    LQ_REQUIRE(N % 16 == 0, "lq_a8w8_fwd: N=%lld must be a multiple of 16", (long long)N);
    LQ_REQUIRE(M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31), "lq_a8w8_fwd: dimension too large");
    LQ_REQUIRE(lq_aligned(x, 16) && lq_aligned(w, 16) && lq_aligned(y, 16) && lq_aligned(sx, 4) && lq_aligned(sw, sw_bf16 ? 2 : 4) &&
                   (!acc_or_null || lq_aligned(acc_or_null, 16)),
               "lq_a8w8_fwd: x, w, y, acc must be 16-byte aligned");
    // 256 x 256 tiles, both operands through LDS, when they occupy more than half of the compute
    // units; below that the staged kernel's smaller tiles fill the device better
    if (lq_gemm_i8_256_workgroups((int)M, (int)N) * 2 > (long long)lq_device_cu_count())
        return lq_gemm_i8_tile_launch(x, w, sx, sw, sw_bf16, bias_or_null, y, acc_or_null, (int)M, (int)N, (int)K, 256, 2, (hipStream_t)stream);
    // the same kernel with 128 x 128 tiles (two workgroups per CU) when there are more of them than
    // compute units; measured 40.6 -> 37.0 us on 2048 x 4096 x 4096
    const long long tiles128 = ((M + 127) / 128) * ((N + 127) / 128);
    const long long cus = lq_device_cu_count();
    if (tiles128 > cus)
        return lq_gemm_i8_tile_launch(x, w, sx, sw, sw_bf16, bias_or_null, y, acc_or_null, (int)M, (int)N, (int)K, 128, 2, (hipStream_t)stream);
    // A workgroup with a CU to itself: four 32 KB stages (loads three steps ahead). Nothing covers such a workgroup's
    // waits but its own prefetch distance, and the weights come from HBM in any real use: timed over 0.4 GB of rotating
    // weight matrices, 14.0 against 18.2 us for two stages on 2048^3, 10.0 against 11.9 at K = 1024, 23.4-24.2
    // against 26.4-26.9 for the staged kernel on 2048 x 2048 x 4096 and 1024 x 4096 x 4096, 30.3 against 33.3 at
    // K = 5120 (with the one weight matrix of a timing loop sitting in the last-level cache the three are within 10 %
    // of each other, in no fixed order).
    return lq_gemm_i8_tile_launch(x, w, sx, sw, sw_bf16, bias_or_null, y, acc_or_null, (int)M, (int)N, (int)K, 128, 4, (hipStream_t)stream);
}

extern "C" int lq_a8w8_fwd(const void *x, const void *w, const float *sx, const float *sw, const void *bias_or_null,
                           void *y, int32_t *acc_or_null, int64_t M, int64_t N, int64_t K, void *stream) {
    return a8w8_fwd_impl(x, w, sx, sw, false, bias_or_null, y, acc_or_null, M, N, K, stream);
}

extern "C" int lq_a8w8_fwd_qs(const void *x, const void *w, const float *sx, const void *qscales_bf16, const void *bias_or_null,
                              void *y, int32_t *acc_or_null, int64_t M, int64_t N, int64_t K, void *stream) {
    return a8w8_fwd_impl(x, w, sx, qscales_bf16, true, bias_or_null, y, acc_or_null, M, N, K, stream);
}
