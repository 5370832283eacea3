// Weight-gradient GEMM for gfx950:  dW[N,K] = dY[M,N]^T . X[M,K]   (bf16 operands, fp32 accumulation)
//
// The reduction runs over the tokens m, the slow dimension of both operands, so neither operand has the
// layout an MFMA lane wants (8 consecutive reduction elements of one row). Both tiles are staged exactly as they
// lie in memory - 64 token rows of 256 contiguous columns, written by LDS-direct loads (no registers, no
// vector-ALU work) - and the fragments are fetched with the transposing LDS read ds_read_b64_tr_b16: within a
// 16-lane block, lane i receives the four elements of column i of the 4 x 16 block the 16 lanes address. No
// transposed copy of dY is made anywhere.
//
// Workgroup: 256 (n) x 256 (k) outputs, 512 threads = 8 waves in a 2 (n) x 4 (k) grid; a wave owns 128 x 64
// outputs (4 x 2 MFMA 32x32x16 tiles, 128 accumulator registers). Two LDS stages of 64 KB (64 rows of dY and 64
// rows of X, 512 bytes each); one workgroup per CU.
//
// Reduction step = 64 tokens in four slices of 16. Lane l: r = l % 32, h = l / 32; in slice t the lane's operand
// for column r of a 32-column fragment is tokens 16 t + 8 h .. + 7: two transposing reads (tokens .. + 3 and
// + 4 .. + 7). In each read block lane i (of 16) addresses row i / 4 of the block's 4 token rows at columns
// 4 (i % 4) .. + 3 of its 16 columns. A row's 512 bytes are sixteen 32-byte segments; segment s of token row m
// sits at position s ^ 2 (m & 3), which spreads the 4 rows x 2 column blocks that 32 lanes read over all 64 banks;
// the swizzle is free, since an LDS-direct load lets a lane choose the global 16 bytes that land in its slot.
//
// Pipeline as in the int8 tile kernel: one s_barrier per step before its last slice, the loads of the step after
// next go into the stage that barrier releases, loads as inline assembly with explicit waits.
//
// D = Xfrag x dYfrag^T: a lane owns 4 consecutive k of one n. Epilogues (through LDS, 16-byte pieces of rows):
//   store  dW rounded to bf16;
//   acc8   the int8 gradient accumulator's add_ form on the bf16-rounded dW: q = quant(dequant(q) + dW) in place
//          with the stored row scale (16 consecutive k per lane = one Philox block), so that neither dW nor the
//          dequantised accumulator ever exists in memory.
#include "lq_common.h"
#include "lq_gradq8_math.h"

#include <type_traits>

namespace {

struct DwParams {
    const unsigned char *dy;  // bf16 [M, N]
    const unsigned char *x;   // bf16 [M, K]
    unsigned short *dw;       // store: bf16 [N, K]
    int accumulate;           // store: dw = bf16(dw + bf16(product)) instead of dw = bf16(product)
    signed char *q;           // acc8: int8 [N, K], updated in place
    const unsigned short *scale;  // acc8: bf16 [N]
    const unsigned short *noise;  // acc8: bf16 [N, K] or null (Philox)
    unsigned long long seed, offset;
    int M, N, K;
    int tiles_n, tiles_k;
};

typedef __attribute__((address_space(3))) void lds_void;
typedef short v4s_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) v4s_t lds_v4s_t;

template <int I>
using ic = std::integral_constant<int, I>;

constexpr int TILE = 256;            // outputs per workgroup along n and along k
constexpr int ROWB = TILE * 2;       // bytes per staged token row of one operand
constexpr int STEP_M = 64;           // tokens per reduction step
constexpr int OP_STAGE = STEP_M * ROWB;  // 32 KB per operand and stage
constexpr int STAGE = 2 * OP_STAGE;
constexpr int NT = 512;
constexpr int LOADS = OP_STAGE / 16 / NT;  // 16-byte loads per thread, operand and stage: 4

template <bool ACC8>
__global__ __launch_bounds__(NT) void gemm_dw_kernel(DwParams p) {
    constexpr int WM = 2, WN = 4;           // waves along n, along k
    constexpr int TM = TILE / WM, TN = TILE / WN;  // wave tile: 128 n x 64 k
    constexpr int FM = TM / 32, FN = TN / 32;
    // two stages; the accumulate epilogue stages every wave's whole 128 x 64 block (144-byte rows) instead
    constexpr int LDS_BYTES = ACC8 && 8 * TM * (TN * 2 + 16) > 2 * STAGE ? 8 * TM * (TN * 2 + 16) : 2 * STAGE;
    __shared__ __attribute__((aligned(16))) unsigned char lds_all[LDS_BYTES];
    auto stage = [&](auto i) -> unsigned char * { return lds_all + decltype(i)::value * STAGE; };

    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int lane = threadIdx.x & 63;
    const int r = lane & 31, h = lane >> 5;
    const int wm = wave % WM, wn = wave / WM;

    // Workgroup ids are dealt round-robin over the 8 XCDs (id % 8): give each XCD a contiguous range of the tile
    // sequence, ordered in bands of GN tile columns walked row by row, so the workgroups resident on one XCD share
    // a few dY column blocks and X column blocks in its L2.
    const int nwg = p.tiles_n * p.tiles_k;
    int id = blockIdx.x;
    {
        const int per = nwg / 8;
        if (id < per * 8) id = (id % 8) * per + id / 8;
    }
    constexpr int GN = 8;
    const int band = id / (p.tiles_n * GN);
    const int within = id - band * (p.tiles_n * GN);
    const int rest = p.tiles_k - band * GN;
    const int bw = rest < GN ? rest : GN;
    const int tile_n = within / bw, tile_k = band * GN + within % bw;
    const int n0 = tile_n * TILE, k0 = tile_k * TILE;
    const int nk = p.M / STEP_M;

    // ---- staging: slot s = i * 512 + thread of an operand's stage is token row s / 32, 16-byte position s % 32;
    // it receives the 16 bytes of segment (pos / 2) ^ 2 (row & 3), half pos & 1. Columns past the end of a matrix
    // re-read its last 8 columns (their results are dropped).
    unsigned a_off[LOADS], b_off[LOADS];
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
        const int s = i * NT + (int)threadIdx.x;
        const int row = s >> 5, pos = s & 31;
        const int c16 = ((((pos >> 1) ^ (2 * (row & 3))) << 1) | (pos & 1));
        int ca = n0 / 8 + c16, cb = k0 / 8 + c16;
        ca = ca < p.N / 8 ? ca : p.N / 8 - 1;
        cb = cb < p.K / 8 ? cb : p.K / 8 - 1;
        a_off[i] = (unsigned)((long long)row * p.N * 2 + (long long)ca * 16);
        b_off[i] = (unsigned)((long long)row * p.K * 2 + (long long)cb * 16);
    }
    // load i of a step: 0 .. LOADS-1 fill the dY rows of the stage, LOADS .. 2 LOADS-1 its X rows
    auto issue_one = [&](int kt, unsigned char *st, int i) {
        const bool is_b = i >= LOADS;
        const int ii = is_b ? i - LOADS : i;
        const unsigned char *src = is_b ? p.x + (long long)kt * STEP_M * p.K * 2 : p.dy + (long long)kt * STEP_M * p.N * 2;
        const unsigned lds_addr = (unsigned)reinterpret_cast<size_t>(
            (lds_void *)(st + (is_b ? OP_STAGE : 0) + (ii * NT + wave * 64) * 16));
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                     :: "s"(lds_addr), "v"(is_b ? b_off[ii < LOADS ? ii : 0] : a_off[ii < LOADS ? ii : 0]), "s"(src) : "memory");
    };

    // ---- fragments. Read block = lane / 16: column block (lane / 16) & 1 of the fragment's 32 columns, token half
    // h; block lane i16 addresses token row (i16 / 4) of the block's 4 and columns 4 (i16 % 4) .. + 3.
    const int i16 = lane & 15, cblk = (lane >> 4) & 1;
    // byte offset of the lane's 8 bytes within a staged row of fragment f (32 columns from column 32 f of the wave's part)
    auto col_off = [&](int col0) {
        const int seg = (col0 >> 4) + cblk;  // 32-byte segment of the row
        return ((seg ^ (2 * (i16 >> 2))) << 5) + ((i16 & 3) << 3);
    };
    int a_col[FM], b_col[FN];
#pragma unroll
    for (int j = 0; j < FM; ++j) a_col[j] = col_off(wm * TM + 32 * j);
#pragma unroll
    for (int i = 0; i < FN; ++i) b_col[i] = OP_STAGE + col_off(wn * TN + 32 * i);
    const int row_lane = (8 * h + (i16 >> 2)) * ROWB;  // + 16 t rows for slice t, + 4 rows for the second read
    auto read_frags = [&](const unsigned char *st, int t, u32x4_t *af, u32x4_t *bf) {
        const unsigned char *base = st + row_lane + t * 16 * ROWB;
#pragma unroll
        for (int j = 0; j < FM; ++j) {
            const v4s_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_t *)(base + a_col[j]));
            const v4s_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_t *)(base + a_col[j] + 4 * ROWB));
            const u32x2_t l2 = __builtin_bit_cast(u32x2_t, lo), h2 = __builtin_bit_cast(u32x2_t, hi);
            af[j] = u32x4_t{l2[0], l2[1], h2[0], h2[1]};
        }
#pragma unroll
        for (int i = 0; i < FN; ++i) {
            const v4s_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_t *)(base + b_col[i]));
            const v4s_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_t *)(base + b_col[i] + 4 * ROWB));
            const u32x2_t l2 = __builtin_bit_cast(u32x2_t, lo), h2 = __builtin_bit_cast(u32x2_t, hi);
            bf[i] = u32x4_t{l2[0], l2[1], h2[0], h2[1]};
        }
    };

    f32x16_t acc[FN][FM];
#pragma unroll
    for (int i = 0; i < FN; ++i)
#pragma unroll
        for (int j = 0; j < FM; ++j)
#pragma unroll
            for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.f;

    u32x4_t af[2][FM], bf[2][FN];
    // Step kt on stage S = kt % 2: the operands of its first slice are already in af[0] / bf[0]. The barrier of a
    // step releases its stage, into which the last slice issues the dY half of step kt + 2 and the next step's
    // first slice the X half.
    auto step = [&](int kt, auto si) {
        constexpr int S = decltype(si)::value;
        unsigned char *cur = stage(ic<S>()), *nxt = stage(ic<S ^ 1>());
        const int kt_b = kt + 1 < nk ? kt + 1 : nk - 1, kt_a = kt + 2 < nk ? kt + 2 : nk - 1;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            if (t == 3) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
            if (t < 3) read_frags(cur, t + 1, af[(t + 1) & 1], bf[(t + 1) & 1]);
            else read_frags(nxt, 0, af[0], bf[0]);
            if (t == 0) {
                // X half of the loads of step kt + 1 (its stage was released by the previous barrier)
#pragma unroll
                for (int i = LOADS; i < 2 * LOADS; ++i) issue_one(kt_b, nxt, i);
            }
            if (t == 3) {
                // dY half of the loads of step kt + 2, into the stage just released
#pragma unroll
                for (int i = 0; i < LOADS; ++i) issue_one(kt_a, cur, i);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < FN; ++i)
#pragma unroll
                for (int j = 0; j < FM; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, bf[t & 1][i]),
                                                                       __builtin_bit_cast(bf16x8_t, af[t & 1][j]), acc[i][j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // prologue: step 0 entirely, the dY half of step 1; wait for step 0
#pragma unroll
    for (int i = 0; i < 2 * LOADS; ++i) issue_one(0, stage(ic<0>()), i);
#pragma unroll
    for (int i = 0; i < LOADS; ++i) issue_one(nk > 1 ? 1 : 0, stage(ic<1>()), i);
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(LOADS) : "memory");
    read_frags(lds_all, 0, af[0], bf[0]);
    __builtin_amdgcn_sched_barrier(0);
    int kt = 0;
    for (; kt + 2 <= nk; kt += 2) {
        step(kt, ic<0>());
        step(kt + 1, ic<1>());
    }
    if (kt < nk) step(kt, ic<0>());
    // the clamped prefetches of the last steps are still writing LDS: drain them
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    // ---- epilogue: acc[i][j][q]: column k0 + TN wn + 32 i + 8 (q / 4) + 4 h + q % 4, row n0 + TM wm + 32 j + r.
    // Every wave passes its block through a private LDS area.
    __syncthreads();
    constexpr int EP = TN * 2 + 16;  // row pitch of the staging area
    const int kw0 = k0 + wn * TN;
    if constexpr (!ACC8) {
        // 32 rows (one j) at a time; 16 bytes per lane, 8 lanes on the 128 contiguous bytes of a row
        unsigned char *ep = lds_all + wave * (32 * EP);
        const int ep_row = lane >> 3, ep_chunk = lane & 7;
        const int kc = kw0 + ep_chunk * 8;
#pragma unroll
        for (int j = 0; j < FM; ++j) {
            const int nrow0 = n0 + wm * TM + j * 32;
#pragma unroll
            for (int i = 0; i < FN; ++i)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const u32x2_t o = {lq_pack_bf16(acc[i][j][4 * q], acc[i][j][4 * q + 1]), lq_pack_bf16(acc[i][j][4 * q + 2], acc[i][j][4 * q + 3])};
                    *reinterpret_cast<u32x2_t *>(ep + r * EP + (i * 32 + 8 * q + 4 * h) * 2) = o;
                }
#pragma unroll
            for (int it = 0; it < 4; ++it) {
                const int row = it * 8 + ep_row;
                const u32x4_t o = *reinterpret_cast<const u32x4_t *>(ep + row * EP + ep_chunk * 16);
                const int nn = nrow0 + row;
                if (nn < p.N && kc < p.K) {
                    unsigned short *dst = p.dw + (long long)nn * p.K + kc;
                    if (p.accumulate) {
                        // the bf16 addition a tensor `add_` of the stored product would make
                        const u32x4_t old = *reinterpret_cast<const u32x4_t *>(dst);
                        u32x4_t sum;
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            sum[e] = lq_pack_bf16(lq_bf16_lo(old[e]) + lq_bf16_lo(o[e]), lq_bf16_hi(old[e]) + lq_bf16_hi(o[e]));
                        *reinterpret_cast<u32x4_t *>(dst) = sum;
                    } else {
                        *reinterpret_cast<u32x4_t *>(dst) = o;
                    }
                }
            }
        }
    } else {
        // The whole 128 x 64 block of the wave goes to LDS as bf16 first (straight-line code), then a rolled loop of
        // 8 passes of 16 rows does the accumulator arithmetic: unrolled over the accumulator registers that
        // arithmetic would be some 50 KB of code, more than the instruction cache holds. 16 consecutive k per lane
        // (one Philox block), 4 lanes per row.
        unsigned char *ep = lds_all + wave * (TM * EP);
#pragma unroll
        for (int j = 0; j < FM; ++j)
#pragma unroll
            for (int i = 0; i < FN; ++i)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const u32x2_t o = {lq_pack_bf16(acc[i][j][4 * q], acc[i][j][4 * q + 1]), lq_pack_bf16(acc[i][j][4 * q + 2], acc[i][j][4 * q + 3])};
                    *reinterpret_cast<u32x2_t *>(ep + (j * 32 + r) * EP + (i * 32 + 8 * q + 4 * h) * 2) = o;
                }
        const int q_row = lane >> 2, q_piece = lane & 3;
        const int kq = kw0 + q_piece * 16;
        const int nw0 = n0 + wm * TM;
        auto fetch = [&](int pass, u32x4_t &oldq, float &sc) {
            const int nn = nw0 + pass * 16 + q_row;
            const bool live = nn < p.N && kq < p.K;
            oldq = *reinterpret_cast<const u32x4_t *>(p.q + (live ? (long long)nn * p.K + kq : 0));
            sc = lq_bf16_bits_to_f32(p.scale[live ? nn : 0]);
        };
        u32x4_t old_next;
        float s_next;
        fetch(0, old_next, s_next);
#pragma unroll 1
        for (int pass = 0; pass < TM / 16; ++pass) {
            const u32x4_t oldq = old_next;
            const float sc = s_next;
            if (pass + 1 < TM / 16) fetch(pass + 1, old_next, s_next);
            const int row = pass * 16 + q_row;
            const int nn = nw0 + row;
            const bool live = nn < p.N && kq < p.K;
            const u32x4_t v0 = *reinterpret_cast<const u32x4_t *>(ep + row * EP + q_piece * 32);
            const u32x4_t v1 = *reinterpret_cast<const u32x4_t *>(ep + row * EP + q_piece * 32 + 16);
            const long long e0 = live ? (long long)nn * p.K + kq : 0;
            u32x4_t z0 = {0u, 0u, 0u, 0u}, z1 = z0;
            if (p.noise) {
                z0 = *reinterpret_cast<const u32x4_t *>(p.noise + e0);
                z1 = *reinterpret_cast<const u32x4_t *>(p.noise + e0 + 8);
            }
            const unsigned long long c = p.offset + (unsigned long long)(e0 >> 4);
            // the reciprocal form is exact for scales between 2^-40 and 2^40; one lane outside sends the wave
            // through the division
            const bool fast = sc >= 0x1p-40f && sc <= 0x1p40f;
            const bool all_fast = __builtin_amdgcn_ballot_w64(!fast) == 0ull;
            u32x4_t o;
            if (p.noise) o = all_fast ? quant16<false, true, true>(v0, v1, oldq, z0, z1, sc, 1.0f / sc, c, p.seed)
                                      : quant16<false, true, false>(v0, v1, oldq, z0, z1, sc, 0.f, c, p.seed);
            else o = all_fast ? quant16<true, true, true>(v0, v1, oldq, z0, z1, sc, 1.0f / sc, c, p.seed)
                              : quant16<true, true, false>(v0, v1, oldq, z0, z1, sc, 0.f, c, p.seed);
            if (live) *reinterpret_cast<u32x4_t *>(p.q + e0) = o;
        }
    }
}

static int launch_dw(DwParams p, bool acc8, hipStream_t st, const char *who) {
    p.tiles_n = (p.N + TILE - 1) / TILE;
    p.tiles_k = (p.K + TILE - 1) / TILE;
    const long long nwg = (long long)p.tiles_n * p.tiles_k;
    if (nwg > 0x7FFFFFFFll) return lq_fail(LQ_ERR_BAD_ARG, "%s: problem too large", who);
    // the 32-bit lane offsets of the loads span 64 token rows
    if (64ll * 2 * (p.N > p.K ? p.N : p.K) >= (1ll << 32)) return lq_fail(LQ_ERR_BAD_ARG, "%s: rows too long", who);
    if (acc8) hipLaunchKernelGGL(gemm_dw_kernel<true>, dim3((unsigned)nwg), dim3(NT), 0, st, p);
    else hipLaunchKernelGGL(gemm_dw_kernel<false>, dim3((unsigned)nwg), dim3(NT), 0, st, p);
    return lq_check_launch(who);
}

static int check_dw(const char *who, const void *dy, const void *x, int64_t M, int64_t N, int64_t K, int k_mult) {
    LQ_REQUIRE(dy && x, "%s: null pointer argument", who);
    LQ_REQUIRE(M > 0 && N > 0 && K > 0 && M < (1ll << 31) && N < (1ll << 31) && K < (1ll << 31), "%s: M, N, K must be positive", who);
    LQ_REQUIRE(M % 64 == 0, "%s: M=%lld (tokens) must be a multiple of 64", who, (long long)M);
    LQ_REQUIRE(N % 8 == 0 && K % k_mult == 0, "%s: N=%lld must be a multiple of 8 and K=%lld of %d", who, (long long)N, (long long)K, k_mult);
    LQ_REQUIRE(lq_aligned(dy, 16) && lq_aligned(x, 16), "%s: dy and x must be 16-byte aligned", who);
    return LQ_OK;
}

}  // namespace

extern "C" int lq_weight_grad(const void *dy, const void *x, void *dw_out, int64_t M, int64_t N, int64_t K, void *stream) {
    int rc = check_dw("lq_weight_grad", dy, x, M, N, K, 8);
    if (rc) return rc;
    LQ_REQUIRE(dw_out && lq_aligned(dw_out, 16), "lq_weight_grad: dw_out must be given, 16-byte aligned");
    DwParams p = {};
    p.dy = (const unsigned char *)dy; p.x = (const unsigned char *)x; p.dw = (unsigned short *)dw_out;
    p.M = (int)M; p.N = (int)N; p.K = (int)K;
    return launch_dw(p, false, (hipStream_t)stream, "lq_weight_grad");
}

extern "C" int lq_weight_grad_acc(const void *dy, const void *x, void *dw_inout, int64_t M, int64_t N, int64_t K, void *stream) {
    int rc = check_dw("lq_weight_grad_acc", dy, x, M, N, K, 8);
    if (rc) return rc;
    LQ_REQUIRE(dw_inout && lq_aligned(dw_inout, 16), "lq_weight_grad_acc: dw_inout must be given, 16-byte aligned");
    DwParams p = {};
    p.dy = (const unsigned char *)dy; p.x = (const unsigned char *)x; p.dw = (unsigned short *)dw_inout;
    p.accumulate = 1;
    p.M = (int)M; p.N = (int)N; p.K = (int)K;
    return launch_dw(p, false, (hipStream_t)stream, "lq_weight_grad_acc");
}

extern "C" int lq_weight_grad_acc8(const void *dy, const void *x, int8_t *q_inout, const void *scale, int64_t M, int64_t N,
                                   int64_t K, const void *noise_or_null, uint64_t philox_seed, uint64_t philox_offset,
                                   void *stream) {
    int rc = check_dw("lq_weight_grad_acc8", dy, x, M, N, K, 16);
    if (rc) return rc;
    LQ_REQUIRE(q_inout && scale && lq_aligned(q_inout, 16) && lq_aligned(scale, 2) && (!noise_or_null || lq_aligned(noise_or_null, 16)),
               "lq_weight_grad_acc8: q and scale must be given; q and noise 16-byte aligned");
    DwParams p = {};
    p.dy = (const unsigned char *)dy; p.x = (const unsigned char *)x; p.q = (signed char *)q_inout;
    p.scale = (const unsigned short *)scale; p.noise = (const unsigned short *)noise_or_null;
    p.seed = philox_seed; p.offset = philox_offset;
    p.M = (int)M; p.N = (int)N; p.K = (int)K;
    return launch_dw(p, true, (hipStream_t)stream, "lq_weight_grad_acc8");
}
