// A8W8 GEMM for gfx950, both operands through LDS-direct loads:
//   Y[M,N] = bf16(((int32) X8[M,K] . W8[N,K]^T) * sx[m] * sw[n] (+ bias)), optional int32 accumulators.
//
// int8 operands need no dequantisation, so both operands go from global memory into LDS with
// LDS-direct loads (no registers, no vector-ALU work) and what bounds a tile scheme is the traffic
// between L2 and the compute units: per unit of MFMA work a 128 x 256 tile moves 1.5 times the
// bytes of a 256 x 256 tile, and at int8 rates (twice the reduction depth per MFMA cycle of bf16)
// that traffic, not the matrix core, set the pace of a 128 x 256 kernel.
//
// Main instance: 256 x 256 tile, 512 threads = 8 waves in a 2 (m) x 4 (n) grid; a wave owns
// 128 x 64 outputs (4 x 2 MFMA 32x32x32 tiles, 128 accumulator registers), two waves per SIMD. One
// workgroup per CU: two LDS stages of 64 KB (256 rows of A and 256 rows of B, 128 bytes = 128 k
// each). For small outputs: 128 x 128 tile, 8 waves (2 x 4, 64 x 32 each), with two stages of
// 32 KB (two workgroups per CU) or four (one workgroup per CU, loads three steps ahead).
//
// Reduction step = 128 k in four slices of 32. Lane l: r = l % 32, h = l / 32. In slice t the
// lane's operand of row r is chunk 4h + t (16 bytes) of the row's 128 bytes, for A and B alike
// (any assignment of k to slices and halves is valid as long as both operands use the same one).
// Chunk c of tile row x sits at position c ^ ((x >> 1) & 7): fragment reads are conflict-free and
// the swizzle is free, since an LDS-direct load lets a lane choose the global chunk that lands in
// its fixed LDS slot.
//
// Pipeline: one s_barrier per step, before the last slice. Past it every wave's fragment reads of
// the current stage have returned, so the last slice and the next step's first slice issue the
// loads of the step after next into it (4 per thread each), while the last slice already reads
// the next stage's first fragments; the wait in front of the barrier covers those loads one step
// later. Loads are inline assembly with explicit waits, as in the other GEMM kernels.
//
// D = Wfrag x Xfrag^T: a lane owns 4 consecutive n of one m; the epilogue applies the scales and
// regroups the bf16 results through LDS into 16-byte pieces of full output rows.
#include "lq_common.h"

#include <type_traits>

namespace {

struct I8Params {
    const unsigned char *x;  // int8 [M, K]
    const unsigned char *w;  // int8 [N, K]
    const float *sx;         // [M]
    const float *sw;         // [N]: fp32, or bf16 when sw_bf16 is set
    int sw_bf16;
    const unsigned short *bias;  // bf16 [N] or null
    int *acc_out;                // optional int32 [M, N]
    unsigned short *y;           // bf16 [M, N]
    int M, N, K;
    int tiles_m, tiles_n;
};

typedef __attribute__((address_space(3))) void lds_void;

template <int I>
using ic = std::integral_constant<int, I>;

constexpr int ROWB = 128;  // bytes (= k) per tile row and step

// BM x BN tile, WM x WN waves. Two instances: 256 x 256 with 2 x 4 waves (one workgroup per CU) and
// 128 x 128 with 2 x 4 waves of 64 x 32 (64 KB of LDS: two per CU) for outputs too small to fill the
// device with the large tile; with 2 x 2 waves of 64 x 64 it was 5-12 % slower (one wave per SIMD
// when a workgroup has a CU to itself).
template <int BM, int BN, int WM, int WN, int NS>
__global__ __launch_bounds__(64 * WM * WN) void gemm_i8_tile_kernel(I8Params p) {
    static_assert(NS == 2 || NS == 4, "two or four stages");
    constexpr int NT = 64 * WM * WN;
    constexpr int A_STAGE = BM * ROWB;       // A rows, then B rows
    constexpr int STAGE = (BM + BN) * ROWB;
    constexpr int TM = BM / WM, TN = BN / WN;  // wave tile
    constexpr int FM = TM / 32, FN = TN / 32;
    constexpr int LA = BM * 8 / NT, LB = BN * 8 / NT;  // 16-byte loads per thread and stage: A, then B
    static_assert(BM * 8 % NT == 0 && BN * 8 % NT == 0 && LA >= 1 && LB >= 1, "a stage divides over the threads");
    __shared__ __attribute__((aligned(16))) unsigned char lds_all[NS * STAGE];
    unsigned char *const lds0 = lds_all;
    auto stage = [&](auto i) -> unsigned char * { return lds_all + decltype(i)::value * STAGE; };

    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int lane = threadIdx.x & 63;
    const int r = lane & 31, h = lane >> 5;
    const int wm = wave % WM, wn = wave / WM;

    // Workgroup ids are dealt round-robin over the 8 XCDs (id % 8): give each XCD a contiguous
    // range of the tile sequence, ordered in bands of GN tile columns walked row by row, so the
    // workgroups resident on one XCD share a few A row-blocks and B column-blocks in its L2.
    const int nwg = p.tiles_m * p.tiles_n;
    int id = blockIdx.x;
    {
        const int per = nwg / 8;
        if (id < per * 8) id = (id % 8) * per + id / 8;
    }
    constexpr int GN = 8;
    const int band = id / (p.tiles_m * GN);
    const int within = id - band * (p.tiles_m * GN);
    const int rest = p.tiles_n - band * GN;
    const int bw = rest < GN ? rest : GN;
    const int tile_m = within / bw, tile_n = band * GN + within % bw;
    const int m0 = tile_m * BM, c0 = tile_n * BN;
    const int nk = p.K / ROWB;

    // ---- staging: 2048 16-byte slots per operand and stage; slot s = i*512 + thread -> row s/8,
    // position s%8. Rows past the end of a matrix re-read its last row (their results are dropped).
    unsigned a_off[LA], b_off[LB];
#pragma unroll
    for (int i = 0; i < (LA > LB ? LA : LB); ++i) {
        const int row = i * (NT / 8) + (int)(threadIdx.x >> 3);
        const int pos = threadIdx.x & 7;
        const int chunk = pos ^ ((row >> 1) & 7);
        int ga = m0 + row, gb = c0 + row;
        ga = ga < p.M ? ga : p.M - 1;
        gb = gb < p.N ? gb : p.N - 1;
        if (i < LA) a_off[i] = (unsigned)((long long)(ga - m0) * p.K + chunk * 16);
        if (i < LB) b_off[i] = (unsigned)((long long)(gb - c0) * p.K + chunk * 16);
    }
    const unsigned char *a_base = p.x + (long long)m0 * p.K;
    const unsigned char *b_base = p.w + (long long)c0 * p.K;
    // load i of a step: 0..LA-1 fill the A rows of the stage, LA..LA+LB-1 its B rows
    auto issue_one = [&](int kt, unsigned char *st, int i) {
        const bool is_b = i >= LA;
        const int ii = is_b ? i - LA : i;
        const unsigned char *src = (is_b ? b_base : a_base) + (long long)kt * ROWB;
        const unsigned lds_addr = (unsigned)reinterpret_cast<size_t>(
            (lds_void *)(st + (is_b ? A_STAGE : 0) + (ii * NT + wave * 64) * 16));
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                     :: "s"(lds_addr), "v"(is_b ? b_off[ii < LB ? ii : 0] : a_off[ii < LA ? ii : 0]), "s"(src) : "memory");
    };

    // ---- fragments: tile row x + r, chunk (4h + t) at position chunk ^ ((r >> 1) & 7)
    int frag[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) frag[t] = r * ROWB + (((4 * h + t) ^ ((r >> 1) & 7)) << 4);
    const int a_rows = wm * TM * ROWB, b_rows = A_STAGE + wn * TN * ROWB;
    auto read_frags = [&](const unsigned char *st, int t, u32x4_t *af, u32x4_t *bf) {
#pragma unroll
        for (int j = 0; j < FM; ++j) af[j] = *reinterpret_cast<const u32x4_t *>(st + a_rows + j * 32 * ROWB + frag[t]);
#pragma unroll
        for (int i = 0; i < FN; ++i) bf[i] = *reinterpret_cast<const u32x4_t *>(st + b_rows + i * 32 * ROWB + frag[t]);
    };

    i32x16_t acc[FN][FM];
#pragma unroll
    for (int i = 0; i < FN; ++i)
#pragma unroll
        for (int j = 0; j < FM; ++j)
#pragma unroll
            for (int q = 0; q < 16; ++q) acc[i][j][q] = 0;

    u32x4_t af[2][FM], bf[2][FN];
    // Step kt on stage S = kt % NS: the operands of its first slice are already in af[0] / bf[0].
    // Loads run NS - 1 steps ahead: the barrier of a step releases its stage, into which the last
    // slice issues the A half of step kt + NS and the next step's first slice the B half; the wait
    // in front of a barrier leaves the loads of the NS - 2 steps after the next one in flight.
    auto step = [&](int kt, auto si) {
        constexpr int S = decltype(si)::value;
        unsigned char *cur = stage(ic<S>()), *nxt = stage(ic<(S + 1) % NS>()), *prv = stage(ic<(S + NS - 1) % NS>());
        const int kt_b = kt + NS - 1 < nk ? kt + NS - 1 : nk - 1, kt_a = kt + NS < nk ? kt + NS : nk - 1;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            if (t == 3) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"((NS - 2) * (LA + LB)) : "memory");
            if (t < 3) read_frags(cur, t + 1, af[(t + 1) & 1], bf[(t + 1) & 1]);
            else read_frags(nxt, 0, af[0], bf[0]);
            if (t == 0) {
                // B half of the loads of step kt + NS - 1 (its stage was released by the previous barrier)
#pragma unroll
                for (int i = LA; i < LA + LB; ++i) issue_one(kt_b, prv, i);
            }
            if (t == 3) {
                // A half of the loads of step kt + NS, into the stage just released
#pragma unroll
                for (int i = 0; i < LA; ++i) issue_one(kt_a, cur, i);
            }
            // the reads and loads above go out before this slice's MFMAs, which cover their latency
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < FN; ++i)
#pragma unroll
                for (int j = 0; j < FM; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(__builtin_bit_cast(i32x4_t, bf[t & 1][i]),
                                                                     __builtin_bit_cast(i32x4_t, af[t & 1][j]), acc[i][j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // prologue: steps 0 .. NS-2 entirely, the A half of step NS-1; wait for step 0 (everything but the
    // loads issued after it)
    auto issue_step = [&](int kt, unsigned char *st, int first, int last) {
        const int k = kt < nk ? kt : nk - 1;
#pragma unroll
        for (int i = first; i < last; ++i) issue_one(k, st, i);
    };
    issue_step(0, stage(ic<0>()), 0, LA + LB);
    if constexpr (NS == 4) {
        issue_step(1, stage(ic<1>()), 0, LA + LB);
        issue_step(2, stage(ic<2>()), 0, LA + LB);
    }
    issue_step(NS - 1, stage(ic<NS - 1>()), 0, LA);
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"((NS - 2) * (LA + LB) + LA) : "memory");
    read_frags(lds0, 0, af[0], bf[0]);
    __builtin_amdgcn_sched_barrier(0);
    int kt = 0;
    if constexpr (NS == 2) {
        for (; kt + 2 <= nk; kt += 2) {
            step(kt, ic<0>());
            step(kt + 1, ic<1>());
        }
        if (kt < nk) step(kt, ic<0>());
    } else {
        for (; kt + 4 <= nk; kt += 4) {
            step(kt, ic<0>());
            step(kt + 1, ic<1>());
            step(kt + 2, ic<2>());
            step(kt + 3, ic<3>());
        }
        if (kt < nk) step(kt, ic<0>());
        if (kt + 1 < nk) step(kt + 1, ic<1>());
        if (kt + 2 < nk) step(kt + 2, ic<2>());
    }
    // the clamped prefetches of the last steps are still writing LDS: drain them
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    // ---- epilogue: acc[i][j][q]: column c0 + TN*wn + 32i + 8*(q/4) + 4h + q%4, row m0 + TM*wm + 32j + r.
    // Every wave passes its block through a private LDS area, 32 rows (one j) at a time, and stores
    // 16 bytes per lane with TN/8 lanes on the contiguous bytes of a row.
    __syncthreads();
    constexpr int EP = TN * 2 + 16;   // row pitch of the staging area
    constexpr int LPR = TN / 8;        // lanes per staged row (16 bytes each)
    constexpr int RPI = 64 / LPR;      // rows per store instruction
    static_assert(NT / 64 * 32 * EP <= NS * STAGE, "epilogue staging fits the stages");
    unsigned char *ep = lds0 + wave * (32 * EP);
    const int ep_row = lane / LPR, ep_chunk = lane % LPR;
    const int cw0 = c0 + wn * TN;
    const int c_lane = cw0 + ep_chunk * 8;  // first of the 8 columns this lane stores
    float bias_v[FN][4][4], sw_v[FN][4][4];
#pragma unroll
    for (int i = 0; i < FN; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int c = cw0 + i * 32 + 8 * q + 4 * h;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const bool in = c + e < p.N;
                bias_v[i][q][e] = (p.bias && in) ? lq_bf16_bits_to_f32(p.bias[c + e]) : 0.0f;
                sw_v[i][q][e] = !in ? 0.0f : p.sw_bf16 ? lq_bf16_bits_to_f32(reinterpret_cast<const unsigned short *>(p.sw)[c + e]) : p.sw[c + e];
            }
        }
#pragma unroll
    for (int j = 0; j < FM; ++j) {
        const int mrow0 = m0 + wm * TM + j * 32;
        const int m = mrow0 + r;
        const float sxm = m < p.M ? p.sx[m] : 0.0f;
#pragma unroll
        for (int i = 0; i < FN; ++i) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    v[e] = ((float)acc[i][j][4 * q + e] * sxm) * sw_v[i][q][e];
                    if (p.bias) v[e] += bias_v[i][q][e];
                }
                u32x2_t o = {lq_pack_bf16(v[0], v[1]), lq_pack_bf16(v[2], v[3])};
                *reinterpret_cast<u32x2_t *>(ep + r * EP + (i * 32 + 8 * q + 4 * h) * 2) = o;
                const int c = cw0 + i * 32 + 8 * q + 4 * h;
                if (p.acc_out && m < p.M && c < p.N) {
                    i32x4_t a4 = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
                    *reinterpret_cast<i32x4_t *>(p.acc_out + (long long)m * p.N + c) = a4;
                }
            }
        }
#pragma unroll
        for (int it = 0; it < 32 / RPI; ++it) {
            const int row = it * RPI + ep_row;
            const u32x4_t o = *reinterpret_cast<const u32x4_t *>(ep + row * EP + ep_chunk * 16);
            const int mm = mrow0 + row;
            if (mm < p.M && c_lane < p.N) *reinterpret_cast<u32x4_t *>(p.y + (long long)mm * p.N + c_lane) = o;
        }
    }
}

}  // namespace

// Number of 256 x 256 tiles of an [M, N] output.
long long lq_gemm_i8_256_workgroups(int M, int N) { return (long long)((M + 255) / 256) * ((N + 255) / 256); }

// Called by lq_a8w8_fwd (lq_gemm.hip) after argument validation: K % 128 == 0, N % 16 == 0.
// tile = 256 or 128 (square tiles, 8 waves each); stages = 2, or 4 with the 128 tile.
int lq_gemm_i8_tile_launch(const void *x8, const void *w8, const float *sx, const void *sw, bool sw_bf16, const void *bias, void *y,
                           int *acc_or_null, int M, int N, int K, int tile, int stages, hipStream_t st) {
    I8Params p = {};
    p.x = (const unsigned char *)x8; p.w = (const unsigned char *)w8; p.sx = sx; p.sw = (const float *)sw; p.sw_bf16 = sw_bf16;
    p.bias = (const unsigned short *)bias; p.y = (unsigned short *)y; p.acc_out = acc_or_null;
    p.M = M; p.N = N; p.K = K;
    p.tiles_m = (M + tile - 1) / tile;
    p.tiles_n = (N + tile - 1) / tile;
    const long long nwg = (long long)p.tiles_m * p.tiles_n;
    if (nwg > 0x7FFFFFFFll) return lq_fail(LQ_ERR_BAD_ARG, "lq_a8w8_fwd: problem too large");
    // the 32-bit lane offsets of the loads span up to 256 rows
    if (256ll * K >= (1ll << 32)) return lq_fail(LQ_ERR_BAD_ARG, "lq_a8w8_fwd: K too large");
    if (tile == 256) hipLaunchKernelGGL((gemm_i8_tile_kernel<256, 256, 2, 4, 2>), dim3((unsigned)nwg), dim3(512), 0, st, p);
    else if (stages == 4) hipLaunchKernelGGL((gemm_i8_tile_kernel<128, 128, 2, 4, 4>), dim3((unsigned)nwg), dim3(512), 0, st, p);
    else hipLaunchKernelGGL((gemm_i8_tile_kernel<128, 128, 2, 4, 2>), dim3((unsigned)nwg), dim3(512), 0, st, p);
    return lq_check_launch("lq_a8w8_fwd");
}
