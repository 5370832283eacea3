// Weights-direct forward GEMM for gfx950:
//   A16W4, M > 16:  Y[M,N] = X[M,K] . deq(W)[N,K]^T (+ bias), bf16 MFMA
//   and, from the same loop, H[M,N] = silu(X . deq(Wg)^T) * (X . deq(Wu)^T) for the gate / up pair of a
//   gated MLP (the fused product of the reference's PTQ/quant/fused_mlp.py:85-168): a wave's two column
//   tiles then are the same 32 output columns of the two matrices, and the product is formed on the fp32
//   accumulators in the epilogue.
//
// The weights never pass through LDS. An MFMA B-side lane needs 8 consecutive k of one weight
// row, and 8 consecutive k of a row are exactly one 32-bit word of packed codes: every lane
// loads the 16 bytes (32 codes) of its own weight row straight from global memory, dequantises
// them in registers and feeds the matrix core. LDS only holds the activation tile, written by
// LDS-direct loads (no registers, no vector-ALU work) and read as fragments.
//
// Per CU this halves the LDS traffic of a tile scheme that stages both operands (LDS write
// bandwidth on this chip is ~1/3 of its read bandwidth, and the LDS pipe, not the matrix core,
// is what such a scheme saturates), and it removes the producer/consumer hand-off for B.
//
// Workgroup: 128 rows (m) x 256 columns (n), 4 waves side by side along n; a wave owns a
// 128 x 64 block (4 x 2 MFMA 32x32x16 tiles, 128 accumulator registers). With <= 256 VGPRs and
// 48 KB of LDS two workgroups share a CU, so one group's barrier and load latencies are covered
// by the other's MFMAs.
//
// Reduction step = 64 k. Lane l of a wave: r = l % 32, h = l / 32.
//   * B: for each of the wave's two 32-column tiles the lane loads 16 bytes of row n = tile
//     base + r at k offset 64*step + 32*h. Word t (t = 0..3) holds k = 32h + 8t .. +7 and becomes
//     the lane's operand of reduction slice t.
//   * A: slice t therefore needs, for row m and half h, the 16 bytes at k = 32h + 8t: chunk
//     4h + t of the 128-byte tile row. Chunk c of row m sits at position c ^ ((m >> 1) & 7),
//     which makes the 16-lane fragment reads conflict-free; the swizzle costs nothing because an
//     LDS-direct load lets each lane choose which global chunk lands in its (fixed) LDS slot.
//   * D = Wfrag x Xfrag^T: D[i][j] has i = n, j = m, so a lane owns 4 consecutive n of one m;
//     the epilogue regroups them through LDS into 16-byte pieces of full output rows.
//
// Dequantisation is bf16(fma(q, s, -(z*s))): z*s and q*s are exact in fp32, so the fma rounds
// the exact (q - z)*s once; for integer zeros this equals the reference's bf16(bf16(q-z)*s).
//
// Pipeline: A tiles are loaded two steps ahead into three LDS stages, codes one step ahead into
// registers, scales/zeros four groups at a time (8 bytes per row every 8 steps). One s_barrier per
// step, issued without a fence, three quarters of the way through the step; the last quarter
// already prepares the first operands of the next step, so the MFMA stream never drains. The
// global loads are inline assembly with explicit s_waitcnt so that they stay in flight across
// barriers and the compiler's wait insertion never sees them; they are spread over the step, one
// kind per half-slice. Only the odd step's wait covers the codes, scales and zeros requested during the even step before
// it (they are first read after that wait), so a request has 1.75 steps to return: weights come from HBM in any real
// use, and with the wait of the requesting step itself (0.75 steps) the forward down launch ran 5 % slower inside a
// training step than in a loop over the one launch, where they come from the last-level cache.
//
// The chip is power-limited on this kernel (under sustained load the shader clock sits at 1.64 GHz with two
// workgroups per compute unit and at 2.0 GHz with one, against 1.81 GHz for a loop of nothing but MFMAs on
// random operands and 2.38 GHz on all-zero ones; lq_calib_gemm_clocks and lq_calib_mfma_loop measure this), so
// what the loop does besides MFMAs costs throughput even where it overlaps them in time: the forms of the loads
// above are chosen to keep the bytes moved between L2 and the CU near the bytes used.
#include "lq_common.h"

#include <type_traits>

namespace {

struct FwdParams {
    const unsigned char *x;   // bf16 [M, K]
    const unsigned char *w;   // packed codes, K/2 bytes per row
    const unsigned short *scales;
    const unsigned short *zeros;
    const unsigned short *bias;  // bf16 [N] or null
    // gate / up mode: the second matrix (w, scales, zeros are the gate's; no bias)
    const unsigned char *w2;
    const unsigned short *scales2;
    const unsigned short *zeros2;
    unsigned short *y;           // bf16 [M, N]
    // gate / up mode, training form: the two products themselves (bf16 [M, N] each) are stored as well when given
    unsigned short *g_out, *u_out;
    int M, N, K;
    int tiles_m, tiles_n;
    // measurement aid (null in normal use): workgroup w writes the shader-cycle counter and the
    // 100 MHz real-time counter at its start and end to clk[4 w .. 4 w + 3]
    unsigned long long *clk;
};

typedef __attribute__((address_space(3))) void lds_void;

template <int I>
using ic = std::integral_constant<int, I>;

constexpr int BM = 128, BN = 256;
constexpr int ROWB = 128;            // bytes of A per tile row and step: 64 bf16
constexpr int STAGE = BM * ROWB;     // 16 KB per A stage

// NT: 32-column tiles per wave (2: the 128 x 256 workgroup tile described above; 1: 128 x 128, a wave owns
// 128 x 32: twice as many workgroups for outputs whose 128 x 256 tiles leave compute units idle, at the price
// of one fragment read per MFMA instead of half of one).
// GU (with NT = 2): gate / up mode. The workgroup then covers 128 output columns (both matrices' rows
// c0 .. c0 + 127) instead of 256.
template <int NT, bool GU>
__global__ __launch_bounds__(256, 2) void gemm_fwd_direct_kernel(FwdParams p) {
    static_assert(NT == 2 || (NT == 1 && !GU), "gate / up mode uses both column tiles");
    constexpr int BNO = (GU || NT == 1) ? BN / 2 : BN;  // output columns per workgroup
    constexpr int WN = BNO / 4;                         // output columns per wave
    constexpr int ESZ = 2;    // bytes per A element
    constexpr int WROW = 32;  // bytes of one weight row consumed per step
    // 16-byte weight loads per lane and column tile in one batch: the pieces of two consecutive
    // steps (steps 2j and 2j+1 are 64 contiguous bytes of a row across the two lane halves: fetched
    // together they pull their cache line through L1 twice instead of four times)
    constexpr int NB = 2;
    __shared__ __attribute__((aligned(16))) unsigned char lds_a0[STAGE];
    __shared__ __attribute__((aligned(16))) unsigned char lds_a1[STAGE];
    __shared__ __attribute__((aligned(16))) unsigned char lds_a2[STAGE];
    auto abuf = [&](auto i) -> unsigned char * {
        constexpr int I = decltype(i)::value;
        return I == 0 ? lds_a0 : I == 1 ? lds_a1 : lds_a2;
    };

    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int lane = threadIdx.x & 63;
    const int r = lane & 31, h = lane >> 5;
    unsigned long long clk_t0 = 0, clk_r0 = 0;
    if (p.clk) {
        clk_t0 = __builtin_amdgcn_s_memtime();
        clk_r0 = __builtin_amdgcn_s_memrealtime();
    }

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
    const int m0 = tile_m * BM, c0 = tile_n * BNO;
    const int nk = p.K * ESZ / ROWB;
    const long long lda = (long long)p.K * ESZ;

    // ---- A staging: 1024 16-byte slots per stage; slot s = i*256 + thread -> row s/8, position s%8
    unsigned a_off[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = i * 32 + (int)(threadIdx.x >> 3);
        const int pos = threadIdx.x & 7;
        const int chunk = pos ^ ((row >> 1) & 7);
        int gr = m0 + row;
        gr = gr < p.M ? gr : p.M - 1;
        a_off[i] = (unsigned)((long long)(gr - m0) * lda + chunk * 16);
    }
    const unsigned char *a_base = p.x + (long long)m0 * lda;
    auto issue_a_one = [&](int kt, unsigned char *la, int i) {
        const unsigned char *src = a_base + (long long)kt * ROWB;
        const unsigned lds_addr = (unsigned)reinterpret_cast<size_t>((lds_void *)(la + (i * 256 + wave * 64) * 16));
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                     :: "s"(lds_addr), "v"(a_off[i]), "s"(src) : "memory");
    };
    auto issue_a = [&](int kt, unsigned char *la) {
#pragma unroll
        for (int i = 0; i < 4; ++i) issue_a_one(kt, la, i);
    };

    // ---- A fragments: row 32j + r, chunk (4h + t) ^ ((r >> 1) & 7)
    int a_frag[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) a_frag[t] = r * 128 + (((4 * h + t) ^ ((r >> 1) & 7)) << 4);

    // ---- B: buffer descriptors over this workgroup's weight rows (rows past N read as zero), the
    // lane's two rows as 32-bit offsets, the reduction step as the scalar offset
    const int groups_per_row = p.K / LQ_GROUP;
    const int rows_here = p.N - c0 < BNO ? p.N - c0 : BNO;
    auto make_rsrc = [](const void *base, unsigned bytes) {
        const unsigned long long a = (unsigned long long)base;
        u32x4_t d = {(unsigned)a, (unsigned)(a >> 32) & 0xFFFFu, bytes, 0x00020000u};
        return d;
    };
    const unsigned wpitch = (unsigned)(p.K / 2);  // bytes per weight row
    const u32x4_t w_rsrc0 = make_rsrc(p.w + (long long)c0 * wpitch, (unsigned)rows_here * wpitch);
    const u32x4_t s_rsrc0 = make_rsrc(p.scales + (long long)c0 * groups_per_row, (unsigned)rows_here * groups_per_row * 2u);
    const u32x4_t z_rsrc0 = make_rsrc(p.zeros + (long long)c0 * groups_per_row, (unsigned)rows_here * groups_per_row * 2u);
    // column tile 1 reads the second matrix in gate / up mode, the same one otherwise
    const u32x4_t w_rsrc1 = GU ? make_rsrc(p.w2 + (long long)c0 * wpitch, (unsigned)rows_here * wpitch) : w_rsrc0;
    const u32x4_t s_rsrc1 = GU ? make_rsrc(p.scales2 + (long long)c0 * groups_per_row, (unsigned)rows_here * groups_per_row * 2u) : s_rsrc0;
    const u32x4_t z_rsrc1 = GU ? make_rsrc(p.zeros2 + (long long)c0 * groups_per_row, (unsigned)rows_here * groups_per_row * 2u) : z_rsrc0;
    unsigned w_off[NT], q_off[NT];
#pragma unroll
    for (int i = 0; i < NT; ++i) {
        const unsigned n = GU ? wave * 32 + r : wave * WN + i * 32 + r;
        w_off[i] = n * wpitch + h * (WROW / 2);
        q_off[i] = n * (unsigned)groups_per_row * 2u;
    }

    f32x16_t acc[NT][4];
#pragma unroll
    for (int i = 0; i < NT; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int q = 0; q < 16; ++q) acc[i][j][q] = 0;

    // All global loads of the loop are inline assembly: the compiler then inserts no vmcnt waits of
    // its own (it could only wait for everything, LDS-direct loads included); the single
    // s_waitcnt of a step is tied to the loaded registers instead.
    u32x4_t cw[NT][NB], cn[NT][NB];  // codes of the current and of the next batch
    // Raw bf16 scales / zeros of four consecutive groups of the lane's two rows (one 8-byte load per
    // row every 8 steps: a 2-byte load per group would pull a whole cache line through L1 each time).
    // The 8-byte loads need 4-byte aligned rows: the launcher requires an even number of groups per row.
    u32x2_t qs[NT], qz[NT];
    float s[NT], nzs[NT];
    auto load_codes_one = [&](int kt, u32x4_t (*c)[NB], int i) {
        const u32x4_t w_rsrc = i == 0 ? w_rsrc0 : w_rsrc1;
        asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen" : "=v"(c[i][0]) : "v"(w_off[i]), "s"(w_rsrc), "s"(kt * WROW));
        asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen offset:32" : "=v"(c[i][1]) : "v"(w_off[i]), "s"(w_rsrc), "s"(kt * WROW));
    };
    auto load_codes = [&](int kt, u32x4_t (*c)[NB]) {
#pragma unroll
        for (int i = 0; i < NT; ++i) load_codes_one(kt, c, i);
    };
    // Called on the even step two steps before group g starts; loads when g opens a quad.
    auto load_qparams_one = [&](int g, int i) {
        if ((g & 3) != 0) return;
        const u32x4_t s_rsrc = i == 0 ? s_rsrc0 : s_rsrc1;
        const u32x4_t z_rsrc = i == 0 ? z_rsrc0 : z_rsrc1;
        asm volatile("buffer_load_dwordx2 %0, %1, %2, %3 offen" : "=v"(qs[i]) : "v"(q_off[i]), "s"(s_rsrc), "s"(g * 2));
        asm volatile("buffer_load_dwordx2 %0, %1, %2, %3 offen" : "=v"(qz[i]) : "v"(q_off[i]), "s"(z_rsrc), "s"(g * 2));
    };
    auto load_qparams = [&](int g) {
#pragma unroll
        for (int i = 0; i < NT; ++i) load_qparams_one(g, i);
    };
    auto use_qparams = [&](int g) {
        const int shift = (g & 3) * 16;
#pragma unroll
        for (int i = 0; i < NT; ++i) {
            const unsigned long long s4 = ((unsigned long long)qs[i][1] << 32) | qs[i][0];
            const unsigned long long z4 = ((unsigned long long)qz[i][1] << 32) | qz[i][0];
            const float sc = __uint_as_float((unsigned)(s4 >> shift) << 16);
            nzs[i] = -(__uint_as_float((unsigned)(z4 >> shift) << 16) * sc);
            s[i] = sc * 512.0f;  // the codes come out of the conversion as q/512
        }
    };
    auto read_a = [&](const unsigned char *la, int t, u32x4_t *af) {
#pragma unroll
        for (int j = 0; j < 4; ++j) af[j] = *reinterpret_cast<const u32x4_t *>(la + j * 4096 + a_frag[t]);
    };
    // par = which step of the batch
    auto deq_one = [&](const u32x4_t (*c)[NB], int par, int t, u32x4_t *bf, int i) {
        float f[8];
        lq_dequant_word_f32(c[i][par][t], s[i], nzs[i], f);
        bf[i] = u32x4_t{lq_pack_bf16(f[0], f[1]), lq_pack_bf16(f[2], f[3]), lq_pack_bf16(f[4], f[5]),
                        lq_pack_bf16(f[6], f[7])};
    };
    auto mfma_half = [&](const u32x4_t *af, const u32x4_t *bf, int i) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, bf[i]),
                                                               __builtin_bit_cast(bf16x8_t, af[j]), acc[i][j], 0, 0, 0);
    };

    // The one synchronisation point of a step (and the end of the prologue): everything this wave
    // loaded has arrived except the NEWEST newest loads, its fragment reads have returned: meet the
    // other waves. The wait is tied to the registers the assembly loads wrote.
    auto wait_and_meet = [&](auto newest, auto with_qparams) {
        constexpr int NEWEST = decltype(newest)::value;
        (void)cn; (void)qs; (void)qz;  // named outside the constexpr branches so that the lambda captures them
        if constexpr (decltype(with_qparams)::value == 2) {
            // a wait that releases no loaded register: nothing requested since the previous wait is read before the next one
            asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" :: "n"(NEWEST) : "memory");
        } else if constexpr (NT == 2) {
            if constexpr (decltype(with_qparams)::value != 0) {
                asm volatile("s_waitcnt vmcnt(%8) lgkmcnt(0)\n\ts_barrier"
                             : "+v"(cn[0][0]), "+v"(cn[0][1]), "+v"(cn[NT - 1][0]), "+v"(cn[NT - 1][1]), "+v"(qs[0]), "+v"(qs[NT - 1]),
                               "+v"(qz[0]), "+v"(qz[NT - 1]) : "n"(NEWEST) : "memory");
            } else {
                asm volatile("s_waitcnt vmcnt(%4) lgkmcnt(0)\n\ts_barrier"
                             : "+v"(cn[0][0]), "+v"(cn[0][1]), "+v"(cn[NT - 1][0]), "+v"(cn[NT - 1][1]) : "n"(NEWEST) : "memory");
            }
        } else {
            if constexpr (decltype(with_qparams)::value != 0) {
                asm volatile("s_waitcnt vmcnt(%4) lgkmcnt(0)\n\ts_barrier"
                             : "+v"(cn[0][0]), "+v"(cn[0][1]), "+v"(qs[0]), "+v"(qz[0]) : "n"(NEWEST) : "memory");
            } else {
                asm volatile("s_waitcnt vmcnt(%2) lgkmcnt(0)\n\ts_barrier" : "+v"(cn[0][0]), "+v"(cn[0][1]) : "n"(NEWEST) : "memory");
            }
        }
    };

    // Operands of the first reduction slice of the step about to run; slice 3 of every step
    // prepares them for the step after it, so the MFMA stream continues across the step boundary.
    u32x4_t af[2][4], bf[2][NT];

    // One reduction step on stage AI with the codes in cw, cut into 8 half-slices of 4 MFMAs (one
    // column tile x four row tiles of one reduction slice). A half-slice also issues the fragment
    // reads and the dequantisation its counterpart in the next slice needs, and at most one kind of
    // global load: a burst of loads would hold the wave at the memory pipeline's queue with its
    // MFMAs behind it. Load order within a step: next step's codes (half-slices 0, 1), on even steps
    // the next group's scale and zero (2, 3), the LDS-direct loads of the tile two steps ahead
    // (4..7). Before half-slice 6 the wave waits for all but the two newest loads, which covers tile
    // kt+1 and the codes of step kt+1, and meets the other waves; slice 3 then reads the first
    // fragments of tile kt+1 and dequantises the first words of step kt+1 (on odd steps with the
    // next group's scale and zero). That barrier also orders this step's reads of stage AI before
    // the next step's loads into it.
    auto step = [&](int kt, auto ai, auto odd) {
        constexpr int AI = decltype(ai)::value;
        constexpr bool ODD = decltype(odd)::value != 0;
        const unsigned char *la = abuf(ic<AI>());
        const unsigned char *la_after = abuf(ic<(AI + 1) % 3>());
        unsigned char *la_load = abuf(ic<(AI + 2) % 3>());
        // the codes of the next pair of steps are loaded on even steps
        const int kt_codes = kt + 2 < nk ? kt + 2 : kt;
        const int kt_a = kt + 2 < nk ? kt + 2 : nk - 1;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
#pragma unroll
            for (int i = 0; i < NT; ++i) {
                if (t == 3 && i == 0) {
                    // Odd step: everything but the two LDS-direct loads just issued has to be here (tile kt+1, and the
                    // codes, scales and zeros the even step before requested: slice 3 starts on them). Even step: only
                    // what earlier steps requested (tile kt+1); its own requests (2 NT code loads, then 2 LDS-direct
                    // loads; on every eighth step 2 NT scale / zero loads in between, which makes the count
                    // conservative there) may stay in flight until the next step's wait, so that codes coming from
                    // HBM have 1.75 steps to arrive instead of 0.75.
                    if constexpr (ODD) wait_and_meet(ic<2>(), ic<1>());
                    else wait_and_meet(ic<2 * NT + 2>(), ic<2>());
                    if (ODD) use_qparams((kt + 1) >> 1);
                }
                const unsigned char *src = t < 3 ? la : la_after;
                const int tn = (t + 1) & 3;
                // all four fragments of the next slice in the first half: a full slice of MFMAs covers
                // their LDS latency
                if (i == 0) read_a(src, tn, af[tn & 1]);
                if (t < 3) deq_one(cw, ODD ? 1 : 0, tn, bf[tn & 1], i);
                else if (ODD) deq_one(cn, 0, 0, bf[0], i);
                else deq_one(cw, 1, 0, bf[0], i);
                if (t == 0 && !ODD) load_codes_one(kt_codes, cn, i);
                if (t == 1 && !ODD) load_qparams_one((kt + 2) >> 1 < groups_per_row ? (kt + 2) >> 1 : groups_per_row - 1, i);
                if (t >= 2) {
                    if constexpr (NT == 2) {
                        issue_a_one(kt_a, la_load, 2 * (t - 2) + i);
                    } else {
                        issue_a_one(kt_a, la_load, 2 * (t - 2));
                        issue_a_one(kt_a, la_load, 2 * (t - 2) + 1);
                    }
                }
                mfma_half(af[t & 1], bf[t & 1], i);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if (ODD) {
#pragma unroll
            for (int i = 0; i < NT; ++i)
#pragma unroll
                for (int b = 0; b < NB; ++b) cw[i][b] = cn[i][b];
        }
    };

    load_qparams(0);
    load_codes(0, cn);
    issue_a(0, lds_a0);
    issue_a(nk > 1 ? 1 : 0, lds_a1);
    wait_and_meet(ic<4>(), ic<1>());
#pragma unroll
    for (int i = 0; i < NT; ++i)
#pragma unroll
        for (int b = 0; b < NB; ++b) cw[i][b] = cn[i][b];
    use_qparams(0);
    read_a(lds_a0, 0, af[0]);
#pragma unroll
    for (int i = 0; i < NT; ++i) deq_one(cw, 0, 0, bf[0], i);
    __builtin_amdgcn_sched_barrier(0);
    int kt = 0;
    for (; kt + 6 <= nk; kt += 6) {
        step(kt, ic<0>(), ic<0>());
        step(kt + 1, ic<1>(), ic<1>());
        step(kt + 2, ic<2>(), ic<0>());
        step(kt + 3, ic<0>(), ic<1>());
        step(kt + 4, ic<1>(), ic<0>());
        step(kt + 5, ic<2>(), ic<1>());
    }
    // kt is a multiple of 6 here, so the stage and parity phases restart at 0; 0..5 steps remain
    // (an even number: K is a multiple of 128 = two steps)
    const int rem = nk - kt;
    if (rem > 0) step(kt, ic<0>(), ic<0>());
    if (rem > 1) step(kt + 1, ic<1>(), ic<1>());
    if (rem > 2) step(kt + 2, ic<2>(), ic<0>());
    if (rem > 3) step(kt + 3, ic<0>(), ic<1>());
    if (rem > 4) step(kt + 4, ic<1>(), ic<0>());
    // the clamped prefetches of the last two steps are still writing LDS: drain them
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    __syncthreads();
    if constexpr (GU || NT == 1) {
        // ---- 32 output columns per wave: column c0 + 32*wave + 8*(q/4) + 4h + q%4, row m0 + 32j + r.
        // Gate / up mode: acc[0] and acc[1] hold the same output element of the two products and
        // H = silu(gate) * up is formed on the fp32 accumulators, rounded once. A wave's 32 rows x 32
        // columns pass through LDS (row pitch 80 bytes) and leave as 16 bytes per lane, 4 lanes on the 64
        // contiguous bytes of a row.
        constexpr int EP = 80;
        unsigned char *ep = ((wave & 2) ? lds_a1 : lds_a0) + (wave & 1) * (32 * EP);
        const int ep_row = lane >> 2, ep_chunk = lane & 3;
        const int c_lane = c0 + wave * WN + ep_chunk * 8;
        float bias_n[4][4];
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int c = c0 + wave * WN + 8 * q + 4 * h + e;
                bias_n[q][e] = (!GU && p.bias && c < p.N) ? lq_bf16_bits_to_f32(p.bias[c]) : 0.0f;
            }
        // which = 0: the output (H, or Y with one matrix); 1, 2 (gate / up mode with g_out): the two products
        const int n_out = (GU && p.g_out) ? 3 : 1;
        for (int which = 0; which < n_out; ++which) {
            unsigned short *dst = which == 0 ? p.y : which == 1 ? p.g_out : p.u_out;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    float v[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float g = acc[0][j][4 * q + e];
                        if constexpr (GU) {
                            const float u = acc[NT - 1][j][4 * q + e];
                            v[e] = which == 0 ? g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)) * u : which == 1 ? g : u;
                        } else {
                            v[e] = g;
                            if (p.bias) v[e] += bias_n[q][e];
                        }
                    }
                    u32x2_t o = {lq_pack_bf16(v[0], v[1]), lq_pack_bf16(v[2], v[3])};
                    *reinterpret_cast<u32x2_t *>(ep + r * EP + (8 * q + 4 * h) * 2) = o;
                }
#pragma unroll
                for (int it = 0; it < 2; ++it) {
                    const int row = it * 16 + ep_row;
                    const u32x4_t o = *reinterpret_cast<const u32x4_t *>(ep + row * EP + ep_chunk * 16);
                    const int mm = m0 + j * 32 + row;
                    if (mm < p.M && c_lane < p.N) *reinterpret_cast<u32x4_t *>(dst + (long long)mm * p.N + c_lane) = o;
                }
            }
        }
    } else {
    // ---- epilogue: acc[i][j][q]: column c0 + 64*wave + 32i + 8*(q/4) + 4h + q%4, row m0 + 32j + r.
    // A lane holds 4 consecutive columns of one row: stored straight from the registers, an
    // instruction would touch 32 rows with 16 bytes each. Instead every wave passes its block
    // through LDS, 32 rows (one j) at a time, and stores 16 bytes per lane with 8 lanes on the 128
    // contiguous bytes of a row: full cache lines. The stages are free once every wave has left the
    // loop and its loads have landed; a wave's staging area is private (waves 0,1 in stage 0, waves
    // 2,3 in stage 1), row pitch 144 bytes.
    constexpr int EP = 144;
    unsigned char *ep = ((wave & 2) ? lds_a1 : lds_a0) + (wave & 1) * (32 * EP);
    const int ep_row = lane >> 3, ep_chunk = lane & 7;
    const int c_lane = c0 + wave * 64 + ep_chunk * 8;  // first of the 8 columns this lane stores
    float bias_v[2][4][4];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int c = c0 + wave * 64 + i * 32 + 8 * q + 4 * h;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const bool in = c + e < p.N;
                bias_v[i][q][e] = (p.bias && in) ? lq_bf16_bits_to_f32(p.bias[c + e]) : 0.0f;
            }
        }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    v[e] = acc[i][j][4 * q + e];
                    if (p.bias) v[e] += bias_v[i][q][e];
                }
                u32x2_t o = {lq_pack_bf16(v[0], v[1]), lq_pack_bf16(v[2], v[3])};
                *reinterpret_cast<u32x2_t *>(ep + r * EP + (i * 32 + 8 * q + 4 * h) * 2) = o;
            }
        }
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int row = it * 8 + ep_row;
            const u32x4_t o = *reinterpret_cast<const u32x4_t *>(ep + row * EP + ep_chunk * 16);
            const int mm = m0 + j * 32 + row;
            if (mm < p.M && c_lane < p.N) *reinterpret_cast<u32x4_t *>(p.y + (long long)mm * p.N + c_lane) = o;
        }
    }
    }
    if (p.clk && threadIdx.x == 0) {
        unsigned long long *c = p.clk + 4ll * blockIdx.x;
        c[0] = clk_t0; c[1] = __builtin_amdgcn_s_memtime(); c[2] = clk_r0; c[3] = __builtin_amdgcn_s_memrealtime();
    }
}

}  // namespace

// Number of workgroups this kernel would launch; the dispatcher in lq_gemm.hip prefers it when they
// can fill the device two per CU.
long long lq_gemm_fwd_direct_workgroups(int M, int N) { return (long long)((M + BM - 1) / BM) * ((N + BN - 1) / BN); }
long long lq_gemm_fwd_direct128_workgroups(int M, int N) { return (long long)((M + BM - 1) / BM) * ((N + BN / 2 - 1) / (BN / 2)); }

template <int NT, bool GU>
static int launch_direct(FwdParams p, hipStream_t st, const char *who) {
    constexpr int BNO = (GU || NT == 1) ? BN / 2 : BN;
    p.tiles_m = (p.M + BM - 1) / BM;
    p.tiles_n = (p.N + BNO - 1) / BNO;
    const long long nwg = (long long)p.tiles_m * p.tiles_n;
    if (nwg > 0x7FFFFFFFll) return lq_fail(LQ_ERR_BAD_ARG, "%s: problem too large", who);
    // the 32-bit lane offsets of the activation and weight loads span 128 / 256 rows
    if ((long long)BN * p.K * 2 >= (1ll << 32)) return lq_fail(LQ_ERR_BAD_ARG, "%s: K too large", who);
    hipLaunchKernelGGL((gemm_fwd_direct_kernel<NT, GU>), dim3((unsigned)nwg), dim3(256), 0, st, p);
    return lq_check_launch(who);
}

// Called by lq_a16w4_fwd (lq_gemm.hip) after argument validation: K % 256 == 0, N % 16 == 0, M > 16.
int lq_gemm_fwd_direct_launch(const void *x, const void *codes, const void *scales, const void *zeros, const void *bias,
                              void *y, int M, int N, int K, hipStream_t st, unsigned long long *clk, bool narrow) {
    FwdParams p = {};
    p.clk = clk;
    p.x = (const unsigned char *)x; p.w = (const unsigned char *)codes;
    p.scales = (const unsigned short *)scales; p.zeros = (const unsigned short *)zeros;
    p.bias = (const unsigned short *)bias; p.y = (unsigned short *)y;
    p.M = M; p.N = N; p.K = K;
    return narrow ? launch_direct<1, false>(p, st, "lq_a16w4_fwd") : launch_direct<2, false>(p, st, "lq_a16w4_fwd");
}

// Called by lq_a16w4_gate_up_silu (lq_gemm.hip) after argument validation: K % 256 == 0, N % 16 == 0, M > 16.
int lq_gemm_fwd_gate_up_launch(const void *x, const void *codes_g, const void *scales_g, const void *zeros_g,
                               const void *codes_u, const void *scales_u, const void *zeros_u, void *h, void *g_out, void *u_out,
                               int M, int N, int K, hipStream_t st) {
    FwdParams p = {};
    p.x = (const unsigned char *)x;
    p.w = (const unsigned char *)codes_g; p.scales = (const unsigned short *)scales_g; p.zeros = (const unsigned short *)zeros_g;
    p.w2 = (const unsigned char *)codes_u; p.scales2 = (const unsigned short *)scales_u; p.zeros2 = (const unsigned short *)zeros_u;
    p.y = (unsigned short *)h;
    p.g_out = (unsigned short *)g_out; p.u_out = (unsigned short *)u_out;
    p.M = M; p.N = N; p.K = K;
    return launch_direct<2, true>(p, st, "lq_a16w4_gate_up_silu");
}
