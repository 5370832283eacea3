/*
 * lq_oracle.c — CPU restatement of latentQ_LLM's quantized-linear hot path.
 *
 * TEST INFRASTRUCTURE ONLY. Nothing shipped by the package may link, load or
 * call this file; it exists so that tests, the smoke check and the benchmark's
 * CPU-baseline leg can compare the HIP kernels against an independent
 * implementation. Plain C99 + OpenMP, no dependency on the package.
 *
 * Every function names the reference lines it follows (paths relative to the
 * reference checkout). Pinning status (what, besides this file, fixes each
 * result) is listed in the header comment of tests/test_oracle_pins.py; in
 * short:
 *   - pack/unpack, dequant, Philox4x32-10, int32 GEMM: pinned (known answers,
 *     exhaustive checks, Random123 vectors, exact integer arithmetic);
 *   - requant: the formula is this build's own (the reference has no such
 *     function); pinned by an exact rational-arithmetic model and invariants;
 *   - A8W8 bf16 epilogue: "parity unpinned" — the reference calls an external,
 *     un-vendored cutlass kernel (torch_int, FWkey/torch-int-bf16, no pinned
 *     version) whose rounding points cannot be read from the reference.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ---------------------------------------------------------------- bf16 -- */
static inline float bf16_to_f32(uint16_t b) {
    uint32_t u = ((uint32_t)b) << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* Round-to-nearest-even fp32 -> bf16, NaN kept quiet (what torch's
 * c10::BFloat16 conversion does). */
static inline uint16_t f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7FFFu + lsb;
    return (uint16_t)(u >> 16);
}
static inline float bf16_round(float f) { return bf16_to_f32(f32_to_bf16(f)); }

uint16_t lqo_f32_to_bf16(float f) { return f32_to_bf16(f); }
float lqo_bf16_to_f32(uint16_t b) { return bf16_to_f32(b); }

/* ------------------------------------------------------- nibble packing -- */
/* python_compress, utils/quant.py:4-9: byte = (c[2i] << 4) + c[2i+1]. */
void lqo_pack(const uint8_t *codes, uint8_t *packed, int64_t n_codes) {
    for (int64_t i = 0; i < n_codes / 2; ++i)
        packed[i] = (uint8_t)(((codes[2 * i] & 0xF) << 4) | (codes[2 * i + 1] & 0xF));
}
/* python_decompress, utils/quant.py:12-19: hi = (b >> 4) % 16, lo = b % 16. */
void lqo_unpack(const uint8_t *packed, uint8_t *codes, int64_t n_codes) {
    for (int64_t i = 0; i < n_codes / 2; ++i) {
        codes[2 * i] = (uint8_t)(packed[i] >> 4);
        codes[2 * i + 1] = (uint8_t)(packed[i] & 0xF);
    }
}
static inline unsigned code_at(const uint8_t *packed, int64_t i) {
    uint8_t b = packed[i >> 1];
    return (i & 1) ? (b & 0xFu) : (b >> 4);
}

/* ---------------------------------------------------------- dequantise -- */
/* DeQfunc_4bit_g, utils/quant.py:66-72: (codes - zeros) * scales in bf16
 * arithmetic: the int8 code is promoted to bf16, the difference is rounded to
 * bf16, the product is rounded to bf16. */
static inline float deq_elem(unsigned q, float s, float z) {
    float d = bf16_round((float)q - z);
    return bf16_round(d * s);
}

void lqo_dequant(const uint8_t *packed, const uint16_t *scales, const uint16_t *zeros, uint16_t *w_out,
                 int64_t N, int64_t K, int group) {
    int64_t total = N * K;
#pragma omp parallel for schedule(static)
    for (int64_t g = 0; g < total / group; ++g) {
        float s = bf16_to_f32(scales[g]), z = bf16_to_f32(zeros[g]);
        for (int64_t i = g * group; i < (g + 1) * group; ++i)
            w_out[i] = f32_to_bf16(deq_elem(code_at(packed, i), s, z));
    }
}

static float *dequant_f32(const uint8_t *packed, const uint16_t *scales, const uint16_t *zeros, int64_t N,
                          int64_t K, int group) {
    float *w = (float *)malloc(sizeof(float) * (size_t)(N * K));
    if (!w) return NULL;
    int64_t total = N * K;
#pragma omp parallel for schedule(static)
    for (int64_t g = 0; g < total / group; ++g) {
        float s = bf16_to_f32(scales[g]), z = bf16_to_f32(zeros[g]);
        for (int64_t i = g * group; i < (g + 1) * group; ++i) w[i] = deq_elem(code_at(packed, i), s, z);
    }
    return w;
}

/* --------------------------------------------------------- A16W4 GEMMs -- */
/* QLinearFunctionW4.forward, utils/quant.py:116-121: Y = X . deq(W)^T (+ bias).
 * Accumulates in double and rounds once to bf16 (the reference accumulates in
 * fp32 inside cuBLAS with an unspecified order; comparisons use a tolerance).
 * If y_f64 is non-NULL the unrounded sums are also stored there. */
int lqo_a16w4_fwd(const uint16_t *x, const uint8_t *packed, const uint16_t *scales, const uint16_t *zeros,
                  const uint16_t *bias, uint16_t *y, double *y_f64, int64_t M, int64_t N, int64_t K, int group) {
    float *w = dequant_f32(packed, scales, zeros, N, K, group);
    if (!w) return -1;
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        float *xf = (float *)malloc(sizeof(float) * (size_t)K);
        for (int64_t k = 0; k < K; ++k) xf[k] = bf16_to_f32(x[m * K + k]);
        for (int64_t n = 0; n < N; ++n) {
            const float *wr = w + n * K;
            double acc = 0.0;
            for (int64_t k = 0; k < K; ++k) acc += (double)xf[k] * (double)wr[k];
            if (bias) acc += (double)bf16_to_f32(bias[n]);
            if (y_f64) y_f64[m * N + n] = acc;
            y[m * N + n] = f32_to_bf16((float)acc);
        }
        free(xf);
    }
    free(w);
    return 0;
}

/* QLinearFunctionW4.backward, utils/quant.py:136-140: dX = dY . deq(W). */
int lqo_a16w4_dx(const uint16_t *dy, const uint8_t *packed, const uint16_t *scales, const uint16_t *zeros,
                 uint16_t *dx, double *dx_f64, int64_t M, int64_t N, int64_t K, int group) {
    float *w = dequant_f32(packed, scales, zeros, N, K, group);
    if (!w) return -1;
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        double *acc = (double *)calloc((size_t)K, sizeof(double));
        for (int64_t n = 0; n < N; ++n) {
            double d = (double)bf16_to_f32(dy[m * N + n]);
            const float *wr = w + n * K;
            for (int64_t k = 0; k < K; ++k) acc[k] += d * (double)wr[k];
        }
        for (int64_t k = 0; k < K; ++k) {
            if (dx_f64) dx_f64[m * K + k] = acc[k];
            dx[m * K + k] = f32_to_bf16((float)acc[k]);
        }
        free(acc);
    }
    free(w);
    return 0;
}

/* ------------------------------------------------------------- Philox -- */
/* Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3",
 * SC'11; Random123). Not part of the reference: the requantizer's noise
 * source is this build's choice. */
void lqo_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
    uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3], k0 = key[0], k1 = key[1];
    for (int r = 0; r < 10; ++r) {
        uint64_t p0 = (uint64_t)0xD2511F53u * c0;
        uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
        uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
        uint32_t n1 = (uint32_t)p1;
        uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
        uint32_t n3 = (uint32_t)p0;
        c0 = n0; c1 = n1; c2 = n2; c3 = n3;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

/* 16-bit draw of flat element i: half (i & 1; 1 = the high half) of word (i >> 1) & 3 of the block
 * Philox4x32-10(counter = offset + i / 8, key = seed). */
static inline uint32_t philox_draw16(int64_t i, uint64_t seed, uint64_t offset) {
    uint64_t c = offset + (uint64_t)(i >> 3);
    uint32_t ctr[4] = {(uint32_t)c, (uint32_t)(c >> 32), 0u, 0u};
    uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    uint32_t o[4];
    lqo_philox4x32_10(ctr, key, o);
    return (o[(i >> 1) & 3] >> (16 * (i & 1))) & 0xFFFFu;
}

/* 8-bit draw of flat element i (gradient accumulator): byte i & 3 of word (i >> 2) & 3 of the block
 * Philox4x32-10(counter = offset + i / 16, key = seed). */
static inline uint32_t philox_draw8(int64_t i, uint64_t seed, uint64_t offset) {
    uint64_t c = offset + (uint64_t)(i >> 4);
    uint32_t ctr[4] = {(uint32_t)c, (uint32_t)(c >> 32), 0u, 0u};
    uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    uint32_t o[4];
    lqo_philox4x32_10(ctr, key, o);
    return (o[(i >> 2) & 3] >> (8 * (i & 3))) & 0xFFu;
}

/* The noise the gradient accumulator adds for element i when none is injected: (2b - 255) / 512 for the 8-bit
 * draw b, i.e. 256 equally spaced bf16 numbers symmetric about zero, as fp32. */
void lqo_gradq8_noise(float *out, int64_t n, uint64_t seed, uint64_t offset) {
    for (int64_t i = 0; i < n; ++i) out[i] = (2.0f * (float)philox_draw8(i, seed, offset) - 255.0f) / 512.0f;
}

/* The uniform the requantizer adds for element i: (a + 1/2) * 2^-16, on the centred 2^-16 grid. */
void lqo_philox_uniform(float *out, int64_t n, uint64_t seed, uint64_t offset) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) out[i] = ((float)philox_draw16(i, seed, offset) + 0.5f) * 0x1p-16f;
}

/* ------------------------------------------------------------ requant -- */
/* Stochastic latent requantize (benchmark configuration 1). The reference has
 * no function with this formula; its nearest relatives are Qfunc_4bit_g_res
 * (utils/quant.py:45-63, Z = t/s + z then round) and the stochastic rounding
 * round(x + U(-.5,.5)) of GradientQTensor.quant (utils/quant.py:867-871).
 * Operation order, fp32, each line one IEEE rounding:
 *   w = bf16(bf16(q - z) * s);  t = fma(-lr, g, w);  r16 = (1 / s) * 65536;  c16 = fma(z, 65536, 0.5);
 *   y = fma(t, r16, c16);                       (t/s + z) in 16.16 fixed point plus one half
 *   X = NaN or y < 0 -> 0, y >= 2^32 -> 2^32 - 1, else trunc(y);   S = min(X + a, 2^32 - 1);
 *   code = min(S >> 16, 15)                     = clamp(floor(x + (a + 1/2) / 65536), 0, 15)
 * with the 16-bit draw a from the Philox stream (u == NULL) or from an injected uniform:
 * a = NaN or u < 0 -> 0, else min(trunc(u * 65536), 65535). */
static inline uint32_t sat_u32(float y) {
    if (!(y >= 0.0f)) return 0u;
    if (y >= 4294967296.0f) return 0xFFFFFFFFu;
    return (uint32_t)y;
}
void lqo_requant(const uint8_t *packed_in, uint8_t *packed_out, const uint16_t *scales, const uint16_t *zeros,
                 const uint16_t *grad, float lr, int64_t N, int64_t K, int group, const float *u, uint64_t seed,
                 uint64_t offset) {
    int64_t total = N * K;
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < total / 2; ++b) {
        unsigned nib[2];
        for (int h = 0; h < 2; ++h) {
            int64_t i = 2 * b + h;
            float s = bf16_to_f32(scales[i / group]), z = bf16_to_f32(zeros[i / group]);
            float w = deq_elem(code_at(packed_in, i), s, z);
            float t = fmaf(-lr, bf16_to_f32(grad[i]), w);
            volatile float r = 1.0f / s;
            volatile float r16 = r * 65536.0f;
            float c16 = fmaf(z, 65536.0f, 0.5f);
            float y = fmaf(t, r16, c16);
            uint32_t a;
            if (u) {
                volatile float ua = u[i] * 65536.0f;
                a = sat_u32(ua);
                if (a > 65535u) a = 65535u;
            } else {
                a = philox_draw16(i, seed, offset);
            }
            uint64_t S = (uint64_t)sat_u32(y) + a;
            if (S > 0xFFFFFFFFull) S = 0xFFFFFFFFull;
            uint32_t c = (uint32_t)(S >> 16);
            nib[h] = c > 15u ? 15u : c;
        }
        packed_out[b] = (uint8_t)((nib[0] << 4) | nib[1]);
    }
}

/* --------------------------------------------------------------- A8W8 -- */
/* linear_a8_w8_bbf16_obf16 (external torch_int) + `* qscales` as used at
 * utils/quant.py:268-271: acc = X8 . W8^T exactly in int32; the fused epilogue
 * of this build is y = bf16((float(acc) * sx[m]) * sw[n] + bias[n]). */
void lqo_a8w8(const int8_t *x, const int8_t *w, const float *sx, const float *sw, const uint16_t *bias, uint16_t *y,
              int32_t *acc_out, int64_t M, int64_t N, int64_t K) {
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        for (int64_t n = 0; n < N; ++n) {
            int32_t acc = 0;
            const int8_t *xr = x + m * K, *wr = w + n * K;
            for (int64_t k = 0; k < K; ++k) acc += (int32_t)xr[k] * (int32_t)wr[k];
            if (acc_out) acc_out[m * N + n] = acc;
            if (y) {
                volatile float f = (float)acc * sx[m];
                f = f * sw[n];
                if (bias) f = f + bf16_to_f32(bias[n]);
                y[m * N + n] = f32_to_bf16(f);
            }
        }
    }
}

/* Activation quantizer of QLinearFunctionA8W8_dynamic.forward,
 * utils/quant.py:264-266, on a bf16 input with a bf16-valued clamp:
 * input*127. (bf16 product) / clampv (bf16 quotient), round half-even,
 * clamp to [-128,127]. */
void lqo_act_quant_i8(const uint16_t *x, float clampv, int8_t *x8, int64_t n) {
    for (int64_t i = 0; i < n; ++i) {
        float a = bf16_round(bf16_to_f32(x[i]) * 127.0f);
        float q = bf16_round(a / clampv);
        float r = nearbyintf(q); /* default rounding mode: half to even */
        if (r != r) r = 0.0f;
        if (r < -128.0f) r = -128.0f;
        if (r > 127.0f) r = 127.0f;
        x8[i] = (int8_t)r;
    }
}

/* The dynamic layers' quantiser, utils/quant.py:259-266 and 319-322: clampv = input.max() (the tensor
 * library's max: NaN as soon as one element is NaN; of -0 and +0 this restatement takes +0), then
 * lqo_act_quant_i8 with it. out2[0] = clampv, out2[1] = alpha = clampv / 127. as the tensor library's GPU
 * kernels form it (a product with the fp32 reciprocal of the host scalar), rounded to bf16 when alpha_bf16
 * (the training Function divides a bf16 0-dim tensor, :271); sx[m] = alpha for every row. */
void lqo_act_quant_i8_dynamic(const uint16_t *x, int8_t *x8, float *sx, float *out2, int64_t M, int64_t K, int alpha_bf16) {
    const int64_t n = M * K;
    float best = bf16_to_f32(x[0]);
    for (int64_t i = 1; i < n && best == best; ++i) {
        float v = bf16_to_f32(x[i]);
        if (v != v || v > best || (v == best && !signbit(v))) best = v;
    }
    if (best != best) best = bf16_to_f32(0x7FC0);
    volatile float rcp = 1.0f / 127.0f;
    volatile float alpha = best * rcp;
    if (alpha_bf16) alpha = bf16_round(alpha);
    out2[0] = best;
    out2[1] = alpha;
    for (int64_t m = 0; m < M; ++m) sx[m] = alpha;
    lqo_act_quant_i8(x, best, x8, n);
}

/* Per-token form of the same step (this build's addition; the reference quantises per tensor): for every row
 * amax = max |x| (NaN if the row holds one), sx = amax / 127, x8 = clamp(rint(x * (127 / amax)), -128, 127), all
 * in fp32 with IEEE division; NaN -> 0; an all-zero row quantises to zeros with scale 0. */
void lqo_act_quant_i8_per_token(const uint16_t *x, int8_t *x8, float *sx, int64_t M, int64_t K) {
    for (int64_t m = 0; m < M; ++m) {
        const uint16_t *row = x + m * K;
        float amax = 0.0f;
        for (int64_t k = 0; k < K && amax == amax; ++k) {
            float a = fabsf(bf16_to_f32(row[k]));
            if (a != a || a > amax) amax = a;
        }
        volatile float inv = amax == 0.0f ? 0.0f : 127.0f / amax;
        volatile float sc = amax / 127.0f;
        sx[m] = sc;
        for (int64_t k = 0; k < K; ++k) {
            volatile float p = bf16_to_f32(row[k]) * inv;
            float r = nearbyintf(p);
            if (r != r) r = 0.0f;
            if (r < -128.0f) r = -128.0f;
            if (r > 127.0f) r = 127.0f;
            x8[m * K + k] = (int8_t)r;
        }
    }
}

/* Qfunc_8bit_res without a residual codec, utils/quant.py:88-103: q = tensor / qscales (a bf16 tensor
 * operation), q.round_() (half to even), clamp_(-128, 127), .to(int8); a NaN converts to 0. */
void lqo_w8_requant(const uint16_t *latent, const uint16_t *qscales, int8_t *codes, int64_t N, int64_t K) {
    for (int64_t n = 0; n < N; ++n) {
        float c = bf16_to_f32(qscales[n]);
        for (int64_t k = 0; k < K; ++k) {
            volatile float quo = bf16_to_f32(latent[n * K + k]) / c;
            float q = bf16_round(quo);
            float r = nearbyintf(q);
            if (r != r) r = 0.0f;
            if (r < -128.0f) r = -128.0f;
            if (r > 127.0f) r = 127.0f;
            codes[n * K + k] = (int8_t)r;
        }
    }
}

/* ------------------------------------------------------- GPTQ layout ---- */
/* QuantLinearGPTQ.pack, PTQ/quant/quant_linear.py:360-372: qweight[k/8, n]
 * holds code(k, n) at bits 4*(k%8). */
void lqo_gptq_to_native(const int32_t *qweight, uint8_t *packed, int64_t N, int64_t K) {
    for (int64_t n = 0; n < N; ++n)
        for (int64_t k = 0; k < K; k += 2) {
            unsigned a = ((uint32_t)qweight[(k / 8) * N + n] >> (4 * (k % 8))) & 0xFu;
            unsigned b = ((uint32_t)qweight[((k + 1) / 8) * N + n] >> (4 * ((k + 1) % 8))) & 0xFu;
            packed[(n * K + k) / 2] = (uint8_t)((a << 4) | b);
        }
}
void lqo_native_to_gptq(const uint8_t *packed, int32_t *qweight, int64_t N, int64_t K) {
    memset(qweight, 0, sizeof(int32_t) * (size_t)(N * K / 8));
    for (int64_t n = 0; n < N; ++n)
        for (int64_t k = 0; k < K; ++k) {
            uint32_t q = code_at(packed, n * K + k);
            uint32_t *wd = (uint32_t *)&qweight[(k / 8) * N + n];
            *wd |= q << (4 * (k % 8));
        }
}

/* ------------------------------------------------- 8-bit gradient tensor -- */
/* GradientQTensor for bit = 8, utils/quant.py:856-898, on a bf16 gradient, every tensor operation
 * rounded to bf16 as torch does it (fp32 inside; x / python_scalar is x * (1.0f / scalar) in the
 * tensor library's GPU kernels):
 *   find_param :856-861  vmax = amax|dw| * 4;  scale = clamp(vmax, min=1e-5) / 127
 *   quant      :864-868  q = clamp(round(fdata / scale + noise), -128, 127)      (round half to even)
 *   dequant    :873-875  qdata.to(bf16) * scale
 *   set_value  :877-885  find_param(fdata); quant(fdata)
 *   add_       :891-898  quant(dequant() + fdata)
 * noise == NULL: noise = (2b - 255) / 512 with the element's 8-bit Philox draw b (lqo_gradq8_noise). */
void lqo_gradq8(const uint16_t *dw, int8_t *q, uint16_t *scale, int accumulate, int64_t N, int64_t K,
                const uint16_t *noise, uint64_t seed, uint64_t offset) {
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n) {
        float s;
        if (!accumulate) {
            float m = 0.0f;
            for (int64_t k = 0; k < K && m == m; ++k) {
                float a = fabsf(bf16_to_f32(dw[n * K + k]));
                if (a != a || a > m) m = a; /* data.abs().amax() returns NaN for a row that holds one */
            }
            float vmax = bf16_round(m * 4.0f);
            float lo = bf16_round(1e-5f);
            volatile float inv = 1.0f / 127.0f;
            /* torch.clamp(vmax, min = 1e-5) keeps a NaN */
            s = vmax != vmax ? vmax : bf16_round((vmax > lo ? vmax : lo) * inv);
            scale[n] = f32_to_bf16(s);
        } else {
            s = bf16_to_f32(scale[n]);
        }
        for (int64_t k = 0; k < K; ++k) {
            int64_t i = n * K + k;
            float x = bf16_to_f32(dw[i]);
            if (accumulate) x = bf16_round(bf16_round((float)q[i] * s) + x);
            float nz = noise ? bf16_to_f32(noise[i])
                             : (2.0f * (float)philox_draw8(i, seed, offset) - 255.0f) / 512.0f;
            volatile float quo = x / s;
            float y = bf16_round(bf16_round(quo) + nz);
            float r = nearbyintf(y);
            if (!(r >= -128.0f)) r = -128.0f; /* also NaN */
            if (r > 127.0f) r = 127.0f;
            q[i] = (int8_t)r;
        }
    }
}

/* ------------------------------------------------ reciprocal-based divide -- */
/* The HIP latent re-quantiser (lbit = 4) and the fused Adam kernels replace t / s by
 * q0 = t*r, e = fma(-q0, s, t), q = fma(e, r, q0) with
 * r = RN(1/s) (Markstein's correction) whenever |s| is in [2^-40, 2^40] and |t| < 2^60. This
 * routine sweeps EVERY bf16 scale in that range (both signs) against `per_scale` pseudo-random
 * numerators and counts (a) quotients that differ from IEEE t/s when |t| >= 2^-60 and (b) final
 * codes floor(clamp((q + z) + u)) that differ for any t, including tiny and zero ones. Both
 * counts must be zero for the substitution to be exact. */
static inline uint32_t xorshift32(uint32_t *st) {
    uint32_t x = *st;
    x ^= x << 13; x ^= x >> 17; x ^= x << 5;
    return *st = x;
}
void lqo_markstein_check(uint32_t seed, int per_scale, int64_t *quot_mismatch, int64_t *code_mismatch,
                         int64_t *cases) {
    int64_t qm = 0, cm = 0, n = 0;
    uint32_t st = seed ? seed : 1u;
    for (uint32_t b = 0; b < 0x10000u; ++b) {
        float s = bf16_to_f32((uint16_t)b);
        float as = fabsf(s);
        if (!(as >= 0x1p-40f && as <= 0x1p40f)) continue;
        volatile float r = 1.0f / s;
        for (int i = 0; i < per_scale; ++i) {
            uint32_t m = xorshift32(&st);
            int e = (int)(xorshift32(&st) % 180u) - 120; /* 2^-120 .. 2^59 */
            float t = ldexpf(1.0f + (float)(m >> 9) * 0x1p-23f, e);
            if (m & 1u) t = -t;
            if (i == 0) t = 0.0f;
            if (i == 1) t = 0x1p-149f;
            if (i == 2) t = -0x1p-130f;
            if (!(fabsf(t) < 0x1p60f)) continue;
            volatile float q0 = t * r;
            volatile float ee = fmaf(-q0, s, t);
            volatile float q = fmaf(ee, r, q0);
            volatile float ref = t / s;
            ++n;
            if (fabsf(t) >= 0x1p-60f) {
                uint32_t a, c;
                float qa = q, qc = ref;
                memcpy(&a, &qa, 4);
                memcpy(&c, &qc, 4);
                if (a != c) ++qm;
            }
            float z = (float)(xorshift32(&st) % 16u);
            float u = (float)(xorshift32(&st) >> 8) * 0x1p-24f;
            if (i < 3) u = 0.0f;
            volatile float v1 = q + z, v2 = ref + z;
            v1 = v1 + u;
            v2 = v2 + u;
            float f1 = floorf(v1), f2 = floorf(v2);
            unsigned c1 = (f1 != f1 || f1 < 0.0f) ? 0u : (f1 > 15.0f ? 15u : (unsigned)f1);
            unsigned c2 = (f2 != f2 || f2 < 0.0f) ? 0u : (f2 > 15.0f ? 15u : (unsigned)f2);
            if (c1 != c2) ++cm;
        }
    }
    *quot_mismatch = qm;
    *code_mismatch = cm;
    *cases = n;
}

/* ------------------------------------------------------ residual codec -- */
/* Restatement of utils/cuda_src/multi_random_quant_kernel.cu for bf16 tensors:
 * quant_kernel_bf :9-67 and launch_quant :345-362 (mode 0), quant_kernel1_bf :241-266 (mode 1),
 * dequant_kernel_bf :130-172 and launch_dequant :384-400 (mode 0), dequant_kernel1_bf :297-314
 * (mode 1). `round` is C's half-away-from-zero; the host-side random offset v0 is
 * `rand()%1000/1000`, an integer division, i.e. always 0. The reference is compiled by nvcc,
 * whose default (-fmad=true) contracts a*b+c into one FMA: fmaf is used where the source has
 * that shape. (On bf16 inputs the contracted and the uncontracted reading give the same level for
 * every input of all four curves: tests/test_oracle_pins.py sweeps them against an exact rational
 * transcription of the kernel, which is what pins this function.) A float level below -8 converts
 * to unsigned 0 (saturating conversion). */
static inline float residual_level(float x, int mode, float c1, float c2, float c3, float b1, float b2, int t1,
                                   int t2) {
    float S = fabsf(x);
    float v = fmaf(S, 499.0f, 0.0f);
    if (mode == 1) {
        v = roundf(v) - v;
        return roundf(fmaf(x, 8.0f, v));
    }
    v -= roundf(v);
    if (S < b1) return roundf(fmaf(x, c1, v));
    float r = (S < b2) ? roundf(fmaf(S - b1, c2, v)) + (float)t1 : roundf(fmaf(S - b2, c3, v)) + (float)t2;
    return x < 0.0f ? -r : r;
}

void lqo_residual_quant(uint16_t *x, uint32_t *q, int64_t n_words, int mode, int k1, float b1, int k2, float b2,
                        int k3) {
    float c1 = 0, c2 = 0, c3 = 0;
    if (mode == 0) {
        c1 = (float)k1 / b1;
        c2 = (float)k2 / (b2 - b1);
        c3 = (float)((double)k3 / (0.5 - (double)b2));
    }
    for (int64_t w = 0; w < n_words; ++w) {
        uint32_t word = 0;
        for (int k = 0; k < 8; ++k) {
            float lv = residual_level(bf16_to_f32(x[8 * w + k]), mode, c1, c2, c3, b1, b2, k1, k1 + k2);
            word <<= 4;
            if (lv > 7.5f) {
                word += 1u;
                x[8 * w + k] = 0x3F80u;
            } else {
                float t = lv + 8.0f;
                word |= (t > 0.0f) ? ((uint32_t)t & 0xFu) : 0u;
                x[8 * w + k] = 0u;
            }
        }
        q[w] = word;
    }
}

/* Deterministic uniform quantiser, utils/cuda_src/multi_random_quant_kernel.cu:219-239 (quant_kernel0): the element
 * is read into a float, level = roundf(x * 8), level > 7.5 stores nibble 1 and carry 1, otherwise nibble level + 8
 * and carry 0. x: the elements already converted to float (the conversion of the tensor's type is the caller's);
 * carry: 0 / 1 per element. */
void lqo_residual_quant_s(const float *x, uint32_t *q, uint8_t *carry, int64_t n_words) {
    for (int64_t w = 0; w < n_words; ++w) {
        uint32_t word = 0;
        for (int k = 0; k < 8; ++k) {
            float lv = roundf(x[8 * w + k] * 8.0f);
            word <<= 4;
            if (lv > 7.5f) {
                word += 1u;
                carry[8 * w + k] = 1;
            } else {
                float t = lv + 8.0f;
                word |= (t > 0.0f) ? ((uint32_t)t & 0xFu) : 0u;
                carry[8 * w + k] = 0;
            }
        }
        q[w] = word;
    }
}

void lqo_residual_dequant(const uint32_t *q, uint16_t *x, int64_t n_words, int mode, int k1, float b1, int k2,
                          float b2, int k3) {
    float ic1 = 0, ic2 = 0, ic3 = 0;
    int t1 = k1, t2 = k1 + k2;
    if (mode == 0) {
        ic1 = b1 / (float)k1;
        ic2 = (b2 - b1) / (float)k2;
        ic3 = (float)((0.5 - (double)b2) / (double)k3);
    }
    for (int64_t w = 0; w < n_words; ++w)
        for (int k = 0; k < 8; ++k) {
            int s = (int)((q[w] >> (28 - 4 * k)) & 0xFu) - 8;
            float v;
            if (mode == 1) v = (float)s * 0.125f;
            else if (s < -t2) v = fmaf((float)(s + t2), ic3, -b2);
            else if (s < -t1) v = fmaf((float)(s + t1), ic2, -b1);
            else if (s <= t1) v = (float)s * ic1;
            else if (s <= t2) v = fmaf((float)(s - t1), ic2, b1);
            else v = fmaf((float)(s - t2), ic3, b2);
            x[8 * w + k] = f32_to_bf16(v);
        }
}
