/*
 * latentq.h — C ABI of liblatentq_hip.so: the MI355X (gfx950) kernels behind the
 * quantized-linear hot path of latentQ_LLM.
 *
 * Conventions (all entry points):
 *   - every pointer is a DEVICE pointer on the current HIP device unless the
 *     parameter is documented as a host value;
 *   - the caller allocates every output; the library allocates nothing, never
 *     synchronises and is re-entrant; the only state it keeps between calls is a
 *     per-thread error text and a per-device cache of the compute-unit count
 *     (one relaxed atomic each);
 *   - work is enqueued on `stream` (a hipStream_t passed as void*; NULL = the
 *     default stream) and the call returns immediately;
 *   - return value: LQ_OK (0) on success, a negative LQ_ERR_* code otherwise;
 *     lq_last_error() returns a thread-local description of the last failure;
 *   - nothing throws across this boundary.
 *
 * Weight layout ("native" = the layout of the reference's QuantTensor.data for
 * wbit 4, reference utils/quant.py:4-19): a flat byte array of N*K/2 bytes,
 * row-major over W[N,K]; byte b of row n holds code(n, 2b) in its HIGH nibble
 * and code(n, 2b+1) in its LOW nibble. Scales and zeros are bf16 arrays of
 * N*K/group entries, entry n*(K/group) + k/group (reference utils/quant.py:
 * 66-72, 427-428). `group` must be 128 (reference GROUPSIZE, utils/quant.py:44)
 * and K a multiple of 128.
 */
#ifndef LATENTQ_H
#define LATENTQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LQ_OK 0
#define LQ_ERR_BAD_ARG (-1)   /* null pointer, bad shape, misaligned buffer */
#define LQ_ERR_LAUNCH (-2)    /* HIP reported an error when launching        */
#define LQ_ERR_UNSUPPORTED (-3)

#define LQ_GROUP 128

/* Version of this ABI; bumped on any incompatible change. */
int lq_abi_version(void);

/* Thread-local, NUL-terminated description of the last error on this thread
 * ("" if none). The pointer stays valid until the next failing call. */
const char *lq_last_error(void);

/* ---------------------------------------------------------------------------
 * (1) Stochastic-rounding latent requantizer.
 *
 * Replaces, on the latent-weight update path, the sequence
 *   DeQfunc_4bit_g -> (update) -> Qfunc_4bit_g_res -> python_compress
 * of the reference (utils/quant.py:1073, 1139-1144, 45-72), for the update
 * rule  code' = clamp(floor((deq(W) - lr*g)/s + z + u), 0, 15)  evaluated as
 *   w  = bf16_rne( bf16_rne(q - z) * s )          (reference dequant arithmetic)
 *   t  = fma(-lr, g, w)                           (fp32, one rounding)
 *   y  = fma(t, (1/s) * 65536, fma(z, 65536, 0.5))   (fp32; 1/s the IEEE quotient:
 *                                                  (t/s + z) in 16.16 fixed point, plus one half)
 *   X  = y as an unsigned 32-bit integer, truncated, saturated (NaN, negative -> 0)
 *   code' = min( min(X + a, 2^32 - 1) >> 16, 15 )
 * where a is a 16-bit uniform integer draw: the noise is u = (a + 1/2) * 2^-16, uniform on the
 * centred 2^-16 grid, and x + u is formed exactly (integer addition), so that the expected new
 * code equals x to within 2^-17 with no common drift.
 * codes_in / codes_out: N*K/2 bytes, native layout (may alias each other).
 * scales, zeros: bf16[N*K/128]. grad: bf16[N,K] row-major. lr: host float.
 * codes_in, codes_out, grad and u must be 16-byte aligned.
 * Noise: if u_or_null != NULL it is an fp32[N,K] array of uniforms and a = floor(u * 65536)
 * (only 16 fractional bits of u are used; u >= 1 counts as 65535, negative or NaN as 0);
 * otherwise a for flat element index i is the 16-bit half i & 1 (1 = the high half) of word
 * (i >> 1) & 3 of Philox4x32-10(counter = philox_offset + i/8 as a 128-bit little-endian
 * integer in the low 64 bits, key = philox_seed). One call consumes N*K/8 counters.
 * ------------------------------------------------------------------------- */
int lq_requant_sr(const void *codes_in, void *codes_out, const void *scales, const void *zeros,
                  const void *grad, float lr, int64_t N, int64_t K, int group,
                  const float *u_or_null, uint64_t philox_seed, uint64_t philox_offset,
                  void *stream);

/* Materialise the uniform stream lq_requant_sr draws from: out[i] = (a_i + 1/2) * 2^-16, i < n,
 * for the draw a_i that element i would receive; feeding out back as u_or_null reproduces the
 * Philox-mode result bit for bit. For exactness checks. */
int lq_philox_uniform(float *out, int64_t n, uint64_t philox_seed, uint64_t philox_offset,
                      void *stream);

/* ---------------------------------------------------------------------------
 * (2) A16W4 dequant-GEMM / GEMV.
 *
 * lq_a16w4_fwd replaces DeQfunc_4bit_g + input.mm(weight.t()) (+ bias) of
 * QLinearFunctionW4.forward / QLinearFunctionW4_eval.forward (reference
 * utils/quant.py:116-121, 153-158):  Y[M,N] = X[M,K] * deq(W)[N,K]^T (+ bias[N]).
 * lq_a16w4_dx replaces DeQfunc_4bit_g + grad_output.mm(weight) of
 * QLinearFunctionW4.backward (utils/quant.py:136-140): dX[M,K] = dY[M,N] * deq(W).
 * x, y, dy, dx, bias: bf16 row-major; accumulation in fp32, output rounded to
 * bf16 (round-to-nearest-even). M <= 16 takes the wavefront GEMV path.
 * The bias is added to the fp32 sum before that single rounding; the reference rounds the
 * product to bf16 first and then adds (utils/quant.py:118-120), one bf16 rounding more.
 * Requirements: K % 128 == 0; N % 16 == 0 for lq_a16w4_fwd, N % 64 == 0 for lq_a16w4_dx;
 * x, dy, codes, y, dx 16-byte aligned; scales and zeros 2-byte aligned.
 * ------------------------------------------------------------------------- */
int lq_a16w4_fwd(const void *x, const void *codes, const void *scales, const void *zeros,
                 const void *bias_or_null, void *y, int64_t M, int64_t N, int64_t K, int group,
                 void *stream);

int lq_a16w4_dx(const void *dy, const void *codes, const void *scales, const void *zeros,
                void *dx, int64_t M, int64_t N, int64_t K, int group, void *stream);

/* The same two products with a scratch buffer the library may use (it allocates nothing itself):
 * when the output has so few 128 x 128 tiles that they would occupy less than half of the device,
 * the reduction is cut into up to 8 slices, each workgroup writes an fp32 partial tile into the
 * workspace and a second kernel adds the slices in a fixed order (results are deterministic), adds
 * the bias and rounds to bf16. workspace: 16-byte aligned device memory of workspace_bytes bytes,
 * or null; M*out_columns*4 bytes per slice are used, fewer slices if the buffer is smaller. Calls
 * that share a workspace must be ordered on one stream. No counterpart in the reference (its
 * dense mm leaves this to the vendor library). */
int lq_a16w4_fwd_ws(const void *x, const void *codes, const void *scales, const void *zeros, const void *bias_or_null,
                    void *y, int64_t M, int64_t N, int64_t K, int group, void *workspace, int64_t workspace_bytes,
                    void *stream);
int lq_a16w4_dx_ws(const void *dy, const void *codes, const void *scales, const void *zeros, void *dx, int64_t M,
                   int64_t N, int64_t K, int group, void *workspace, int64_t workspace_bytes, void *stream);

/* lq_a16w4_fwd_ws with the library's own scratch instead of a caller's workspace: a static device
 * array of LQ_STATIC_SCRATCH_BYTES that is part of the code object (every device the library runs
 * on holds it until the process ends). No counterpart in the reference; it is for callers that
 * cannot allocate device memory and have none to pass: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc. Neither this call nor anything it runs allocates or frees.
 * Results equal lq_a16w4_fwd_ws called with a workspace of LQ_STATIC_SCRATCH_BYTES bytes bit for bit.
 * For M > 16 the output must satisfy 8*M*N <= LQ_STATIC_SCRATCH_BYTES (two fp32 slices), otherwise
 * LQ_ERR_BAD_ARG; M <= 16 (GEMV) uses no scratch. All calls on one device share that device's
 * array: calls that may overlap on one device (different streams, different threads) race and must
 * be ordered by the caller. Nothing in the array needs clearing between calls (every word that is
 * read was written by the same call). The first call on a device looks the array's address up
 * (hipGetSymbolAddress); make it outside graph capture. */
#define LQ_STATIC_SCRATCH_BYTES (32 << 20)
int lq_a16w4_fwd_static(const void *x, const void *codes, const void *scales, const void *zeros,
                        const void *bias_or_null, void *y, int64_t M, int64_t N, int64_t K, int group,
                        void *stream);

/* Gate / up pair of a gated MLP in one launch: h[M,N] = silu(X . deq(Wgate)^T) * (X . deq(Wup)^T) with
 * silu(v) = v / (1 + exp(-v)), both products accumulated in fp32 and the result rounded to bf16 once.
 * Replaces the fused product of the reference's GPTQ-side MLP (PTQ/quant/fused_mlp.py:85-168,
 * fusedmatmul_248_kernel: "C = silu(A * B1) * (A * B2)", called from QuantLlamaMLP.triton_llama_mlp
 * :206-218), on the native code layout. Neither product is rounded on its own, so h differs from
 * running lq_a16w4_fwd twice and multiplying in bf16 by the roundings that path adds.
 * Both matrices [N,K] with their own scales and zeros; no bias. N % 16 == 0; K % 128 == 0, and
 * K % 256 == 0 for M > 16. Up to 16 tokens run as one GEMV pass over both matrices (sums in fp32, the
 * weights not rounded to bf16 first, as in lq_a16w4_fwd for such M), more tokens through the MFMA
 * kernel of lq_a16w4_fwd. */
int lq_a16w4_gate_up_silu(const void *x, const void *codes_gate, const void *scales_gate, const void *zeros_gate,
                          const void *codes_up, const void *scales_up, const void *zeros_up, void *h, int64_t M,
                          int64_t N, int64_t K, int group, void *stream);

/* The gated MLP block in training, three entry points that take the tensor-library glue between the six
 * products of `down(silu(gate(x)) * up(x))` and its backward into the GEMM epilogues. In the reference that
 * block is transformers' LlamaMLP with its three nn.Linear replaced by QLinearA16W4 (main0.py:300-343), i.e.
 * QLinearFunctionW4.forward / backward (utils/quant.py:112-146) around bf16 silu, products and an addition
 * run by autograd; there is no counterpart function.
 *   lq_a16w4_gate_up_silu_save: lq_a16w4_gate_up_silu that also stores the two products it forms,
 *     g = X . deq(Wgate)^T and u = X . deq(Wup)^T (bf16 [M,N] each, rounded from the same fp32 sums h is formed
 *     from), which the backward pass needs. Up to 16 tokens: one GEMV pass per product plus the fused pass.
 *   lq_a16w4_dx_silu_bwd: the backward of the down projection with the backward of h = silu(g) * u as its
 *     epilogue. P = dY . deq(Wdown) [M,K] is rounded to bf16 (it is the dh autograd would hand on) and
 *       dg = bf16(P * u * s * (1 + g * (1 - s))),  du = bf16(P * g * s),  s = 1 / (1 + exp(-g))
 *     are stored instead of it (fp32 arithmetic on the bf16 values of P, g, u; one rounding each, where the
 *     tensor operations round silu(g) and P * u to bf16 in between). g, u, dg_out, du_out: bf16 [M,K].
 *   lq_a16w4_dx_acc: dx_inout = bf16(dx_inout + bf16(dY . deq(W))): the second of the two products that
 *     both flow into the block's input gradient; the same bits as lq_a16w4_dx followed by a bf16 addition.
 *   lq_a16w4_dx_pair: dx = bf16(dY1 . deq(W1) + dY2 . deq(W2)) for two layers of one shape [N,K] fed by the same
 *     input (gate and up): one launch whose reduction runs through both products, the sum kept in fp32 (one rounding
 *     where lq_a16w4_dx followed by lq_a16w4_dx_acc has two). dy1, dy2: bf16 [M,N]; dx: bf16 [M,K]; N % 64 == 0.
 * Shapes and alignment as lq_a16w4_dx / lq_a16w4_gate_up_silu; all outputs 16-byte aligned. */
int lq_a16w4_gate_up_silu_save(const void *x, const void *codes_gate, const void *scales_gate, const void *zeros_gate,
                               const void *codes_up, const void *scales_up, const void *zeros_up, void *h, void *g_out,
                               void *u_out, int64_t M, int64_t N, int64_t K, int group, void *stream);
int lq_a16w4_dx_silu_bwd(const void *dy, const void *codes, const void *scales, const void *zeros, const void *g,
                         const void *u, void *dg_out, void *du_out, int64_t M, int64_t N, int64_t K, int group,
                         void *stream);
int lq_a16w4_dx_acc(const void *dy, const void *codes, const void *scales, const void *zeros, void *dx_inout,
                    int64_t M, int64_t N, int64_t K, int group, void *stream);
int lq_a16w4_dx_pair(const void *dy1, const void *codes1, const void *scales1, const void *zeros1, const void *dy2,
                     const void *codes2, const void *scales2, const void *zeros2, void *dx, int64_t M, int64_t N,
                     int64_t K, int group, void *stream);

/* Which kernel lq_a16w4_fwd(_ws) (backward = 0) or lq_a16w4_dx(_ws) (backward = 1) would run for a
 * shape and a workspace size, and how it would cut the reduction; launches nothing. *kernel is
 * one of LQ_PLAN_*; *splits > 1 means a split reduction of *steps_per_split 64-deep steps per slice
 * followed by the reduce kernel. compute_units <= 0 asks the current device. The choice follows a
 * rough cost model of measured per-step times (see lq_gemm.hip); it is exposed so that callers and
 * tests can see it. No counterpart in the reference. */
#define LQ_PLAN_GEMV 0         /* M <= 16: one GEMV launch */
#define LQ_PLAN_GEMV_CHUNKS 1  /* 17..128 tokens: GEMV launches of 16 tokens each */
#define LQ_PLAN_DIRECT 2       /* weights-direct forward kernel, 128 x 256 tiles */
#define LQ_PLAN_STAGED_128 3   /* staged kernel, 128 x 128 tiles */
#define LQ_PLAN_STAGED_256 4   /* staged kernel, 256 x 128 tiles */
#define LQ_PLAN_DIRECT_128 5   /* weights-direct forward kernel, 128 x 128 tiles */
int lq_a16w4_plan(int backward, int64_t M, int64_t N, int64_t K, int64_t workspace_bytes, int compute_units,
                  int *kernel, int *splits, int *steps_per_split);

/* Dequantise the whole matrix to bf16[N,K] with the reference arithmetic
 * (DeQfunc_4bit_g, utils/quant.py:66-72). Used for the dW-side consumers and
 * for checks; not on the forward/backward GEMM path. */
int lq_a16w4_dequant(const void *codes, const void *scales, const void *zeros, void *w_out,
                     int64_t N, int64_t K, int group, void *stream);

/* ---------------------------------------------------------------------------
 * (3) A8W8 int8 GEMM with fused scale epilogue.
 *
 * Replaces torch_int._CUDA.linear_a8_w8_bbf16_obf16 and the trailing
 * `* qscales.view(1,-1)` (reference utils/quant.py:268-271 and its siblings):
 *   acc[m,n] = sum_k x[m,k] * w[n,k]                    (exact int32)
 *   y[m,n]   = bf16_rne( (float(acc) * sx[m]) * sw[n] + bias[n] )
 * x: int8[M,K], w: int8[N,K] row-major; sx: fp32[M]; sw: fp32[N];
 * bias_or_null: bf16[N]; y: bf16[M,N]; acc_or_null: int32[M,N] (written when
 * non-NULL, for the bit-exact accumulator check). K % 128 == 0, N % 16 == 0;
 * x, w, y, acc 16-byte aligned, sx and sw 4-byte aligned.
 * ------------------------------------------------------------------------- */
int lq_a8w8_fwd(const void *x, const void *w, const float *sx, const float *sw,
                const void *bias_or_null, void *y, int32_t *acc_or_null, int64_t M, int64_t N,
                int64_t K, void *stream);

/* lq_a8w8_fwd with the per-channel scales as the reference's modules store them: qscales is the bf16[N]
 * buffer `qscales` of QLinearA8W8 / QLinearQAT (utils/quant.py:496-498), read and widened in the epilogue
 * (sw[n] = float(qscales[n]), exact), so that a layer's forward needs no conversion pass. */
int lq_a8w8_fwd_qs(const void *x, const void *w, const float *sx, const void *qscales_bf16,
                   const void *bias_or_null, void *y, int32_t *acc_or_null, int64_t M, int64_t N,
                   int64_t K, void *stream);

/* Input gradient of an 8-bit-weight layer from its int8 codes: dX[M,K] = dY[M,N] . Wf[N,K] with
 * Wf[n,k] = bf16(w[n,k] * qscales[n]), the dequantised weight the reference's backward materialises
 * (`weight_d.to(dtype) * qscales`, utils/quant.py:200-206, 239-245, 281-288) and multiplies with
 * `grad_output.mm(weight_forward)`; here it is formed tile by tile inside the GEMM and never stored.
 * dy: bf16 [M,N]; w: int8 [N,K]; qscales_bf16: bf16 [N]; dx: bf16 [M,K]; N % 64 == 0, K % 128 == 0; dy, w, dx
 * 16-byte aligned. fp32 accumulation, one bf16 rounding of the result. */
int lq_a8w8_dx(const void *dy, const void *w, const void *qscales_bf16, void *dx, int64_t M, int64_t N, int64_t K,
               void *stream);

/* Per-tensor symmetric activation quantizer used in front of lq_a8w8_fwd:
 *   x8 = clamp(round_half_even(x * (127/clampv)), -128, 127)
 * (reference utils/quant.py:264-266). x: bf16[n]; clampv: DEVICE fp32 scalar;
 * x8: int8[n]. */
int lq_act_quant_i8(const void *x, const float *clampv_dev, int8_t *x8, int64_t n, void *stream);

/* The same quantiser with the clamp value the dynamic layers of the reference use, the maximum of the
 * activation tensor itself (`clampv = input.max()`, utils/quant.py:259-266, 319-322), found on the device:
 * two launches, no host synchronisation and no other kernel. A NaN anywhere in x makes the clamp value NaN
 * (as the tensor library's max does) and every x8 zero.
 *   clampv = max_i x[i];  x8 as lq_act_quant_i8 with that value;
 *   sx[m]  = alpha for every m < M, alpha = clampv * fl32(1/127) (how the tensor library divides a tensor by
 *            the host scalar 127.), rounded to bf16 when alpha_bf16 != 0 (the training Function divides a bf16
 *            0-dim tensor, :271; the eval Function a host float, :326): the per-row scales lq_a8w8_fwd reads.
 * x: bf16[M,K], 16-byte aligned; x8: int8[M,K], 8-byte aligned; sx: fp32[M];
 * work: fp32[LQ_ACT_WORK_FLOATS] device scratch; on return work[0] = clampv and work[1] = alpha (device values). */
#define LQ_ACT_WORK_FLOATS 1032
int lq_act_quant_i8_dynamic(const void *x, int8_t *x8, float *sx, float *work, int64_t M, int64_t K, int alpha_bf16,
                            void *stream);

/* Per-token activation quantiser, one pass: for every token row m
 *   amax  = max_k |x[m,k]|                         (NaN if the row holds one)
 *   sx[m] = amax / 127                             (fp32, IEEE division)
 *   x8[m,k] = clamp(round_half_even(x[m,k] * (127 / amax)), -128, 127)   (fp32; NaN -> 0; an all-zero row: 0)
 * so that lq_a8w8_fwd's epilogue (acc * sx[m]) * sw[n] is the per-token x per-channel scaling. The reference
 * quantises per tensor only (utils/quant.py:259-266); this is the per-token form of the same step.
 * x: bf16[M,K], 16-byte aligned, K % 8 == 0; x8: int8[M,K]; sx: fp32[M]. */
int lq_act_quant_i8_per_token(const void *x, int8_t *x8, float *sx, int64_t M, int64_t K, void *stream);

/* The quantised activations back as bf16 for the backward pass: out[m,k] = bf16(x8[m,k] * bf16(s)), s = scale[m]
 * (per_token != 0) or scale[0]: the values of `x8.to(dtype) * scale.to(dtype)` that the training Function's backward
 * multiplies dY^T with (utils/quant.py:277-280) as one pass instead of two tensor operations. x8: int8 [M,K], 16-byte
 * aligned, K % 16 == 0; scale: fp32 [M] or [1]; out: bf16 [M,K], 16-byte aligned. */
int lq_act_dequant_i8(const int8_t *x8, const float *scale, int per_token, void *out, int64_t M, int64_t K, void *stream);

/* Fake quantisation of the activations for the backward pass of the Functions that save the bf16 input
 * (QLinearFunctionA8W8_static.backward, QLinearFunctionQAT_dynamic.backward: utils/quant.py:197-199, 358-360):
 * out = bf16(clamp(rne(bf16(x * s)), -128, 127) / s), the chain (input * s).round_().clamp_(-128, 127).div_(s) with
 * its bf16 roundings as one pass. x, out: bf16[n], 16-byte aligned; s: one bf16 number on the device (127 / clampv). */
int lq_act_fake_quant(const void *x, const void *s_bf16_dev, void *out, int64_t n, void *stream);

/* Per-channel int8 re-quantiser of the latent weight of an 8-bit-weight layer: the reference's
 * Qfunc_8bit_res (utils/quant.py:88-103) for a latent kept as a plain tensor (lbit 0, 16, 32), called
 * from MyAdam.update_step (:1141):
 *   codes[n,k] = clamp(round_half_even(bf16(latent[n,k] / qscales[n])), -128, 127)      NaN -> 0
 * latent: bf16[N,K], 16-byte aligned; qscales: bf16[N]; codes: int8[N,K], 8-byte aligned; K % 8 == 0.
 * (With a 4-bit residual codec, lbit = 4: lq_latent_w8_requant.) */
int lq_w8_requant(const void *latent, const void *qscales, int8_t *codes, int64_t N, int64_t K, void *stream);

/* ---------------------------------------------------------------------------
 * 4-bit residual codec of the latent weight (exact lbit = 4 mode).
 *
 * Replaces the MyQuantDequant extension of the reference: pybind names
 * `quant` / `dequant` (utils/cuda_src/multi_random_quant.cpp:13-21,
 * kernels multi_random_quant_kernel.cu:9-67, 130-172) for mode 0 and
 * `uniform_quant` / `uniform_dequant` (multi_random_quant.cpp:23-31, kernels
 * :241-266, :297-314) for mode 1; called from cuda_quant_3fold /
 * cuda_dequant_3fold / cuda_quant_linear / cuda_dequant_linear
 * (utils/quant.py:723-763). Argument meaning as in the reference:
 * (k1, b1, k2, b2, k3) are the level counts and breakpoints of the three
 * companding segments (ignored in mode 1).
 * x_inout / x_out: bf16[8 * n_words]; q: int32[n_words], element k of a word in
 * bits 28-4k. lq_residual_quant OVERWRITES x with the carry flags (bf16 1.0
 * where the level rounded up past 7, else 0.0), as the reference does.
 * ------------------------------------------------------------------------- */
int lq_residual_quant(void *x_inout, int32_t *q_out, int64_t n_words, int mode, int k1, float b1, int k2,
                      float b2, int k3, void *stream);
int lq_residual_dequant(const int32_t *q, void *x_out, int64_t n_words, int mode, int k1, float b1, int k2,
                        float b2, int k3, void *stream);

/* The reference's deterministic uniform quantiser, pybind name `uniform_quant_s`
 * (utils/cuda_src/multi_random_quant.cpp:33-36, 48-50; kernel quant_kernel0,
 * multi_random_quant_kernel.cu:219-239; launcher :376-381): level = roundf(float(x) * 8) with halves
 * away from zero and no dither, nibble and carry as in lq_residual_quant, carries written back over
 * x in x's own type. The reference dispatches it for fp32, fp16 and fp64 tensors (dtype 0, 1, 2; a
 * double is converted to float first, as its kernel does); dtype 3 = bf16 is an addition. Nothing in the
 * reference calls it. x_inout: 8 * n_words elements of that type, 16-byte aligned. Levels below -8
 * (|x| > 1, undefined in the reference) store nibble 0. */
int lq_residual_quant_s(void *x_inout, int32_t *q_out, int64_t n_words, int dtype, void *stream);

/* ---------------------------------------------------------------------------
 * Fused latent-weight passes of the A16W4 layer in its 4-bit-residual mode (lbit = 4), three-segment
 * codec with the parameters of lq_residual_quant. Each is one pass instead of a chain of bf16
 * tensor operations around the codec kernel, with the chain's rounding points kept (bit-identical).
 *   lq_latent_w4_reconstruct: latent = bf16(bf16(value(nibble) * s) + bf16(bf16(q - z) * s))
 *     replaces ResidualTensor.add(DeQfunc_4bit_g(...)), utils/quant.py:66-72, 826-837, 1066-1079.
 *   lq_latent_w4_requant: Z = bf16(bf16(t / s) + z), q = rint(Z), residual nibble and carry from
 *     bf16(Z - q), code = clamp(q + carry, 0, 15); replaces Qfunc_4bit_g_res + ResidualTensor.set_value,
 *     utils/quant.py:45-63, 803-811.
 * codes: native layout; residual: int32[N*K/8], first element in the top nibble; latent: bf16[N,K];
 * all three 16-byte aligned. A NaN in the latent gives code 0 (the tensor-op chain leaves it undefined).
 * ------------------------------------------------------------------------- */
int lq_latent_w4_reconstruct(const void *codes, const void *scales, const void *zeros, const int32_t *residual,
                             void *latent_out, int64_t N, int64_t K, int group, int k1, float b1, int k2, float b2,
                             int k3, void *stream);
int lq_latent_w4_requant(const void *latent, const void *scales, const void *zeros, void *codes_out,
                         int32_t *residual_out, int64_t N, int64_t K, int group, int k1, float b1, int k2, float b2,
                         int k3, void *stream);

/* The same two passes for an 8-bit-weight layer whose latent is codes + 4-bit residual (QuantTensor(wbit = 8,
 * lbit = 4)): one bf16 scale per weight row instead of scale and zero per group.
 *   lq_latent_w8_reconstruct: latent = bf16(bf16(value(nibble) * s[n]) + bf16(q * s[n]))
 *     replaces ResidualTensor.add((p.data * p.qparam).to(dtype)), utils/quant.py:826-837, 1069-1070.
 *   lq_latent_w8_requant: Z = bf16(t / s[n]), q = rint(Z), residual nibble and carry from bf16(Z - q),
 *     code = clamp(q + carry, -128, 127); replaces Qfunc_8bit_res with a ResidualTensor, utils/quant.py:88-103
 *     (+ ResidualTensor.set_value :803-811). NaN -> code 0.
 * codes: int8 [N,K]; qscales: bf16 [N]; residual: int32 [N*K/8]; latent: bf16 [N,K]; K % 16 == 0; codes and latent
 * 16-byte, residual 8-byte aligned. */
int lq_latent_w8_reconstruct(const int8_t *codes, const void *qscales, const int32_t *residual, void *latent_out,
                             int64_t N, int64_t K, int k1, float b1, int k2, float b2, int k3, void *stream);
int lq_latent_w8_requant(const void *latent, const void *qscales, int8_t *codes_out, int32_t *residual_out, int64_t N,
                         int64_t K, int k1, float b1, int k2, float b2, int k3, void *stream);

/* ---------------------------------------------------------------------------
 * One Adam step on 8-bit block-wise moments, the chain of tensor operations of
 * MyAdam.update_step (reference utils/quant.py:1081-1134) with Qfunc_8bit_opt /
 * DeQfunc_8bit_opt (:22-41) as a single pass with the chain's rounding points kept:
 *   m = bf16(max1 - q1*scale1), v = bf16((max2 - q2*scale2)^2),
 *   m = bf16(bf16(m*beta1) + (1-beta1)*g), v = bf16(bf16(v*beta2) + (1-beta2)*g*g),
 *   d = bf16(bf16(sqrt(v)) + eps), param = bf16(param - step_size*(m/d))   (or direction = bf16(m/d)),
 *   then m and d re-quantised per block: max = max(x), scale = (max - min(x))/255 + 1e-10,
 *   q = clamp(rint((max - x)/scale), 0, 255).
 * grad, param, direction: bf16[n], 16-byte aligned; exactly one of param (updated in place) and
 * direction (written) is non-null. state1/state2: uint8[n], 8-byte aligned, updated in place;
 * scale1/max1/scale2/max2: fp32[n/block_elems], updated in place (the reference's qmap1/absmax1/
 * qmap2/absmax2). block_elems is 2048 or 128 and divides n. Weight decay and the periodic
 * update of the residual codec's range are not part of this call.
 * ------------------------------------------------------------------------- */
int lq_adam8_update(const void *grad, void *param_or_null, void *direction_or_null, uint8_t *state1, uint8_t *state2,
                    float *scale1, float *max1, float *scale2, float *max2, int64_t n, int block_elems, double beta1,
                    double beta2, double eps, double step_size, void *stream);

/* The same step for an A16W4 layer in its exact 4-bit-residual mode (lbit = 4), with the two passes
 * around it folded in: the parameter is rebuilt from codes and residual words exactly as
 * lq_latent_w4_reconstruct does (curve dk1..dk3: the one the residual was stored with), updated,
 * and re-quantised exactly as lq_latent_w4_requant does (curve qk1..qk3: the current one). One call
 * replaces ResidualTensor.add(DeQfunc_4bit_g(...)), the Adam chain and Qfunc_4bit_g_res of
 * MyAdam.update_step (utils/quant.py:1066-1144). codes (native layout, N*K/2 bytes) and residual
 * (int32[N*K/8]) are updated in place and need 4-byte alignment; the rest as lq_adam8_update
 * with n = N*K.
 */
int lq_adam8_latent_w4_step(const void *grad, void *codes, int32_t *residual, const void *scales, const void *zeros,
                            uint8_t *state1, uint8_t *state2, float *scale1, float *max1, float *scale2, float *max2,
                            int64_t N, int64_t K, int group, int block_elems, int dk1, float db1, int dk2, float db2,
                            int dk3, int qk1, float qb1, int qk2, float qb2, int qk3, double beta1, double beta2,
                            double eps, double step_size, void *stream);

/* The same for an 8-bit-weight layer (QLinearA8W8 with lbit = 4): the parameter is rebuilt from the int8 codes, the
 * per-row bf16 scales and the residual words exactly as lq_latent_w8_reconstruct does
 * (ResidualTensor.add((p.data * p.qparam).to(dtype)), utils/quant.py:826-837, 1069-1070), updated, and re-quantised
 * exactly as lq_latent_w8_requant does (Qfunc_8bit_res, utils/quant.py:88-103). codes: int8 [N, K], 8-byte aligned,
 * K % 8 == 0; qscales: bf16 [N]; residual: int32 [N*K/8]; the rest as lq_adam8_latent_w4_step with n = N*K. */
int lq_adam8_latent_w8_step(const void *grad, int8_t *codes, int32_t *residual, const void *qscales, uint8_t *state1,
                            uint8_t *state2, float *scale1, float *max1, float *scale2, float *max2, int64_t N, int64_t K,
                            int block_elems, int dk1, float db1, int dk2, float db2, int dk3, int qk1, float qb1, int qk2,
                            float qb2, int qk3, double beta1, double beta2, double eps, double step_size, void *stream);

/* ---------------------------------------------------------------------------
 * 8-bit gradient accumulator: GradientQTensor.find_param / quant / dequant / set_value / add_ of
 * the reference (utils/quant.py:856-898) for bit = 8 as one pass over the bf16 weight gradient,
 * with the bf16 rounding of every tensor operation of that chain kept.
 *   accumulate == 0 (set_value):  scale[n] = bf16(max(bf16(4 * max_k |dw[n,k]|), bf16(1e-5)) * (1/127))
 *                                 is computed and written; x = dw
 *   accumulate != 0 (add_):       scale[n] is read; x = bf16(bf16(q * scale[n]) + dw)
 *   q[n,k] = clamp(rint(bf16(bf16(x / scale[n]) + noise[n,k])), -128, 127)        (written in place)
 * dw: bf16[N,K]; q_inout: int8[N,K]; scale_inout: bf16[N]; K % 16 == 0; dw, q and noise 16-byte
 * aligned. Noise: noise_or_null is a bf16[N,K] array (the reference draws it with
 * uniform_(-0.5, 0.5)), otherwise noise = (2b - 255) / 512 with the 8-bit Philox draw b of flat element
 * i = n*K + k: byte i & 3 of word (i >> 2) & 3 of Philox4x32-10(counter = philox_offset + i / 16,
 * key = philox_seed); a call consumes N*K/16 counters.
 * ------------------------------------------------------------------------- */
int lq_gradq8_quant(const void *dw, int8_t *q_inout, void *scale_inout, int accumulate, int64_t N, int64_t K,
                    const void *noise_or_null, uint64_t philox_seed, uint64_t philox_offset, void *stream);

/* ---------------------------------------------------------------------------
 * Weight gradient of a quantised linear layer, dW[N,K] = dY[M,N]^T . X[M,K] (bf16, fp32 accumulation):
 * `grad_output.t().mm(input)` of QLinearFunctionW4.backward and its A8W8 / QAT siblings (reference
 * utils/quant.py:141-142, 207, 248, 289, 370). Both operands are read as they lie in memory (no transposed
 * copy). dy: bf16 [M,N]; x: bf16 [M,K]; M % 64 == 0, N % 8 == 0; dy, x and the output 16-byte aligned.
 *   lq_weight_grad:      dw_out = bf16(dW), bf16 [N,K], K % 8 == 0.
 *   lq_weight_grad_acc:  dw_inout = bf16(dw_inout + bf16(dW)): the `module.weight.grad.add_(dW)` of backward_hook_fn
 *     (utils/quant.py:398-411) on every micro-batch after the first when the gradient is kept in bf16 (gbit = 16),
 *     as the GEMM's epilogue; the same bits as lq_weight_grad followed by a bf16 tensor addition.
 *   lq_weight_grad_acc8: the product with the add_ form of the 8-bit gradient accumulator as its epilogue
 *     (GradientQTensor.add_, utils/quant.py:891-898, reached from backward_hook_fn :398-411 on every
 *     micro-batch after the first): with d = bf16(dW),
 *       x = bf16(bf16(q * scale[n]) + d),  q[n,k] = clamp(rint(bf16(bf16(x / scale[n]) + noise[n,k])), -128, 127)
 *     in place; exactly lq_weight_grad followed by lq_gradq8_quant(accumulate = 1) with the same noise
 *     arguments, without dW ever being stored. q_inout: int8 [N,K]; scale: bf16 [N] (read); K % 16 == 0.
 * ------------------------------------------------------------------------- */
int lq_weight_grad(const void *dy, const void *x, void *dw_out, int64_t M, int64_t N, int64_t K, void *stream);
int lq_weight_grad_acc(const void *dy, const void *x, void *dw_inout, int64_t M, int64_t N, int64_t K, void *stream);
int lq_weight_grad_acc8(const void *dy, const void *x, int8_t *q_inout, const void *scale, int64_t M, int64_t N,
                        int64_t K, const void *noise_or_null, uint64_t philox_seed, uint64_t philox_offset,
                        void *stream);

/* ---------------------------------------------------------------------------
 * Layout converters (device side).
 * GPTQ layout (reference PTQ/quant/quant_linear.py:343-389): qweight is
 * int32[K/8, N] with code(k, n) at bits 4*(k%8) of word [k/8, n].
 * ------------------------------------------------------------------------- */
int lq_repack_gptq_to_native(const int32_t *qweight_gptq, void *codes_native, int64_t N, int64_t K,
                             void *stream);
int lq_repack_native_to_gptq(const void *codes_native, int32_t *qweight_gptq, int64_t N, int64_t K,
                             void *stream);

/* ---------------------------------------------------------------------------
 * dst[c][r] = src[r][c] for a row-major bf16 [R, C] matrix (R, C multiples of 8, both buffers
 * 16-byte aligned, not overlapping). Used for the weight gradient dW = dY^T X of
 * QLinearFunctionW4.backward (reference utils/quant.py:141-142, `grad_output.t().mm(input)`): the
 * dense GEMM runs faster on a transposed copy of dY than on the strided view.
 * ------------------------------------------------------------------------- */
int lq_transpose_bf16(const void *src, void *dst, int64_t R, int64_t C, void *stream);

/* ---------------------------------------------------------------------------
 * Measurement aid, no counterpart in the reference: a plain streaming copy of
 * nbytes (a multiple of 16, both pointers 16-byte aligned) from src to dst.
 * Its known traffic (nbytes read + nbytes written) calibrates the HBM byte
 * counters of a profiler run and gives the copy bandwidth this device sustains.
 * ------------------------------------------------------------------------- */
int lq_calib_copy(const void *src, void *dst, int64_t nbytes, void *stream);

/* Measurement aid, no counterpart in the reference: a plain streaming READ of nbytes (a multiple of 16, src
 * 16-byte aligned) with 16-byte loads and nothing written (sink: 64 words of device memory that receive at most
 * a checksum word). workgroups <= 0: one thread per 16 bytes (every load of the grid in flight at once, the
 * shape of the GEMV's weight loads); otherwise that many workgroups of 256 threads, grid-stride. The time of
 * this launch is what reading that many bytes costs on this device, the floor under a bandwidth-bound kernel
 * that reads them. */
int lq_calib_read(const void *src, int64_t nbytes, int workgroups, void *sink, void *stream);

/* Measurement aids for the GEMM's ceiling, no counterpart in the reference.
 * lq_calib_mfma_loop: nothing but matrix instructions in the forward GEMM's shape: workgroups of 4
 * waves (workgroups_per_cu = 1 or 2 per compute unit), each wave 8 accumulator tiles of 32 x 32 and the
 * 8 MFMAs (32x32x16 bf16) of one reduction slice per iteration, operand fragments loaded once from
 * a and b (bf16, n_elems each: zeros and random data draw different power). Every wave writes the
 * shader-cycle counter at the start and end of its loop and the 100 MHz real-time counter at the same
 * two points to clocks[4 w .. 4 w + 3] and a checksum to sink[w]; *waves receives the wave count
 * (4 x workgroups). Work per wave: iters x 8 x 32768 flop.
 * lq_calib_gemm_clocks: one lq_a16w4_fwd (backward = 0, bias-free) or lq_a16w4_dx (backward = 1)
 * launch, M > 16, without workspace, in which every workgroup writes the same four counters at its
 * start and end to clocks[4 g .. 4 g + 3]; *workgroups receives their number. Shader clock granted
 * to a workgroup = (cycles end - start) / (real time end - start) x 100 MHz.
 * ------------------------------------------------------------------------- */
int lq_calib_mfma_loop(const void *a, const void *b, int64_t n_elems, int64_t iters, int workgroups_per_cu,
                       uint64_t *clocks, int64_t clocks_capacity, float *sink, int64_t *waves, void *stream);
/* lq_calib_mfma_loop on the int8 matrix instruction of lq_a8w8_fwd (32x32x32, int32 accumulators): a and b are
 * n_bytes of int8 each; work per wave: iters x 8 x 65536 operations; sink: int32[waves]. */
int lq_calib_mfma_loop_i8(const void *a, const void *b, int64_t n_bytes, int64_t iters, int workgroups_per_cu,
                          uint64_t *clocks, int64_t clocks_capacity, int32_t *sink, int64_t *waves, void *stream);
int lq_calib_gemm_clocks(int backward, const void *a, const void *codes, const void *scales, const void *zeros,
                         void *out, int64_t M, int64_t N, int64_t K, int group, uint64_t *clocks,
                         int64_t clocks_capacity, int64_t *workgroups, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* LATENTQ_H */
