/*
 * kq_oracle.h — CPU oracle for the GGUF k-quant dequant-matmul path.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a plain-C restatement of the reference's
 * CPU algorithm (dequantise to fp32, then a strictly sequential fp32 dot
 * product).  Only the test-suite, the smoke check and the benchmark's
 * cpu_baseline leg may call it, and only as the checker or as the reported
 * CPU figure.  The shipped library never links or loads it.
 *
 * Every function cites the reference lines it follows (paths relative to the
 * reference checkout):
 *   runtime/gguf_loader.h:108-124       KQuantPacked, pack_* prototypes
 *   runtime/gguf_loader.cpp:359-379     pack_q4k
 *   runtime/gguf_loader.cpp:403-424     pack_q6k
 *   runtime/gguf_loader.cpp:428-453     kq_fp16_to_f32
 *   runtime/gguf_loader.cpp:460-496     dequant_kquant, Q4_K branch
 *   runtime/gguf_loader.cpp:537-571     dequant_kquant, Q6_K branch
 *   runtime/tests/kernel_test.cpp:1682  matvec, zero start
 *   runtime/tests/kernel_test.cpp:1728  batched matvec, bias first
 *   runtime/tests/kernel_test.cpp:62-112  Rng and truncating f32ToF16
 *   runtime/tests/kernel_test.cpp:298-317 assertClose
 *   runtime/kernels/moe/topk_softmax.wgsl:23-67
 *   runtime/kernels/moe/compute_offsets.wgsl:25-36
 *   runtime/kernels/moe/weighted_accumulate_decode.wgsl:21-29
 *   runtime/kernels/moe/weighted_add_indirect_batched.wgsl:53-70
 *   runtime/kernels/fused/silu_mul_fused.wgsl:39-49
 *
 * Pinning status (what fixes each function independently of this file):
 *   kqo_fp16_to_f32        exhaustive 65536 inputs vs the closed form and vs
 *                          the compiler's _Float16 conversion
 *   kqo_q4k_scale_min      brute force over every byte triple vs the ggml
 *                          get_scale_min_k4 definition written bit by bit
 *   kqo_dequant            fp64 closed form rounded once (Q4_K) / exact
 *                          product (Q6_K); differential vs the compiled
 *                          reference object when oracle/_ref is built
 *   kqo_pack               byte-for-byte vs the compiled reference; padding
 *                          rule vs the stated row-stride formulas
 *   kqo_matmul             x = e_k, x = 1, linearity, fp64 dot error model,
 *                          the reference's nine in-test recipes replayed
 *                          against the compiled reference
 *   kqo_moe_*              reduce to dense kqo_matmul on a row slice; brute
 *                          force on tiny expert counts.  The reference holds
 *                          no test of a Q4_K/Q6_K expert matvec: parity of
 *                          the MoE composition is unpinned beyond that.
 *   kqo_matmul_bf16        the reference has no M>=256 k-quant GEMM; the pin
 *                          is kqo_matmul on bf16-rounded inputs: parity of
 *                          the prefill GEMM is unpinned beyond that.
 */
#ifndef KQ_ORACLE_H
#define KQ_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* GGUF tensor type codes, runtime/gguf_loader.h:29-30 */
#define KQO_TYPE_Q4_K 12
#define KQO_TYPE_Q5_K 13
#define KQO_TYPE_Q6_K 14

#define KQO_QK_K 256
#define KQO_Q4K_BLOCK_BYTES 144
#define KQO_Q5K_BLOCK_BYTES 176
#define KQO_Q6K_BLOCK_BYTES 210

/* ---- scalar pieces ------------------------------------------------------ */

float kqo_fp16_to_f32(uint16_t h);
uint32_t kqo_fp16_to_f32_bits(uint16_t h);   /* same value as a bit pattern */

/* 6-bit scale and min of sub-block sb (0..7) from the 12 packed bytes. */
void kqo_q4k_scale_min(const uint8_t s[12], int sb, uint32_t *sc, uint32_t *mn);

/* ---- layout ------------------------------------------------------------- */

uint32_t kqo_block_bytes(int type);               /* 144 / 210, 0 if unknown */
uint32_t kqo_n_blocks(uint32_t K);                /* ceil(K / 256)            */
uint32_t kqo_row_stride_words(int type, uint32_t K);

/* Copy N rows of raw GGUF blocks into the padded u32 layout.  `out` holds
 * N * row_stride_words words.  Returns 0, or -1 for an unknown type. */
int kqo_pack(int type, const void *raw, uint32_t N, uint32_t K, uint32_t *out);

/* ---- dequantisation ----------------------------------------------------- */

/* raw: N rows of K/256 contiguous blocks (unpadded GGUF layout).
 * out: N*K floats.  K must be a multiple of 256. */
int kqo_dequant(int type, const void *raw, float *out, uint32_t N, uint32_t K);

/* Same arithmetic, reading one row of the padded layout. */
int kqo_dequant_packed_row(int type, const uint32_t *packed,
                           uint32_t row_stride_words, uint32_t row, uint32_t K,
                           float *out);

/* Rows picked by id (negative ids clamp to 0), the q6k_gather contract. */
int kqo_dequant_rows(int type, const uint32_t *packed, uint32_t row_stride_words,
                     const int32_t *rows, uint32_t M, uint32_t K, float *out);

/* ---- matmul ------------------------------------------------------------- */

/* Y[m*ldy + y_offset + n] = bias[n] + sum_k X[m*K+k] * deq(W)[n,k], k ascending,
 * all in fp32, the bias entering first.  bias may be NULL (sum starts at +0).
 * ldy = N when 0 is passed. */
int kqo_matmul(int type, const float *X, const uint32_t *packed, const float *bias,
               float *Y, uint32_t M, uint32_t N, uint32_t K,
               uint32_t row_stride_words, uint32_t y_offset, uint32_t ldy);

/* What the fused decode forms apply to X before the contraction
 * (pro 1: runtime/kernels/norm/rms_norm.wgsl:15-20 and
 * quant_kq/q4k_matmul_norm.wgsl:50-91, x * rstd * w with
 * rstd = 1/sqrt(sum(x^2)/K + eps), the squares summed in k order;
 * pro 2: kernels/fused/silu_mul_fused.wgsl:39-49, g/(exp(-g)+1) * u;
 * pro 3: kernels/fused/gelu_mul_fused.wgsl:22-32, the tanh form).  For pro 2/3
 * the rows of X are gate | up, 2K floats.  out: M x K.  The reference holds no
 * test of these kernels: the restatement is pinned on closed forms in fp64
 * (tests/test_oracle_pins.py), the composition with the matmul is unpinned
 * beyond that. */
int kqo_prologue(int pro, const float *X, const float *norm_w, float eps,
                 uint32_t M, uint32_t K, float *out);

/* Same contraction in fp64 with no bias rounding: the ground truth that both
 * fp32 summation orders are compared with. */
int kqo_matmul_f64(int type, const float *X, const uint32_t *packed,
                   const float *bias, double *Y, uint32_t M, uint32_t N,
                   uint32_t K, uint32_t row_stride_words);

/* X given as bf16 bit patterns; widened exactly to fp32, then kqo_matmul. */
int kqo_matmul_bf16(int type, const uint16_t *Xbf16, const uint32_t *packed,
                    const float *bias, float *Y, uint32_t M, uint32_t N,
                    uint32_t K, uint32_t row_stride_words);

/* Timed legs for the benchmark's CPU baseline: dequantise the whole matrix to
 * fp32 scratch (deq, N*K floats), then the sequential dot.  Returns seconds
 * spent in each leg through the out-parameters. */
int kqo_matmul_timed(int type, const float *X, const void *raw, float *deq,
                     float *Y, uint32_t M, uint32_t N, uint32_t K,
                     double *t_dequant, double *t_dot);

/* ---- MoE ---------------------------------------------------------------- */

/* Iterated arg-max with lowest-index tie break, soft-max over the k picked
 * values, normalised when `normalize` is non-zero. */
void kqo_moe_topk_softmax(const float *logits, uint32_t n_experts, uint32_t k,
                          int normalize, uint32_t *idx, float *wt);

/* offsets[s] = idx[s] * rows_per_expert */
void kqo_moe_offsets(const uint32_t *idx, uint32_t k, uint32_t rows_per_expert,
                     uint32_t *offsets);

/* One matvec per (token, slot) against the expert's row slice of a stacked
 * matrix [n_experts*N, K]:  Y[(t*k+s)*N + n] = sum_k X[xrow*K+k] * W[e*N+n, k]
 * with e = expert_idx[t*k+s] and xrow = t (x_per_slot == 0) or t*k+s. */
int kqo_moe_matmul(int type, const float *X, const uint32_t *packed,
                   const uint32_t *expert_idx, float *Y, uint32_t T, uint32_t k,
                   uint32_t N, uint32_t K, uint32_t row_stride_words,
                   int x_per_slot);

/* Full expert FFN for T tokens: gate/up (type_gu) -> silu(gate)*up -> down
 * (type_dn) -> out[t] = sum_s w[t,s] * down_s, slot 0 written, later slots
 * added in slot order. */
int kqo_moe_ffn(int type_gu, int type_dn, const float *X,
                const uint32_t *gate, const uint32_t *up, const uint32_t *down,
                const uint32_t *expert_idx, const float *expert_wt, float *out,
                uint32_t T, uint32_t k, uint32_t hidden, uint32_t inter);

/* ---- the reference test-suite's generators ------------------------------ */

typedef struct { uint32_t s[4]; } kqo_rng;
void     kqo_rng_seed(kqo_rng *r, uint32_t seed);
uint32_t kqo_rng_next(kqo_rng *r);
float    kqo_rng_uniform(kqo_rng *r, float lo, float hi);
float    kqo_rng_randn(kqo_rng *r);
void     kqo_rng_randn_vec(kqo_rng *r, float *out, int n);
uint16_t kqo_f32_to_f16_trunc(float f);

/* |a-e| <= atol + rtol*|e| for every element; returns the count that fail and
 * the worst excess through *worst (may be NULL). */
int kqo_assert_close(const float *actual, const float *expected, int n,
                     float atol, float rtol, float *worst);

#ifdef __cplusplus
}
#endif
#endif
