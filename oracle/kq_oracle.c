/*
 * kq_oracle.c — CPU oracle for the GGUF k-quant dequant-matmul path.
 *
 * TEST INFRASTRUCTURE ONLY: see kq_oracle.h for who may call this and for the
 * pinning status of every function.  Build with -O2 -ffp-contract=off so the
 * sequential fp32 sums are evaluated exactly as written.
 */
#include "kq_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

/* ------------------------------------------------------------------------ */
/* fp16 -> fp32, runtime/gguf_loader.cpp:428-453.                           */
/* Value: (-1)^s * 2^(e-15) * (1 + m/1024) for 0<e<31; subnormals m * 2^-24;  */
/* e == 31 maps to inf / NaN with the payload shifted up 13 bits.            */
/* ------------------------------------------------------------------------ */
uint32_t kqo_fp16_to_f32_bits(uint16_t h)
{
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = ((uint32_t)h >> 10) & 31u;
    uint32_t m = (uint32_t)h & 1023u;
    uint32_t bits;

    if (e == 31u) {
        bits = sign | 0x7F800000u | (m << 13);
    } else if (e != 0u) {
        bits = sign | ((e + 112u) << 23) | (m << 13);
    } else if (m == 0u) {
        bits = sign;
    } else {
        /* normalise the subnormal: shift until the hidden bit appears */
        int shift = 0;
        while (!(m & 1024u)) { m <<= 1; ++shift; }
        bits = sign | ((uint32_t)(113 - shift) << 23) | ((m & 1023u) << 13);
    }
    return bits;
}

float kqo_fp16_to_f32(uint16_t h)
{
    const uint32_t bits = kqo_fp16_to_f32_bits(h);
    float f;
    memcpy(&f, &bits, sizeof f);
    return f;
}

/* ------------------------------------------------------------------------ */
/* Q4_K 6-bit scale / min, runtime/gguf_loader.cpp:474-481.                  */
/* Bytes 0..3 carry sc0..3 in their low 6 bits, bytes 4..7 carry mn0..3;     */
/* bytes 8..11 carry the low nibbles of sc4..7 (low half) and mn4..7 (high   */
/* half), whose top two bits sit in bits 6..7 of bytes 0..3 and 4..7.        */
/* ------------------------------------------------------------------------ */
void kqo_q4k_scale_min(const uint8_t s[12], int sb, uint32_t *sc, uint32_t *mn)
{
    if (sb < 4) {
        *sc = s[sb] & 63u;
        *mn = s[sb + 4] & 63u;
    } else {
        const int j = sb - 4;
        *sc = (s[8 + j] & 15u) | (((uint32_t)s[j] >> 6) << 4);
        *mn = ((uint32_t)s[8 + j] >> 4) | (((uint32_t)s[4 + j] >> 6) << 4);
    }
}

/* ------------------------------------------------------------------------ */
/* layout, runtime/gguf_loader.cpp:359-379 and :403-424                      */
/* ------------------------------------------------------------------------ */
uint32_t kqo_block_bytes(int type)
{
    if (type == KQO_TYPE_Q4_K) return KQO_Q4K_BLOCK_BYTES;
    if (type == KQO_TYPE_Q5_K) return KQO_Q5K_BLOCK_BYTES;   /* pack_q5k, runtime/gguf_loader.cpp:381-401 */
    if (type == KQO_TYPE_Q6_K) return KQO_Q6K_BLOCK_BYTES;
    return 0;
}

uint32_t kqo_n_blocks(uint32_t K) { return (K + KQO_QK_K - 1) / KQO_QK_K; }

uint32_t kqo_row_stride_words(int type, uint32_t K)
{
    const uint32_t bb = kqo_block_bytes(type);
    if (!bb) return 0;
    /* Q4_K rows are a whole number of words already; Q6_K rows are rounded up */
    return (kqo_n_blocks(K) * bb + 3u) / 4u;
}

int kqo_pack(int type, const void *raw, uint32_t N, uint32_t K, uint32_t *out)
{
    const uint32_t bb = kqo_block_bytes(type);
    if (!bb) return -1;
    const size_t row_bytes = (size_t)kqo_n_blocks(K) * bb;
    const size_t stride = (size_t)kqo_row_stride_words(type, K) * 4u;
    const uint8_t *src = (const uint8_t *)raw;
    uint8_t *dst = (uint8_t *)out;
    for (uint32_t n = 0; n < N; ++n) {
        memcpy(dst + n * stride, src + n * row_bytes, row_bytes);
        if (stride > row_bytes)
            memset(dst + n * stride + row_bytes, 0, stride - row_bytes);
    }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* one superblock -> 256 floats                                              */
/* ------------------------------------------------------------------------ */

/* runtime/gguf_loader.cpp:460-496.  out = (d*sc)*q - (dmin*mn), each product
 * rounded to fp32 in that order. */
static void q4k_block(const uint8_t *blk, float *out)
{
    uint16_t hd, hm;
    memcpy(&hd, blk, 2);
    memcpy(&hm, blk + 2, 2);
    const float d = kqo_fp16_to_f32(hd);
    const float dmin = kqo_fp16_to_f32(hm);
    const uint8_t *scales = blk + 4;
    const uint8_t *qs = blk + 16;

    for (int sb = 0; sb < 8; ++sb) {
        uint32_t sc_u, mn_u;
        kqo_q4k_scale_min(scales, sb, &sc_u, &mn_u);
        const float sc = d * (float)sc_u;
        const float mn = dmin * (float)mn_u;
        const uint8_t *q = qs + (sb >> 1) * 32;
        const int shift = (sb & 1) * 4;
        for (int i = 0; i < 32; ++i) {
            const uint32_t nib = ((uint32_t)q[i] >> shift) & 15u;
            out[sb * 32 + i] = sc * (float)nib - mn;
        }
    }
}

/* runtime/gguf_loader.cpp:497-536.  d, dmin fp16 @0, 2; 12 scale bytes @4 (the Q4_K packing); 32
 * bytes of fifth bits @16 (bit sb of byte i belongs to element i of sub-block sb); 128 nibble bytes
 * @48.  out = (d*sc)*(nibble | bit<<4) - (dmin*mn), each product rounded to fp32 in that order. */
static void q5k_block(const uint8_t *blk, float *out)
{
    uint16_t hd, hm;
    memcpy(&hd, blk, 2);
    memcpy(&hm, blk + 2, 2);
    const float d = kqo_fp16_to_f32(hd);
    const float dmin = kqo_fp16_to_f32(hm);
    const uint8_t *scales = blk + 4;
    const uint8_t *qh = blk + 16;
    const uint8_t *qs = blk + 48;

    for (int sb = 0; sb < 8; ++sb) {
        uint32_t sc_u, mn_u;
        kqo_q4k_scale_min(scales, sb, &sc_u, &mn_u);
        const float sc = d * (float)sc_u;
        const float mn = dmin * (float)mn_u;
        const uint8_t *q = qs + (sb >> 1) * 32;
        const int shift = (sb & 1) * 4;
        for (int i = 0; i < 32; ++i) {
            const uint32_t nib = ((uint32_t)q[i] >> shift) & 15u;
            const uint32_t hi = ((uint32_t)qh[i] >> sb) & 1u;
            out[sb * 32 + i] = sc * (float)(nib | (hi << 4)) - mn;
        }
    }
}

/* runtime/gguf_loader.cpp:537-571.  out = d * (float)scale * (float)(q-32),
 * evaluated left to right. */
static void q6k_block(const uint8_t *blk, float *out)
{
    uint16_t hd;
    memcpy(&hd, blk + 208, 2);
    const float d = kqo_fp16_to_f32(hd);

    for (int half = 0; half < 2; ++half) {
        const uint8_t *ql = blk + 64 * half;
        const uint8_t *qh = blk + 128 + 32 * half;
        const int8_t *sc = (const int8_t *)(blk + 192 + 8 * half);
        float *o = out + 128 * half;
        for (int l = 0; l < 32; ++l) {
            const int is = l >> 4;
            const uint32_t h = qh[l];
            const int q0 = (int)((ql[l] & 15u)      | (((h >> 0) & 3u) << 4)) - 32;
            const int q1 = (int)((ql[l + 32] & 15u) | (((h >> 2) & 3u) << 4)) - 32;
            const int q2 = (int)((uint32_t)(ql[l] >> 4)      | (((h >> 4) & 3u) << 4)) - 32;
            const int q3 = (int)((uint32_t)(ql[l + 32] >> 4) | (((h >> 6) & 3u) << 4)) - 32;
            o[l]      = d * (float)sc[is]     * (float)q0;
            o[l + 32] = d * (float)sc[is + 2] * (float)q1;
            o[l + 64] = d * (float)sc[is + 4] * (float)q2;
            o[l + 96] = d * (float)sc[is + 6] * (float)q3;
        }
    }
}

static void dequant_row_bytes(int type, const uint8_t *row, uint32_t nb, float *out)
{
    if (type == KQO_TYPE_Q4_K) {
        for (uint32_t b = 0; b < nb; ++b)
            q4k_block(row + (size_t)b * KQO_Q4K_BLOCK_BYTES, out + (size_t)b * KQO_QK_K);
    } else if (type == KQO_TYPE_Q5_K) {
        for (uint32_t b = 0; b < nb; ++b)
            q5k_block(row + (size_t)b * KQO_Q5K_BLOCK_BYTES, out + (size_t)b * KQO_QK_K);
    } else {
        for (uint32_t b = 0; b < nb; ++b)
            q6k_block(row + (size_t)b * KQO_Q6K_BLOCK_BYTES, out + (size_t)b * KQO_QK_K);
    }
}

int kqo_dequant(int type, const void *raw, float *out, uint32_t N, uint32_t K)
{
    const uint32_t bb = kqo_block_bytes(type);
    if (!bb || K % KQO_QK_K) return -1;
    const uint32_t nb = K / KQO_QK_K;
    const uint8_t *src = (const uint8_t *)raw;
    for (uint32_t n = 0; n < N; ++n)
        dequant_row_bytes(type, src + (size_t)n * nb * bb, nb, out + (size_t)n * K);
    return 0;
}

int kqo_dequant_packed_row(int type, const uint32_t *packed,
                           uint32_t row_stride_words, uint32_t row, uint32_t K,
                           float *out)
{
    if (!kqo_block_bytes(type) || K % KQO_QK_K) return -1;
    const uint8_t *p = (const uint8_t *)packed + (size_t)row * row_stride_words * 4u;
    dequant_row_bytes(type, p, K / KQO_QK_K, out);
    return 0;
}

int kqo_dequant_rows(int type, const uint32_t *packed, uint32_t row_stride_words,
                     const int32_t *rows, uint32_t M, uint32_t K, float *out)
{
    for (uint32_t m = 0; m < M; ++m) {
        /* runtime/kernels/quant_kq/q6k_gather_batched.wgsl:17 clamps at zero */
        const uint32_t r = rows[m] > 0 ? (uint32_t)rows[m] : 0u;
        if (kqo_dequant_packed_row(type, packed, row_stride_words, r, K,
                                   out + (size_t)m * K))
            return -1;
    }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* matmul, runtime/tests/kernel_test.cpp:1682 / :1728                        */
/* ------------------------------------------------------------------------ */
int kqo_matmul(int type, const float *X, const uint32_t *packed, const float *bias,
               float *Y, uint32_t M, uint32_t N, uint32_t K,
               uint32_t row_stride_words, uint32_t y_offset, uint32_t ldy)
{
    if (!kqo_block_bytes(type) || K % KQO_QK_K) return -1;
    if (!ldy) ldy = N;
    float *w = (float *)malloc((size_t)K * sizeof(float));
    if (!w) return -2;
    for (uint32_t n = 0; n < N; ++n) {
        kqo_dequant_packed_row(type, packed, row_stride_words, n, K, w);
        for (uint32_t m = 0; m < M; ++m) {
            const float *x = X + (size_t)m * K;
            float a = bias ? bias[n] : 0.0f;
            for (uint32_t k = 0; k < K; ++k) a += x[k] * w[k];
            Y[(size_t)m * ldy + y_offset + n] = a;
        }
    }
    free(w);
    return 0;
}

int kqo_prologue(int pro, const float *X, const float *norm_w, float eps,
                 uint32_t M, uint32_t K, float *out)
{
    if (pro < 1 || pro > 3) return -1;
    for (uint32_t m = 0; m < M; ++m) {
        float *o = out + (size_t)m * K;
        if (pro == 1) {
            const float *x = X + (size_t)m * K;
            float ss = 0.0f;
            for (uint32_t k = 0; k < K; ++k) ss += x[k] * x[k];
            const float rstd = 1.0f / sqrtf(ss / (float)K + eps);
            for (uint32_t k = 0; k < K; ++k) o[k] = x[k] * rstd * norm_w[k];
        } else {
            const float *g = X + (size_t)m * 2u * K, *u = g + K;
            for (uint32_t k = 0; k < K; ++k) {
                float a;
                if (pro == 2) {
                    a = g[k] / (expf(0.0f - g[k]) + 1.0f);
                } else {
                    const float inner = 0.7978845608f * (g[k] + 0.044715f * g[k] * g[k] * g[k]);
                    a = 0.5f * g[k] * (1.0f + tanhf(inner));
                }
                o[k] = a * u[k];
            }
        }
    }
    return 0;
}

int kqo_matmul_f64(int type, const float *X, const uint32_t *packed,
                   const float *bias, double *Y, uint32_t M, uint32_t N,
                   uint32_t K, uint32_t row_stride_words)
{
    if (!kqo_block_bytes(type) || K % KQO_QK_K) return -1;
    float *w = (float *)malloc((size_t)K * sizeof(float));
    if (!w) return -2;
    for (uint32_t n = 0; n < N; ++n) {
        kqo_dequant_packed_row(type, packed, row_stride_words, n, K, w);
        for (uint32_t m = 0; m < M; ++m) {
            const float *x = X + (size_t)m * K;
            double a = bias ? (double)bias[n] : 0.0;
            for (uint32_t k = 0; k < K; ++k) a += (double)x[k] * (double)w[k];
            Y[(size_t)m * N + n] = a;
        }
    }
    free(w);
    return 0;
}

static float bf16_to_f32(uint16_t b)
{
    const uint32_t u = (uint32_t)b << 16;
    float f;
    memcpy(&f, &u, sizeof f);
    return f;
}

int kqo_matmul_bf16(int type, const uint16_t *Xbf16, const uint32_t *packed,
                    const float *bias, float *Y, uint32_t M, uint32_t N,
                    uint32_t K, uint32_t row_stride_words)
{
    float *X = (float *)malloc((size_t)M * K * sizeof(float));
    if (!X) return -2;
    for (size_t i = 0; i < (size_t)M * K; ++i) X[i] = bf16_to_f32(Xbf16[i]);
    const int rc = kqo_matmul(type, X, packed, bias, Y, M, N, K, row_stride_words, 0, 0);
    free(X);
    return rc;
}

static double now_s(void)
{
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}

int kqo_matmul_timed(int type, const float *X, const void *raw, float *deq,
                     float *Y, uint32_t M, uint32_t N, uint32_t K,
                     double *t_dequant, double *t_dot)
{
    const double t0 = now_s();
    if (kqo_dequant(type, raw, deq, N, K)) return -1;
    const double t1 = now_s();
    for (uint32_t m = 0; m < M; ++m)
        for (uint32_t n = 0; n < N; ++n) {
            const float *x = X + (size_t)m * K;
            const float *w = deq + (size_t)n * K;
            float a = 0.0f;
            for (uint32_t k = 0; k < K; ++k) a += x[k] * w[k];
            Y[(size_t)m * N + n] = a;
        }
    const double t2 = now_s();
    if (t_dequant) *t_dequant = t1 - t0;
    if (t_dot) *t_dot = t2 - t1;
    return 0;
}

/* ------------------------------------------------------------------------ */
/* MoE                                                                       */
/* ------------------------------------------------------------------------ */

/* runtime/kernels/moe/topk_softmax.wgsl:23-67 */
void kqo_moe_topk_softmax(const float *logits, uint32_t n_experts, uint32_t k,
                          int normalize, uint32_t *idx, float *wt)
{
    unsigned char *taken = (unsigned char *)calloc(n_experts ? n_experts : 1, 1);
    for (uint32_t s = 0; s < k; ++s) {
        float best = -3.4e38f;
        uint32_t bi = 0;
        for (uint32_t e = 0; e < n_experts; ++e)
            if (!taken[e] && logits[e] > best) { best = logits[e]; bi = e; }
        idx[s] = bi;
        wt[s] = best;
        taken[bi] = 1;
    }
    free(taken);
    float mx = wt[0];
    for (uint32_t s = 1; s < k; ++s) if (wt[s] > mx) mx = wt[s];
    float sum = 0.0f;
    for (uint32_t s = 0; s < k; ++s) { wt[s] = expf(wt[s] - mx); sum += wt[s]; }
    const float inv = (normalize && sum > 0.0f) ? 1.0f / sum : 1.0f;
    for (uint32_t s = 0; s < k; ++s) wt[s] *= inv;
}

/* runtime/kernels/moe/compute_offsets.wgsl:25-36 */
void kqo_moe_offsets(const uint32_t *idx, uint32_t k, uint32_t rows_per_expert,
                     uint32_t *offsets)
{
    for (uint32_t s = 0; s < k; ++s) offsets[s] = idx[s] * rows_per_expert;
}

/* runtime/kernels/quant_kq/iq4xs_matmul_moe.wgsl:55-66 (row = col + offset)
 * and runtime/ops/moe.cpp:486-592 (expert = expert_indices[tok*k + slot]). */
int kqo_moe_matmul(int type, const float *X, const uint32_t *packed,
                   const uint32_t *expert_idx, float *Y, uint32_t T, uint32_t k,
                   uint32_t N, uint32_t K, uint32_t row_stride_words,
                   int x_per_slot)
{
    for (uint32_t t = 0; t < T; ++t)
        for (uint32_t s = 0; s < k; ++s) {
            const uint32_t pair = t * k + s;
            const uint32_t e = expert_idx[pair];
            const uint32_t *w = packed + (size_t)e * N * row_stride_words;
            const float *x = X + (size_t)(x_per_slot ? pair : t) * K;
            if (kqo_matmul(type, x, w, NULL, Y + (size_t)pair * N, 1, N, K,
                           row_stride_words, 0, 0))
                return -1;
        }
    return 0;
}

/* runtime/model_runner.cpp:3584-3651 (per-slot gate, up, act, down, weighted
 * add), runtime/kernels/fused/silu_mul_fused.wgsl:39-49 (g / (exp(-g)+1) * u),
 * runtime/kernels/moe/weighted_add_indirect_batched.wgsl:53-70 (slot 0 writes,
 * later slots add). */
int kqo_moe_ffn(int type_gu, int type_dn, const float *X,
                const uint32_t *gate, const uint32_t *up, const uint32_t *down,
                const uint32_t *expert_idx, const float *expert_wt, float *out,
                uint32_t T, uint32_t k, uint32_t hidden, uint32_t inter)
{
    const uint32_t rs_gu = kqo_row_stride_words(type_gu, hidden);
    const uint32_t rs_dn = kqo_row_stride_words(type_dn, inter);
    float *g = (float *)malloc((size_t)inter * sizeof(float));
    float *u = (float *)malloc((size_t)inter * sizeof(float));
    float *y = (float *)malloc((size_t)hidden * sizeof(float));
    if (!g || !u || !y) { free(g); free(u); free(y); return -2; }
    int rc = 0;
    for (uint32_t t = 0; t < T && !rc; ++t) {
        const float *x = X + (size_t)t * hidden;
        float *o = out + (size_t)t * hidden;
        for (uint32_t s = 0; s < k && !rc; ++s) {
            const uint32_t e = expert_idx[t * k + s];
            const float w = expert_wt[t * k + s];
            rc |= kqo_matmul(type_gu, x, gate + (size_t)e * inter * rs_gu, NULL, g,
                             1, inter, hidden, rs_gu, 0, 0);
            rc |= kqo_matmul(type_gu, x, up + (size_t)e * inter * rs_gu, NULL, u,
                             1, inter, hidden, rs_gu, 0, 0);
            for (uint32_t i = 0; i < inter; ++i)
                g[i] = g[i] / (expf(-g[i]) + 1.0f) * u[i];
            rc |= kqo_matmul(type_dn, g, down + (size_t)e * hidden * rs_dn, NULL, y,
                             1, hidden, inter, rs_dn, 0, 0);
            for (uint32_t i = 0; i < hidden; ++i)
                o[i] = s == 0 ? w * y[i] : o[i] + w * y[i];
        }
    }
    free(g); free(u); free(y);
    return rc;
}

/* ------------------------------------------------------------------------ */
/* the reference test-suite's generators, kernel_test.cpp:62-112             */
/* ------------------------------------------------------------------------ */
void kqo_rng_seed(kqo_rng *r, uint32_t seed)
{
    r->s[0] = seed;
    r->s[1] = seed ^ 0x9E3779B9u;
    r->s[2] = seed ^ 0x6A09E667u;
    r->s[3] = seed ^ 0xBB67AE85u;
    for (int i = 0; i < 8; ++i) (void)kqo_rng_next(r);
}

uint32_t kqo_rng_next(kqo_rng *r)
{
    uint32_t *s = r->s;
    const uint32_t out = s[0] + s[3];
    const uint32_t t = s[1] << 9;
    s[2] ^= s[0];
    s[3] ^= s[1];
    s[1] ^= s[2];
    s[0] ^= s[3];
    s[2] ^= t;
    s[3] = (s[3] << 11) | (s[3] >> 21);
    return out;
}

float kqo_rng_uniform(kqo_rng *r, float lo, float hi)
{
    const float u = (float)(kqo_rng_next(r) >> 8) / (float)(1 << 24);
    return lo + u * (hi - lo);
}

float kqo_rng_randn(kqo_rng *r)
{
    const float u1 = kqo_rng_uniform(r, 1e-6f, 1.0f);
    const float u2 = kqo_rng_uniform(r, 0.0f, 6.2831853f);
    return sqrtf(-2.0f * logf(u1)) * cosf(u2);
}

void kqo_rng_randn_vec(kqo_rng *r, float *out, int n)
{
    for (int i = 0; i < n; ++i) out[i] = kqo_rng_randn(r);
}

/* Truncating fp32->fp16 used only to build test inputs: mantissa chopped,
 * results below the normal range become signed zero, above become inf. */
uint16_t kqo_f32_to_f16_trunc(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    const uint32_t sign = (u >> 16) & 0x8000u;
    const int e = (int)((u >> 23) & 255u) - 112;
    if (e <= 0) return (uint16_t)sign;
    if (e >= 31) return (uint16_t)(sign | 0x7C00u);
    return (uint16_t)(sign | ((uint32_t)e << 10) | ((u >> 13) & 1023u));
}

/* runtime/tests/kernel_test.cpp:298-317 */
int kqo_assert_close(const float *actual, const float *expected, int n,
                     float atol, float rtol, float *worst)
{
    int bad = 0;
    float w = 0.0f;
    for (int i = 0; i < n; ++i) {
        const float diff = fabsf(actual[i] - expected[i]);
        const float tol = atol + rtol * fabsf(expected[i]);
        if (!(diff <= tol)) {
            ++bad;
            if (diff - tol > w || diff != diff) w = diff - tol;
        }
    }
    if (worst) *worst = w;
    return bad;
}
