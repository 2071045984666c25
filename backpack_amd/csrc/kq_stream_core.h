// kq_stream_core.h — the per-lane pieces of the lanes-along-K decode matvec, shared by the kernels that
// walk weight rows with the lanes of a wave laid along K (kq_stream.hip: one launch per matvec;
// kq_chain.hip: one launch for a chain of matvecs): nibble-to-fp16-subnormal dot products of one lane's
// piece of a Q4_K / Q5_K / Q6_K row, the register ring of rows in flight with hand-waited loads, and the
// wave-wide sum.
#pragma once
#include "kq_format.h"
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace kq {

typedef _Float16 s_half2 __attribute__((ext_vector_type(2)));
typedef uint32_t s_u32x4 __attribute__((ext_vector_type(4)));

constexpr int STREAM_PRO_NONE = 0;   // x = X
constexpr int STREAM_PRO_NORM = 1;   // x = X * rsqrt(mean(X^2) + eps) * norm_w   (quant_kq/q4k_matmul_norm.wgsl:50-91)
constexpr int STREAM_PRO_SILU = 2;   // x = silu(X) * X2                          (fused/silu_mul_fused.wgsl:39-49)
constexpr int STREAM_PRO_GELU = 3;   // x = gelu_tanh(X) * X2                     (quant_kq/q4k_down_gelu.wgsl:50-56)

// silu(g) = g / (exp(-g) + 1) and the tanh form of gelu the reference uses.  The grouped (MoE) kernels
// evaluate silu with expf and a true division, the formula of moe_silu_mul_kernel, so that their fused
// and separate forms agree to the bit; the dense fused kernels use the hardware exponential and
// reciprocal (a few units in the last place, far inside the path's 1e-3), because this arithmetic sits
// in front of the first weight of every launch.
template <int PRO, bool FAST>
__device__ __forceinline__ float stream_act(float g, float u)
{
    if constexpr (PRO == STREAM_PRO_SILU) {
        if constexpr (FAST) return g * __builtin_amdgcn_rcpf(__expf(-g) + 1.0f) * u;
        else return g / (expf(-g) + 1.0f) * u;
    } else {
        const float inner = 0.7978845608f * (g + 0.044715f * g * g * g);
        // tanh(z) = 1 - 2 / (exp(2z) + 1); 0.5 g (1 + tanh z) = g - g / (exp(2z) + 1)
        const float e = __expf(2.0f * inner);
        return (g - g * __builtin_amdgcn_rcpf(e + 1.0f)) * u;
    }
}

__device__ __forceinline__ float s_fma_h(_Float16 h, float x, float acc) { return __builtin_fmaf((float)h, x, acc); }

template <int CTRL>
__device__ __forceinline__ float s_dpp(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

// Sum over the 64 lanes; the result is wave-uniform.
__device__ __forceinline__ float wave_sum(float v)
{
    v += s_dpp<0xB1>(v);    // quad: lanes ^ 1
    v += s_dpp<0x4E>(v);    // quad: lanes ^ 2
    v += s_dpp<0x141>(v);   // mirror within 8
    v += s_dpp<0x140>(v);   // mirror within 16
    const float a = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
    const float b = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
    const float c = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
    const float d = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
    return (a + b) + (c + d);
}

// (A source that includes this header carries the build's no-spill marker, so that the build refuses it
// if any kernel in it spills.)
// Weight loads whose completion is waited for by hand.  The compiler's own
// s_waitcnt placement drains the whole queue at the loop head when a register
// ring is refilled inside a loop, which serialises fetch and arithmetic; these
// loads are invisible to it.  Rules that keep this sound: (1) a register
// filled by one of these loads is not read until it has passed through
// ring_wait<N>() below (the "+v" operands make every later use depend on the
// wait); (2) vector memory operations complete in issue order, so after
// s_waitcnt vmcnt(N) every load but the N youngest has landed; (3) loads the
// compiler does track only ever wait for more than they need; (4) the
// destination is an in/out operand, so a ring variable keeps its register from
// one refill to the next, and the file is built with a check that nothing
// spills: a register that was saved and reused before its load landed would
// be overwritten by the late data.
typedef uint32_t s_u32x2 __attribute__((ext_vector_type(2)));

// Every such load and wait carries a marker in its assembly text (a comment that names the registers), and
// the build reads the generated code: in each kernel the registers the marked loads write must be exactly
// the registers the marked waits pass through.  A register copied between its load and its wait (a split
// live range, a copy on a loop's back edge) would show up as a load whose register no wait names.
// With KQ_TRACKED_LOADS defined the same kernels are built with ordinary loads that the compiler waits for
// itself (slower: it drains the queue at every refill): the fallback for a compiler the check rejects.
typedef uint32_t s_u32x4_u __attribute__((ext_vector_type(4), aligned(2)));
typedef uint32_t s_u32x2_u __attribute__((ext_vector_type(2), aligned(2)));

__device__ __forceinline__ void ring_load16(s_u32x4& v, const uint8_t* ptr)
{
#ifdef KQ_TRACKED_LOADS
    v = *(const s_u32x4_u*)ptr;
#else
    asm volatile("global_load_dwordx4 %0, %1, off ; ringld" : "+v"(v) : "v"(ptr));
#endif
}

__device__ __forceinline__ void ring_load8(s_u32x2& v, const uint8_t* ptr)
{
#ifdef KQ_TRACKED_LOADS
    v = *(const s_u32x2_u*)ptr;
#else
    asm volatile("global_load_dwordx2 %0, %1, off ; ringld" : "+v"(v) : "v"(ptr));
#endif
}

__device__ __forceinline__ void ring_load2(uint32_t& v, const uint8_t* ptr)
{
#ifdef KQ_TRACKED_LOADS
    v = *(const uint16_t*)ptr;
#else
    asm volatile("global_load_ushort %0, %1, off ; ringld" : "+v"(v) : "v"(ptr));
#endif
}

// One lane's share of one pass of a Q4_K row, for MT tokens (the unpack is shared).
//   hdr: the block's first 16 bytes; q: 16 quant bytes (piece j of the block)
//   xlo/xhi: activations of the piece's 16 elements in the even / odd sub-block
//   sel_hi: lane constant, j/2 >= 2;  sh: lane constant, 16 * ((j/2) & 1)
// Q5: qh holds the 16 bytes of fifth bits of the piece's elements (bit 2g of a byte for the even sub-block,
// bit 2g+1 for the odd one, sbit = 2g); the bit joins its nibble in the fp16 mantissa (bit 4 beside a low
// nibble, bit 8 beside a high one: a five-bit value is still a subnormal).
template <int MT, bool Q5 = false>
__device__ __forceinline__ void q4k_piece_dot(const s_u32x4 hdr, const s_u32x4 q, const float (&xlo)[MT][16],
                                              const float (&xhi)[MT][16], const float (&xs_lo)[MT],
                                              const float (&xs_hi)[MT], bool sel_hi, uint32_t sh, float (&acc)[MT],
                                              const s_u32x4 qh = s_u32x4{0, 0, 0, 0}, uint32_t sbit = 0)
{
    float alo[MT], ahi[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) { alo[t] = 0.0f; ahi[t] = 0.0f; }
#pragma unroll
    for (int m = 0; m < 4; ++m) {
        const uint32_t w = q[m];
        const uint32_t w8 = w >> 8;
        uint32_t ua = w & 0x000F000Fu;     // low nibbles of bytes 0, 2
        uint32_t ub = w & 0x00F000F0u;     // high nibbles of bytes 0, 2 (x16)
        uint32_t uc = w8 & 0x000F000Fu;    // low nibbles of bytes 1, 3
        uint32_t ud = w8 & 0x00F000F0u;    // high nibbles of bytes 1, 3 (x16)
        if constexpr (Q5) {
            const uint32_t hb = qh[m] >> sbit;   // bit 0 of each byte: even sub-block; bit 1: odd sub-block
            ua |= (hb << 4) & 0x00100010u;
            uc |= (hb >> 4) & 0x00100010u;
            ub |= (hb << 7) & 0x01000100u;
            ud |= (hb >> 1) & 0x01000100u;
        }
        const s_half2 a = __builtin_bit_cast(s_half2, ua);
        const s_half2 b = __builtin_bit_cast(s_half2, ub);
        const s_half2 c = __builtin_bit_cast(s_half2, uc);
        const s_half2 d = __builtin_bit_cast(s_half2, ud);
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            alo[t] = s_fma_h(a.x, xlo[t][4 * m + 0], alo[t]);
            ahi[t] = s_fma_h(b.x, xhi[t][4 * m + 0], ahi[t]);
            alo[t] = s_fma_h(c.x, xlo[t][4 * m + 1], alo[t]);
            ahi[t] = s_fma_h(d.x, xhi[t][4 * m + 1], ahi[t]);
            alo[t] = s_fma_h(a.y, xlo[t][4 * m + 2], alo[t]);
            ahi[t] = s_fma_h(b.y, xhi[t][4 * m + 2], ahi[t]);
            alo[t] = s_fma_h(c.y, xlo[t][4 * m + 3], alo[t]);
            ahi[t] = s_fma_h(d.y, xhi[t][4 * m + 3], ahi[t]);
        }
    }
    // 6-bit scale and min of sub-blocks 2g and 2g+1: two adjacent bytes of each
    // scale word, at bit sh
    const uint32_t y2 = hdr.y >> sh, z2 = hdr.z >> sh, w2 = hdr.w >> sh;
    const uint32_t sc_a = y2 & 0x3F3Fu, mn_a = z2 & 0x3F3Fu;
    const uint32_t sc_b = (w2 & 0x0F0Fu) | ((y2 >> 2) & 0x3030u);
    const uint32_t mn_b = ((w2 >> 4) & 0x0F0Fu) | ((z2 >> 2) & 0x3030u);
    const uint32_t sc = sel_hi ? sc_b : sc_a;
    const uint32_t mn = sel_hi ? mn_b : mn_a;
    const float sc0 = (float)(sc & 0xFFu), sc1 = (float)(sc >> 8) * 0.0625f;
    const float mn0 = (float)(mn & 0xFFu), mn1 = (float)(mn >> 8);
    const float d24 = half_bits_to_float(hdr.x & 0xFFFFu) * 16777216.0f;
    const float dmin = half_bits_to_float(hdr.x >> 16);
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        // alo carries 2^-24, ahi 2^-20
        const float tt = __builtin_fmaf(sc1, ahi[t], sc0 * alo[t]);
        const float u = __builtin_fmaf(mn1, xs_hi[t], mn0 * xs_lo[t]);
        acc[t] += __builtin_fmaf(d24, tt, -(dmin * u));
    }
}

// One row in flight for the Q4_K / Q5_K kernel: P headers and P quant pieces per lane, for Q5_K also P
// pieces of fifth bits (blocks of 176 bytes: header, 32 bytes of fifth bits, quants).
template <int P, bool Q5>
struct Q4Slot {
    s_u32x4 hdr[P], q[P], qh[Q5 ? P : 1];
    __device__ __forceinline__ void fill(const uint8_t* row, const uint32_t (&hoff)[P], uint32_t j)
    {
#pragma unroll
        for (int pass = 0; pass < P; ++pass) {
            ring_load16(hdr[pass], row + hoff[pass]);
            ring_load16(q[pass], row + hoff[pass] + (Q5 ? 48u : 16u) + 16u * j);
            if constexpr (Q5) ring_load16(qh[pass], row + hoff[pass] + 16u + 16u * (j & 1u));
        }
    }
    // Every register of the slot passes through the wait.
    template <int N>
    __device__ __forceinline__ void wait()
    {
        if constexpr (Q5 && P == 1)
            asm volatile("s_waitcnt vmcnt(%3) ; ringwait %0 %1 %2" : "+v"(hdr[0]), "+v"(q[0]), "+v"(qh[0]) : "n"(N));
        else if constexpr (Q5)
            asm volatile("s_waitcnt vmcnt(%6) ; ringwait %0 %1 %2 %3 %4 %5"
                         : "+v"(hdr[0]), "+v"(q[0]), "+v"(qh[0]), "+v"(hdr[1]), "+v"(q[1]), "+v"(qh[1])
                         : "n"(N));
        else if constexpr (P == 1)
            asm volatile("s_waitcnt vmcnt(%2) ; ringwait %0 %1" : "+v"(hdr[0]), "+v"(q[0]) : "n"(N));
        else
            asm volatile("s_waitcnt vmcnt(%4) ; ringwait %0 %1 %2 %3" : "+v"(hdr[0]), "+v"(q[0]), "+v"(hdr[1]), "+v"(q[1]) : "n"(N));
    }
};

struct Q6Piece {
    s_u32x2 a, b, h, sc;
    uint32_t d;
};

// One row in flight for the Q6_K kernel: P pieces per lane, 5 loads each.
template <int P>
struct Q6Slot {
    Q6Piece v[P];
    __device__ __forceinline__ void fill(const uint8_t* row, const uint32_t (&boff)[P], uint32_t n, uint32_t lg)
    {
#pragma unroll
        for (int pass = 0; pass < P; ++pass) {
            const uint8_t* blk = row + boff[pass];
            ring_load8(v[pass].a, blk + 64u * n + 8u * lg);
            ring_load8(v[pass].b, blk + 64u * n + 32u + 8u * lg);
            ring_load8(v[pass].h, blk + 128u + 32u * n + 8u * lg);
            ring_load8(v[pass].sc, blk + 192u + 8u * n);
            ring_load2(v[pass].d, blk + 208u);
        }
    }
    template <int N>
    __device__ __forceinline__ void wait()
    {
        if constexpr (P == 1)
            asm volatile("s_waitcnt vmcnt(%5) ; ringwait %0 %1 %2 %3 %4"
                         : "+v"(v[0].a), "+v"(v[0].b), "+v"(v[0].h), "+v"(v[0].sc), "+v"(v[0].d)
                         : "n"(N));
        else
            asm volatile("s_waitcnt vmcnt(%10) ; ringwait %0 %1 %2 %3 %4 %5 %6 %7 %8 %9"
                         : "+v"(v[0].a), "+v"(v[0].b), "+v"(v[0].h), "+v"(v[0].sc), "+v"(v[0].d), "+v"(v[1].a),
                           "+v"(v[1].b), "+v"(v[1].h), "+v"(v[1].sc), "+v"(v[1].d)
                         : "n"(N));
    }
};

// x[t][k][i]: activation of element 128n + 32k + 8lg + i of token t;  m32xs[t][k] = -32 * sum_i x[t][k][i]
template <int MT>
__device__ __forceinline__ void q6k_piece_dot(const Q6Piece& v, const float (&x)[MT][4][8], const float (&m32xs)[MT][4],
                                              uint32_t sc_shift, float (&acc)[MT])
{
    float a[MT][4];
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int k = 0; k < 4; ++k) a[t][k] = 0.0f;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const uint32_t A = v.a[u], B = v.b[u], H = v.h[u];
        const uint32_t A8 = A >> 8, B8 = B >> 8;
        const uint32_t Hl4 = H << 4, Hl2 = H << 2, Hr4 = H >> 4, Hr6 = H >> 6;
        // [k][pair]: pair a holds positions l, l+2; pair b holds l+1, l+3
        const s_half2 q0a = __builtin_bit_cast(s_half2, (A & 0x000F000Fu) | (Hl4 & 0x00300030u));
        const s_half2 q2a = __builtin_bit_cast(s_half2, (A & 0x00F000F0u) | (Hl4 & 0x03000300u));
        const s_half2 q1a = __builtin_bit_cast(s_half2, (B & 0x000F000Fu) | (Hl2 & 0x00300030u));
        const s_half2 q3a = __builtin_bit_cast(s_half2, (B & 0x00F000F0u) | (Hl2 & 0x03000300u));
        const s_half2 q0b = __builtin_bit_cast(s_half2, (A8 & 0x000F000Fu) | (Hr4 & 0x00300030u));
        const s_half2 q2b = __builtin_bit_cast(s_half2, (A8 & 0x00F000F0u) | (Hr4 & 0x03000300u));
        const s_half2 q1b = __builtin_bit_cast(s_half2, (B8 & 0x000F000Fu) | (Hr6 & 0x00300030u));
        const s_half2 q3b = __builtin_bit_cast(s_half2, (B8 & 0x00F000F0u) | (Hr6 & 0x03000300u));
        const int i = 4 * u;
#pragma unroll
        for (int t = 0; t < MT; ++t) {
            a[t][0] = s_fma_h(q0a.x, x[t][0][i + 0], a[t][0]);
            a[t][1] = s_fma_h(q1a.x, x[t][1][i + 0], a[t][1]);
            a[t][2] = s_fma_h(q2a.x, x[t][2][i + 0], a[t][2]);
            a[t][3] = s_fma_h(q3a.x, x[t][3][i + 0], a[t][3]);
            a[t][0] = s_fma_h(q0b.x, x[t][0][i + 1], a[t][0]);
            a[t][1] = s_fma_h(q1b.x, x[t][1][i + 1], a[t][1]);
            a[t][2] = s_fma_h(q2b.x, x[t][2][i + 1], a[t][2]);
            a[t][3] = s_fma_h(q3b.x, x[t][3][i + 1], a[t][3]);
            a[t][0] = s_fma_h(q0a.y, x[t][0][i + 2], a[t][0]);
            a[t][1] = s_fma_h(q1a.y, x[t][1][i + 2], a[t][1]);
            a[t][2] = s_fma_h(q2a.y, x[t][2][i + 2], a[t][2]);
            a[t][3] = s_fma_h(q3a.y, x[t][3][i + 2], a[t][3]);
            a[t][0] = s_fma_h(q0b.y, x[t][0][i + 3], a[t][0]);
            a[t][1] = s_fma_h(q1b.y, x[t][1][i + 3], a[t][1]);
            a[t][2] = s_fma_h(q2b.y, x[t][2][i + 3], a[t][2]);
            a[t][3] = s_fma_h(q3b.y, x[t][3][i + 3], a[t][3]);
        }
    }
    // scale of (half n, k, l/16) is byte 2k + l/16 of the half's eight: sc_shift = 8 * (l/16)
    const uint32_t s01 = v.sc.x >> sc_shift, s23 = v.sc.y >> sc_shift;
    const float sc0 = (float)(int)(int8_t)(s01 & 255u), sc1 = (float)(int)(int8_t)((s01 >> 16) & 255u);
    const float sc2 = (float)(int)(int8_t)(s23 & 255u), sc3 = (float)(int)(int8_t)((s23 >> 16) & 255u);
    const float d = half_bits_to_float(v.d);
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        float tot = sc0 * __builtin_fmaf(a[t][0], 16777216.0f, m32xs[t][0]);
        tot = __builtin_fmaf(sc1, __builtin_fmaf(a[t][1], 16777216.0f, m32xs[t][1]), tot);
        tot = __builtin_fmaf(sc2, __builtin_fmaf(a[t][2], 1048576.0f, m32xs[t][2]), tot);
        tot = __builtin_fmaf(sc3, __builtin_fmaf(a[t][3], 1048576.0f, m32xs[t][3]), tot);
        acc[t] += d * tot;
    }
}

}  // namespace kq
