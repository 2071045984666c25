// kq_mtile.hip — fused dequant-matmul for M = 2..16 tokens on the matrix cores,
// tiles of 16 weight rows x 16 tokens (speculative-decode verify batches).
//
// v_mfma_f32_16x16x32_f16 multiplies a 16 x 32 block of activations (A, one
// token per row) with a 32 x 16 block of weights (B, one weight row per column)
// into a 16 x 16 fp32 tile.  Lane l of the wave holds, for both operands, eight
// consecutive k (8*(l/16) .. +7) of token / weight row l%16, and of the result
// the four tokens 4*(l/16) .. +3 of weight row l%16: a lane deals with a single
// weight row, so block and sub-block scales are per-lane scalars.
//
// Weights.  The eight k of a lane are eight consecutive bytes of the block's
// quants (one 64-bit load): their low nibbles belong to sub-block 2g, their
// high nibbles to sub-block 2g+1.  A masked nibble left in the low mantissa
// bits of an fp16 is the subnormal q * 2^-24 (q * 2^-20 four bits up), which
// the matrix cores multiply exactly, so ten bit-ops per 8 bytes yield the B
// operands of two sub-blocks.  Every weight byte is fetched once per launch and
// used for all tokens.
//
// Activations.  fp32 X cannot go through fp16 unharmed, so a token's 256
// elements of a superblock are scaled by a power of two that puts the largest
// just below 2^15 and split into hi = fp16(x*s) and lo = fp16(x*s - hi), 22 bits
// in all; each sub-block costs two MFMAs into the same accumulator.  The
// workgroup converts a chunk of four superblocks of X at a time into LDS, in
// operand order, together with the per-sub-block sums of x that the Q4_K minima
// multiply.
//
// Q6_K.  Its scales cover 16 elements, half of one MFMA's k.  The token axis
// pays for that: with at most 8 tokens, token m appears twice, as (m, first
// half of k) in slot m and (m, second half) in slot m + 8, each with the other
// half of its operand zeroed.  One MFMA then yields both 16-element sums, each
// in lanes of its own that apply their own scale, and the two are added once
// at the end.  The -32 offset of the 6-bit values is applied against the sums
// of x over 16 elements.  With 9..16 tokens every token keeps a slot of its own
// and the weights pay instead: each run of 32 is multiplied twice, once whole
// and once with the operand lanes of its second half zeroed, which gives the
// sum over the first 16 elements and, by difference, the sum over the second
// (twice the matrix instructions, but every weight byte is still fetched and
// unpacked once for all 16 tokens).
//
// Work split.  A workgroup owns R tiles of 16 rows.  With R = NW every wave
// owns a tile and walks all of K; with R = 1 (matrices of few rows) the waves of
// the workgroup take different superblocks of the chunk and fold their partial
// tiles through LDS at the end.  There is no fold across workgroups.
#include <cmath>

#include "kq_format.h"
#include "kq_kernels.h"
#include "kq_wave.h"

namespace kq {

typedef _Float16 t_half8 __attribute__((ext_vector_type(8)));
typedef _Float16 t_half2 __attribute__((ext_vector_type(2)));
typedef float t_f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t t_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t t_u32x2 __attribute__((ext_vector_type(2)));

// Orders a wave's own LDS traffic (writes of a staging pass against the reads around it); no s_barrier.
__device__ __forceinline__ void wave_window_fence()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

constexpr int MT_KC = 4;                       // superblocks of X staged at a time
// The A operands in LDS: [block][sub-block] pairs of planes (hi, lo; or, with hi / lo slots, this chunk's and the
// next one's) of 64 positions of 16 bytes.  A matrix instruction's lane (slot, kq) reads position
// mt_xa_pos(slot, kq) of a plane: 1 KB runs, conflict-free.  The converting threads write one position each,
// 16 lanes at a time spread over sub-blocks and superblocks: the pitch of a pair is 16 bytes more than its 2 KB
// and a slot is rotated by 4 * kq inside its group of 16, so that those 16 writes (and a 16-thread pair's, whose
// two halves differ in kq) fall into 16 different bank groups; with pairs 2 KB apart and slots unrotated
// they all hit one (measured: a quarter of the 16-token kernel's cycles were LDS bank conflicts).
constexpr int MT_XA_PITCH = 2 * 1024 + 16;
constexpr int MT_XA_BYTES = MT_KC * 8 * MT_XA_PITCH;
__device__ __forceinline__ uint32_t mt_xa_pos(uint32_t slot, uint32_t kq) { return ((slot + 4u * kq) & 15u) + 16u * kq; }
constexpr int MT_XS_FLOATS = MT_KC * 8 * 32;        // [block][sub-block][token], or [block][sub-block][half][token]
constexpr int MT_INV_FLOATS = MT_KC * 16;           // [block][token]
constexpr int MT_XV_BYTES = MT_KC * 2 * 1024;       // [block][hi/lo][lane] 16 B: the sub-block sums as an A operand (Q4_K)
constexpr int MT_STAGE_BYTES = MT_XA_BYTES + (MT_XS_FLOATS + MT_INV_FLOATS) * 4 + MT_XV_BYTES;

// Kernel variant beside the GGUF type codes: Q6_K blocks, 16 token slots.
constexpr int MT_TYPE_Q6K_WIDE = 114;

struct MtileParams {
    const float* X;
    const uint8_t* W;
    const float* bias;
    float* Y;
    uint32_t M, N, K, n_blocks, row_stride_bytes, y_offset, ldy;
    uint32_t tiles_per_wg;   // R == NW kernels: waves below this own a tile, the others only help convert X
    // K split over blockIdx.z (dense calls): split z walks chunks [z * chunks_per_split, ...); each split
    // leaves its partial tile in partial[z][token][tile row], the last workgroup of a row group to arrive
    // adds them in split order
    uint32_t n_splits, chunks_per_split;
    float* partial;
    uint32_t* counters;      // one per blockIdx.x, zero between launches
    // grouped mode (tiles != nullptr): blockIdx.y walks records {expert, count, pair ids...} of up to
    // 16 (Q4_K) / 8 (Q6_K) (token, slot) pairs that share an expert; N is the rows of one expert
    // fused forms (the FUSED instantiations, dense calls of up to 16 tokens).  pro 1: x = X * rsqrt(mean(X^2) + eps)
    // * norm_w; pro 2 / 3: X rows are gate | up, 2K floats, x = silu / gelu_tanh (gate) * up.  residual is added to
    // every output (indexed like Y, may be Y).  epi 2 / 3: W is gate | up stacked, the first half of a workgroup's
    // waves own gate tiles, the second half the up tiles pair_tile0 further on, and Y = act(gate) * up.
    int pro, epi;
    float eps;
    const float* norm_w;
    const float* residual;
    uint32_t x_stride;      // floats between rows of X
    uint32_t pair_tile0;    // tiles of gate rows (= outputs / 16)
    const uint32_t* tiles;
    const uint32_t* n_tiles;
    const uint8_t* W2;      // DUAL kernels (grouped calls): a twin matrix (up beside gate); Y = silu(W x) * (W2 x)
    uint32_t tile_iters;    // grouped calls whose K is a single chunk: tiles a wave walks with X staged once
    uint32_t tile_stride;   // words per record
    uint32_t k_slots;
    int x_per_slot;         // X row of a pair: the pair itself (1) or its token, pair / k_slots (0)
};

// silu(g) * u (ACT 2) or gelu_tanh(g) * u (ACT 3), as the fused entry point defines them
template <int ACT>
__device__ __forceinline__ float mtile_act(float g, float u)
{
    if constexpr (ACT == 2) {
        return g / (__expf(-g) + 1.0f) * u;
    } else {
        const float inner = 0.7978845608f * (g + 0.044715f * g * g * g);
        // tanh(z) = 1 - 2 / (exp(2z) + 1); 0.5 g (1 + tanh z) = g - g / (exp(2z) + 1)
        return (g - g / (__expf(2.0f * inner) + 1.0f)) * u;
    }
}

// Conversion of a chunk's activations.  Thread (pair, sub) handles EPT
// consecutive elements of one (token, superblock) pair; pairs are numbered
// token-major, so a wave covers few tokens and waves whose tokens are all
// beyond M have nothing to do after their slots were zeroed once.
// TOK = 16 or 8 (4 works too): the tokens the workgroup's threads are spread over; a launch with few tokens takes a
// small TOK so that every wave converts a share instead of the first waves converting everything.
// XV: also stage the sub-block sums as an A operand (the Q4_K kernels that put the minima on the matrix cores).
// HALF: the sums of x go out per half run of 16 elements, [run][half][token] (the 16-token Q6_K kernel).
// PRO: the prologues of the fused forms.  1: RMSNorm, the chunk's norm weights are read from LDS (nw, staged by
// the kernel); 2: act(gate) * up, up travels with X.
// HL8: at most 8 tokens; a token's hi part goes to slot token and its lo part to slot token + 8 of ONE operand, so
// that a single matrix instruction multiplies both (the two partial tiles are added once at the end).
template <int NT, bool SPLIT16, int TOK, bool XV, bool HALF = false, int PRO = 0, bool HL8 = false>
struct MtileStager {
    static_assert(!(HL8 && (SPLIT16 || HALF)), "hi / lo slots are a form of the Q4_K / Q5_K kernels");
    static_assert(!(SPLIT16 && HALF), "half sums live in token slots (SPLIT16) or in a second plane (HALF)");
    static constexpr uint32_t XSR = HALF ? 32u : 16u;   // floats of xs per run
    static constexpr int TPP = NT / (MT_KC * TOK);  // threads per (token, block) pair
    static constexpr int EPT = 256 / TPP;           // elements per thread
    static_assert(TPP <= 64 && (EPT == 64 || EPT == 32 || EPT == 16 || EPT == 8), "a pair is converted inside one wave");
    float4 v[EPT / 4];
    float4 v2[PRO == 2 ? EPT / 4 : 1];
    float ss = 0.0f;   // norm prologue: sum of squares of this thread's elements so far
    uint32_t token, bb, sub;
    bool live_token;

    uint32_t xrow;   // row of X this thread converts
    __device__ __forceinline__ void init(const MtileParams& p, const uint32_t* rec, uint32_t count)
    {
        const uint32_t pair = threadIdx.x / TPP;
        sub = threadIdx.x % TPP;
        bb = pair % MT_KC;
        token = pair / MT_KC;
        live_token = token < count && (!(SPLIT16 || HL8) || token < 8u);
        xrow = token;
        if (rec && live_token) {
            const uint32_t pr = rec[2u + token];
            xrow = p.x_per_slot ? pr : pr / p.k_slots;
        }
    }
    // requests the chunk's elements (nothing for tokens beyond M; superblocks beyond K re-read the last
    // one, which is parked but never multiplied)
    __device__ __forceinline__ void fetch(const MtileParams& p, uint32_t c0)
    {
        if (!live_token) return;   // wave-uniform for whole waves of dead tokens
        const uint32_t b = min(c0 + bb, p.n_blocks - 1u);
        if constexpr (PRO == 2) {
            const float4* src = (const float4*)(p.X + (size_t)xrow * p.x_stride + (size_t)b * KQ_QK + sub * EPT);
            const float4* src2 = (const float4*)((const float*)src + p.K);
#pragma unroll
            for (int i = 0; i < EPT / 4; ++i) v[i] = src[i];
#pragma unroll
            for (int i = 0; i < EPT / 4; ++i) v2[i] = src2[i];
            return;
        }
        const float4* src = (const float4*)(p.X + (size_t)xrow * p.K + (size_t)b * KQ_QK + sub * EPT);
#pragma unroll
        for (int i = 0; i < EPT / 4; ++i) v[i] = src[i];
    }
    // the prologue on what fetch() brought.  The norm's 1 / rms is a factor per token: it is applied to the
    // outputs, and the sum of squares it needs is gathered here (live: the superblock exists).  nw: the chunk's
    // norm weights in LDS, [superblock of the chunk][256].
    __device__ __forceinline__ void prologue(const MtileParams& p, bool live, const float* nw)
    {
        if (!live_token) return;
        if constexpr (PRO == 1) {
            const float4* w4 = (const float4*)(nw + bb * KQ_QK + sub * EPT);
#pragma unroll
            for (int i = 0; i < EPT / 4; ++i) {
                if (live) {
                    ss = fmaf(v[i].x, v[i].x, ss); ss = fmaf(v[i].y, v[i].y, ss);
                    ss = fmaf(v[i].z, v[i].z, ss); ss = fmaf(v[i].w, v[i].w, ss);
                }
                const float4 w = w4[i];
                v[i].x *= w.x; v[i].y *= w.y; v[i].z *= w.z; v[i].w *= w.w;
            }
        } else if constexpr (PRO == 2) {
            if (p.pro == 2) {
#pragma unroll
                for (int i = 0; i < EPT / 4; ++i) {
                    v[i].x = mtile_act<2>(v[i].x, v2[i].x); v[i].y = mtile_act<2>(v[i].y, v2[i].y);
                    v[i].z = mtile_act<2>(v[i].z, v2[i].z); v[i].w = mtile_act<2>(v[i].w, v2[i].w);
                }
            } else {
#pragma unroll
                for (int i = 0; i < EPT / 4; ++i) {
                    v[i].x = mtile_act<3>(v[i].x, v2[i].x); v[i].y = mtile_act<3>(v[i].y, v2[i].y);
                    v[i].z = mtile_act<3>(v[i].z, v2[i].z); v[i].w = mtile_act<3>(v[i].w, v2[i].w);
                }
            }
        }
    }
    // converts what fetch() brought and parks it in LDS (slots of tokens beyond M stay zero)
    __device__ __forceinline__ void park(uint8_t* xa, float* xs, float* xinv, uint8_t* xv)
    {
        if (!live_token) return;   // wave-uniform for whole waves of dead tokens
        // largest magnitude of the pair's 256 elements, as float bits (orders like the floats)
        uint32_t amax = 0;
#pragma unroll
        for (int i = 0; i < EPT / 4; ++i) {
            amax = max(amax, __builtin_bit_cast(uint32_t, v[i].x) & 0x7FFFFFFFu);
            amax = max(amax, __builtin_bit_cast(uint32_t, v[i].y) & 0x7FFFFFFFu);
            amax = max(amax, __builtin_bit_cast(uint32_t, v[i].z) & 0x7FFFFFFFu);
            amax = max(amax, __builtin_bit_cast(uint32_t, v[i].w) & 0x7FFFFFFFu);
        }
        // (DPP moves: an LDS-routed shuffle costs a hundred cycles, and this chain sits in front of the barrier)
        if constexpr (TPP > 1) amax = max(amax, (uint32_t)group_partner<1>((int)amax));
        if constexpr (TPP > 2) amax = max(amax, (uint32_t)group_partner<2>((int)amax));
        if constexpr (TPP > 4) amax = max(amax, (uint32_t)group_partner<4>((int)amax));
        if constexpr (TPP > 8) amax = max(amax, (uint32_t)group_partner<8>((int)amax));
        static_assert(TPP <= 16, "the largest magnitude is reduced inside a row of 16 lanes");
        uint32_t e = amax >> 23;                  // biased exponent of the largest |x|
        e = e < 15u ? 15u : (e > 253u ? 253u : e);
        const float s = __builtin_bit_cast(float, (268u - e) << 23);     // 2^(141-e): amax*s in [2^14, 2^15)
        const float inv = __builtin_bit_cast(float, (e - 14u) << 23);    // 2^(e-141)
        if (sub == 0) {
            xinv[bb * 16u + token] = inv;
            if (SPLIT16 || HL8) xinv[bb * 16u + token + 8u] = inv;
        }
        // Q4_K: the sum over sub-block sb also goes out as element sb of an A operand (lane = token, the
        // lanes of k >= 8 stay zero), scaled by s / 32 so that 32 elements of at most 2^15 fit an fp16
        auto put_sum = [&](uint32_t sb, float sum) {
            if (!XV) return;
            const float a = sum * (s * 0.03125f);
            const _Float16 h = (_Float16)a;
            const _Float16 l = (_Float16)(a - (float)h);
            _Float16* dst = (_Float16*)(xv + ((size_t)(bb * 2u) * 64u + token) * 16u) + sb;
            dst[0] = h;
            dst[HL8 ? 64 : 512] = l;   // the lo operand: 1024 bytes on, or (HL8) slot token + 8
        };
        // Q6_K: the sum over the 16 elements of group g (its scale's reach) goes out as an A operand too, hi and lo
        // in one: element g % 8 of lane (token, g / 8) and of lane (token, 2 + g / 8), scaled like the Q4_K sums.
        // The product with the 16 scales of a weight row is then one matrix instruction per superblock.
        auto put_half = [&](uint32_t g, float sum) {
            const float a = sum * (s * 0.03125f);
            const _Float16 h = (_Float16)a;
            const _Float16 l = (_Float16)(a - (float)h);
            _Float16* dst = (_Float16*)(xv + (size_t)bb * 2048u + (token + 16u * (g >> 3)) * 16u) + (g & 7u);
            dst[0] = h;
            dst[256] = l;   // 32 lanes on
        };
        // groups of 8 consecutive k -> one operand slot: halves in the order k+0, k+2, k+1, k+3, k+4, k+6, k+5, k+7
#pragma unroll
        for (int g8 = 0; g8 < EPT / 8; ++g8) {
            const float4 lo4 = v[2 * g8], hi4 = v[2 * g8 + 1];
            const float a[8] = {lo4.x * s, lo4.y * s, lo4.z * s, lo4.w * s, hi4.x * s, hi4.y * s, hi4.z * s, hi4.w * s};
            _Float16 h[8], l[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                h[i] = (_Float16)a[i];
                l[i] = (_Float16)(a[i] - (float)h[i]);
            }
            const t_half8 hv = {h[0], h[2], h[1], h[3], h[4], h[6], h[5], h[7]};
            const t_half8 lv = {l[0], l[2], l[1], l[3], l[4], l[6], l[5], l[7]};
            const uint32_t k = sub * EPT + g8 * 8u;     // element of the superblock
            const uint32_t sb = k >> 5, kq = (k >> 3) & 3u;
            // SPLIT16: the first half of a 32-run goes to slot token, the second to slot token + 8
            const uint32_t slot = SPLIT16 ? token + 8u * (kq >> 1) : token;
            uint8_t* pair = xa + (size_t)(bb * 8u + sb) * MT_XA_PITCH;
            *(t_half8*)(pair + mt_xa_pos(slot, kq) * 16u) = hv;
            if (HL8) *(t_half8*)(pair + mt_xa_pos(slot + 8u, kq) * 16u) = lv;
            else *(t_half8*)(pair + 1024 + mt_xa_pos(slot, kq) * 16u) = lv;
        }
        // sums of the unscaled x over each run of 32 (or, SPLIT16, each half run of 16)
        if constexpr (EPT >= 32) {
#pragma unroll
            for (int q = 0; q < EPT / 32; ++q) {
                float h0 = 0.0f, h1 = 0.0f;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    h0 += (v[8 * q + i].x + v[8 * q + i].y) + (v[8 * q + i].z + v[8 * q + i].w);
                    h1 += (v[8 * q + 4 + i].x + v[8 * q + 4 + i].y) + (v[8 * q + 4 + i].z + v[8 * q + 4 + i].w);
                }
                float* dst = xs + (bb * 8u + (sub * EPT) / 32u + q) * XSR + token;
                if (SPLIT16 || HALF) { put_half(2u * ((sub * EPT) / 32u + q), h0); put_half(2u * ((sub * EPT) / 32u + q) + 1u, h1); }
                else { if (!HL8) dst[0] = h0 + h1; put_sum((sub * EPT) / 32u + q, h0 + h1); }   // (HL8 reads xv only)
            }
        } else {
            // the run is spread over 32 / EPT neighbouring threads: partial sums meet by lane exchange
            float h = 0.0f;
#pragma unroll
            for (int i = 0; i < EPT / 4; ++i) h += (v[i].x + v[i].y) + (v[i].z + v[i].w);
            constexpr int PER16 = 16 / EPT;   // threads per half run: 1 (EPT 16) or 2 (EPT 8)
            if (PER16 == 2) h += group_partner<1>(h);
            const uint32_t half = (sub / PER16) & 1u, run = sub / (2u * PER16);
            float* dst = xs + (bb * 8u + run) * XSR + token;
            if (SPLIT16 || HALF) {
                if (sub % PER16 == 0u) put_half(2u * run + half, h);
            } else {
                h += group_partner<PER16>(h);
                if (sub % (2u * PER16) == 0u) { if (!HL8) dst[0] = h; put_sum(run, h); }
            }
        }
    }
};

// One superblock of one 16-row tile: adds this block's contribution to tot[4]
// (tokens 4*(lane/16) .. +3 of weight row lane%16).  The LDS operands of sub-block s+1 are requested
// before the matrix instructions of sub-block s, and the scale arithmetic on a result runs one sub-block
// behind the instructions that produce it, so neither latency is waited for.
struct MtileA {
    t_half8 hi, lo;
};
template <bool HL8 = false>
__device__ __forceinline__ MtileA mtile_read_a(const uint8_t* xa_b, int sb, uint32_t lane)
{
    const uint8_t* ap = xa_b + (size_t)sb * MT_XA_PITCH + mt_xa_pos(lane & 15u, lane >> 4) * 16u;
    MtileA a;
    a.hi = *(const t_half8*)ap;
    a.lo = a.hi;
    if constexpr (!HL8) a.lo = *(const t_half8*)(ap + 1024);   // (HL8: hi and lo share the one operand)
    return a;
}

// The minima ride on the matrix cores as well: sum over sub-blocks of mn[row][sb] * xsum[token][sb] is one more
// product with k = sub-block (8 of the 32 k used): A = the staged sums (xv_b), B = the eight 6-bit minima of
// the lane's row as subnormals.  B's lanes of k >= 8 hold the same finite values; A is zero there.
// Q5: qhw holds the eight bytes of fifth bits of the lane's eight positions (bit sb of a byte belongs to
// sub-block sb); the bit joins its nibble in the fp16 mantissa (bit 4 beside a low nibble, bit 8 beside a high
// one: a five-bit value is still a subnormal), four more bit-ops per operand.
template <bool Q5>
__device__ __forceinline__ void q5_join(t_u32x4& blo, t_u32x4& bhi, const t_u32x2 qhw, uint32_t sbit)
{
    if constexpr (Q5) {
        const uint32_t h0 = qhw.x >> sbit, h1 = qhw.y >> sbit;   // bit 0 of each byte: sub-block sbit, bit 1: sbit + 1
        blo.x |= (h0 << 4) & 0x00100010u; blo.y |= (h0 >> 4) & 0x00100010u;
        blo.z |= (h1 << 4) & 0x00100010u; blo.w |= (h1 >> 4) & 0x00100010u;
        bhi.x |= (h0 << 7) & 0x01000100u; bhi.y |= (h0 >> 1) & 0x01000100u;
        bhi.z |= (h1 << 7) & 0x01000100u; bhi.w |= (h1 >> 1) & 0x01000100u;
    }
}

template <bool Q5, bool HL8 = false>
__device__ __forceinline__ void q4k_mtile_block(const t_u32x4 hdr, const t_u32x2 (&w)[4], const t_u32x2 qhw, const uint8_t* xa_b,
                                                const uint8_t* xv_b, const float* xinv_b, uint32_t lane,
                                                t_f32x4& tot)
{
    const float d = half_bits_to_float(hdr.x & 0xFFFFu);
    const float dmin = half_bits_to_float(hdr.x >> 16);
    const uint32_t scA = hdr.y & 0x3F3F3F3Fu;
    const uint32_t mnA = hdr.z & 0x3F3F3F3Fu;
    const uint32_t scB = (hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u);
    const uint32_t mnB = ((hdr.w >> 4) & 0x0F0F0F0Fu) | ((hdr.z >> 2) & 0x30303030u);
    t_f32x4 U = {0, 0, 0, 0};
    MtileA a_cur = mtile_read_a<HL8>(xa_b, 0, lane);
    const t_half8 vhi = *(const t_half8*)(xv_b + (size_t)lane * 16u);
    t_half8 vlo = vhi;
    if constexpr (!HL8) vlo = *(const t_half8*)(xv_b + 1024 + (size_t)lane * 16u);
    t_f32x4 D_prev = {0, 0, 0, 0};
    t_u32x4 blo = {0, 0, 0, 0}, bhi = {0, 0, 0, 0};
    auto scale_in = [&](int sb, const t_f32x4& D) {
        const uint32_t scw = sb < 4 ? scA : scB;
        // high nibbles sit four bits up: 1/16 goes into their scale
        const float sc = (float)((scw >> (8 * (sb & 3))) & 255u) * ((sb & 1) ? 0.0625f : 1.0f);
        U.x = fmaf(sc, D.x, U.x); U.y = fmaf(sc, D.y, U.y); U.z = fmaf(sc, D.z, U.z); U.w = fmaf(sc, D.w, U.w);
    };
#pragma unroll
    for (int sb = 0; sb < 8; ++sb) {
        MtileA a_next = a_cur;
        if (sb < 7) a_next = mtile_read_a<HL8>(xa_b, sb + 1, lane);
        if ((sb & 1) == 0) {
            const uint32_t d0 = w[sb >> 1].x, d1 = w[sb >> 1].y;
            const uint32_t e0 = d0 >> 8, e1 = d1 >> 8;
            blo = t_u32x4{d0 & 0x000F000Fu, e0 & 0x000F000Fu, d1 & 0x000F000Fu, e1 & 0x000F000Fu};
            bhi = t_u32x4{d0 & 0x00F000F0u, e0 & 0x00F000F0u, d1 & 0x00F000F0u, e1 & 0x00F000F0u};
            q5_join<Q5>(blo, bhi, qhw, (uint32_t)sb);
        }
        const t_half8 bq = __builtin_bit_cast(t_half8, (sb & 1) ? bhi : blo);
        t_f32x4 D = {0, 0, 0, 0};
        D = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_cur.hi, bq, D, 0, 0, 0);
        if constexpr (!HL8) D = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_cur.lo, bq, D, 0, 0, 0);
        if (sb > 0) scale_in(sb - 1, D_prev);
        __builtin_amdgcn_sched_barrier(0);   // keeps the three stages of this step together
        D_prev = D;
        a_cur = a_next;
    }
    // bytes of mnA / mnB -> fp16 subnormals mn * 2^-24, element sb in position sb
    const t_u32x4 bm = {__builtin_amdgcn_perm(0u, mnA, 0x0c010c00u), __builtin_amdgcn_perm(0u, mnA, 0x0c030c02u),
                        __builtin_amdgcn_perm(0u, mnB, 0x0c010c00u), __builtin_amdgcn_perm(0u, mnB, 0x0c030c02u)};
    const t_half8 bmn = __builtin_bit_cast(t_half8, bm);
    t_f32x4 V = {0, 0, 0, 0};
    V = __builtin_amdgcn_mfma_f32_16x16x32_f16(vhi, bmn, V, 0, 0, 0);
    if constexpr (!HL8) V = __builtin_amdgcn_mfma_f32_16x16x32_f16(vlo, bmn, V, 0, 0, 0);
    scale_in(7, D_prev);
    // U carries 2^-24 from the subnormal nibbles and the token's scale s; V carries 2^-24 and s / 32
    const float4 inv = *(const float4*)(xinv_b + 4u * (lane >> 4));
    const float d24 = d * 16777216.0f, m24 = dmin * (16777216.0f * 32.0f);
    tot.x += inv.x * fmaf(d24, U.x, -(m24 * V.x));
    tot.y += inv.y * fmaf(d24, U.y, -(m24 * V.y));
    tot.z += inv.z * fmaf(d24, U.z, -(m24 * V.z));
    tot.w += inv.w * fmaf(d24, U.w, -(m24 * V.w));
}

// The same arithmetic with every operand read where it is used: fewer registers (the grouped kernel is held
// to 128 so that two of its workgroups share a CU).
template <bool Q5>
__device__ __forceinline__ void q4k_mtile_block_compact(const t_u32x4 hdr, const t_u32x2 (&w)[4], const t_u32x2 qhw,
                                                        const uint8_t* xa_b, const float* xs_b, const float* xinv_b, uint32_t lane,
                                                        t_f32x4& tot)
{
    const float d = half_bits_to_float(hdr.x & 0xFFFFu);
    const float dmin = half_bits_to_float(hdr.x >> 16);
    const uint32_t scA = hdr.y & 0x3F3F3F3Fu;
    const uint32_t mnA = hdr.z & 0x3F3F3F3Fu;
    const uint32_t scB = (hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u);
    const uint32_t mnB = ((hdr.w >> 4) & 0x0F0F0F0Fu) | ((hdr.z >> 2) & 0x30303030u);
    const uint32_t tq = lane >> 4;
    t_f32x4 U = {0, 0, 0, 0}, V = {0, 0, 0, 0};
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const uint32_t d0 = w[g].x, d1 = w[g].y;
        const uint32_t e0 = d0 >> 8, e1 = d1 >> 8;
        t_u32x4 blo = {d0 & 0x000F000Fu, e0 & 0x000F000Fu, d1 & 0x000F000Fu, e1 & 0x000F000Fu};
        t_u32x4 bhi = {d0 & 0x00F000F0u, e0 & 0x00F000F0u, d1 & 0x00F000F0u, e1 & 0x00F000F0u};
        q5_join<Q5>(blo, bhi, qhw, 2u * (uint32_t)g);
#pragma unroll
        for (int hn = 0; hn < 2; ++hn) {
            const int sb = 2 * g + hn;
            const uint8_t* ap = xa_b + (size_t)sb * MT_XA_PITCH + mt_xa_pos(lane & 15u, lane >> 4) * 16u;
            const t_half8 ahi = *(const t_half8*)ap;
            const t_half8 alo = *(const t_half8*)(ap + 1024);
            const t_half8 bq = __builtin_bit_cast(t_half8, hn ? bhi : blo);
            t_f32x4 D = {0, 0, 0, 0};
            D = __builtin_amdgcn_mfma_f32_16x16x32_f16(ahi, bq, D, 0, 0, 0);
            D = __builtin_amdgcn_mfma_f32_16x16x32_f16(alo, bq, D, 0, 0, 0);
            const uint32_t scw = sb < 4 ? scA : scB, mnw = sb < 4 ? mnA : mnB;
            // high nibbles sit four bits up: 1/16 goes into their scale
            const float sc = (float)((scw >> (8 * (sb & 3))) & 255u) * (hn ? 0.0625f : 1.0f);
            const float mn = (float)((mnw >> (8 * (sb & 3))) & 255u);
            const float4 xsum = *(const float4*)(xs_b + sb * 16 + 4u * tq);
            U.x = fmaf(sc, D.x, U.x); U.y = fmaf(sc, D.y, U.y); U.z = fmaf(sc, D.z, U.z); U.w = fmaf(sc, D.w, U.w);
            V.x = fmaf(mn, xsum.x, V.x); V.y = fmaf(mn, xsum.y, V.y); V.z = fmaf(mn, xsum.z, V.z); V.w = fmaf(mn, xsum.w, V.w);
        }
    }
    // D carries 2^-24 from the subnormal nibbles and the token's scale
    const float4 inv = *(const float4*)(xinv_b + 4u * tq);
    const float d24 = d * 16777216.0f;
    tot.x += fmaf(d24 * inv.x, U.x, -(dmin * V.x));
    tot.y += fmaf(d24 * inv.y, U.y, -(dmin * V.y));
    tot.z += fmaf(d24 * inv.z, U.z, -(dmin * V.z));
    tot.w += fmaf(d24 * inv.w, U.w, -(dmin * V.w));
}

// Q6_K: the weights of one superblock for one lane: 8 bytes of ql per (half, t&1), 8 of qh per half,
// the 16 scales and d.
struct Q6TileW {
    t_u32x2 ql[2][2], qh[2];
    t_u32x4 sc;
    uint32_t d;
};

__device__ __forceinline__ void q6k_mtile_load(const uint8_t* blk, uint32_t kq, Q6TileW& w)
{
    // blocks are 210 bytes: these loads are 2-byte aligned, which the hardware accepts
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        __builtin_memcpy(&w.ql[h][0], blk + 64u * h + 8u * kq, 8);
        __builtin_memcpy(&w.ql[h][1], blk + 64u * h + 32u + 8u * kq, 8);
        __builtin_memcpy(&w.qh[h], blk + 128u + 32u * h + 8u * kq, 8);
    }
    __builtin_memcpy(&w.sc, blk + 192u, 16);
    uint16_t d16;
    __builtin_memcpy(&d16, blk + 208u, 2);
    w.d = d16;
}

// The B operand of the product of a superblock's 16 scales with the staged sums of x per group of 16: lane
// (row, kq) holds the scales of groups 8 * (kq & 1) .. +7 (hi part of the sums for kq < 2, lo part above).  scu:
// the scale bytes with the sign bit flipped (s + 128); 0x6400 | (s + 128) is the fp16 1024 + 128 + s.
__device__ __forceinline__ t_half8 q6k_scale_operand(const t_u32x4 scu, uint32_t kq)
{
    const uint32_t a = (kq & 1u) ? scu.z : scu.x, b = (kq & 1u) ? scu.w : scu.y;
    const t_half2 off = {(_Float16)1152.0f, (_Float16)1152.0f};
    const t_half2 p0 = __builtin_bit_cast(t_half2, __builtin_amdgcn_perm(0x64646464u, a, 0x04010400u)) - off;
    const t_half2 p1 = __builtin_bit_cast(t_half2, __builtin_amdgcn_perm(0x64646464u, a, 0x04030402u)) - off;
    const t_half2 p2 = __builtin_bit_cast(t_half2, __builtin_amdgcn_perm(0x64646464u, b, 0x04010400u)) - off;
    const t_half2 p3 = __builtin_bit_cast(t_half2, __builtin_amdgcn_perm(0x64646464u, b, 0x04030402u)) - off;
    return t_half8{p0.x, p0.y, p1.x, p1.y, p2.x, p2.y, p3.x, p3.y};
}

// One superblock of one 16-row tile, Q6_K.  Lanes 0..31 (tq < 2) hold the sums over the first
// 16 elements of each run of 32 for tokens 4*tq .. +3, lanes 32..63 those over the second 16.  The -32 of the
// 6-bit values: 32 * d * sum over groups of scale * (sum of x over the group), one more matrix instruction
// (xv_b: those sums as an operand, in the slots of tq < 2 only).
__device__ __forceinline__ void q6k_mtile_block(const Q6TileW& w, const uint8_t* xa_b, const uint8_t* xv_b,
                                                const float* xinv_b, uint32_t lane, t_f32x4& tot)
{
    const uint32_t tq = lane >> 4, u = tq >> 1;
    const t_u32x4 scu = {w.sc.x ^ 0x80808080u, w.sc.y ^ 0x80808080u, w.sc.z ^ 0x80808080u, w.sc.w ^ 0x80808080u};
    // this lane's scales are the bytes 2t + u: moved down to the even bytes once
    const t_u32x4 scl = {scu.x >> (8u * u), scu.y >> (8u * u), scu.z >> (8u * u), scu.w >> (8u * u)};
    const t_half8 vx = *(const t_half8*)(xv_b + (size_t)lane * 16u);
    t_f32x4 V = {0, 0, 0, 0};
    V = __builtin_amdgcn_mfma_f32_16x16x32_f16(vx, q6k_scale_operand(scu, tq), V, 0, 0, 0);
    t_f32x4 U = {0, 0, 0, 0}, U16 = {0, 0, 0, 0};   // U16: the runs whose fields sit four bits up
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        t_u32x4 bq[4];   // B operands of runs t = 0..3 of this half
#pragma unroll
        for (int wd = 0; wd < 2; ++wd) {
            const uint32_t A = w.ql[h][0][wd], B = w.ql[h][1][wd], H = w.qh[h][wd];
            const uint32_t A8 = A >> 8, B8 = B >> 8;
            const uint32_t Hl4 = H << 4, Hl2 = H << 2, Hr4 = H >> 4, Hr6 = H >> 6;
            // pair a: bytes 0, 2; pair b: bytes 1, 3 of the word
            bq[0][2 * wd] = (A & 0x000F000Fu) | (Hl4 & 0x00300030u);
            bq[0][2 * wd + 1] = (A8 & 0x000F000Fu) | (Hr4 & 0x00300030u);
            bq[1][2 * wd] = (B & 0x000F000Fu) | (Hl2 & 0x00300030u);
            bq[1][2 * wd + 1] = (B8 & 0x000F000Fu) | (Hr6 & 0x00300030u);
            bq[2][2 * wd] = (A & 0x00F000F0u) | (Hl4 & 0x03000300u);
            bq[2][2 * wd + 1] = (A8 & 0x00F000F0u) | (Hr4 & 0x03000300u);
            bq[3][2 * wd] = (B & 0x00F000F0u) | (Hl2 & 0x03000300u);
            bq[3][2 * wd + 1] = (B8 & 0x00F000F0u) | (Hr6 & 0x03000300u);
        }
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int run = 4 * h + t;
            const uint8_t* ap = xa_b + (size_t)run * MT_XA_PITCH + mt_xa_pos(lane & 15u, lane >> 4) * 16u;
            const t_half8 ahi = *(const t_half8*)ap;
            const t_half8 alo = *(const t_half8*)(ap + 1024);
            const t_half8 b8 = __builtin_bit_cast(t_half8, bq[t]);
            t_f32x4 D = {0, 0, 0, 0};
            D = __builtin_amdgcn_mfma_f32_16x16x32_f16(ahi, b8, D, 0, 0, 0);
            D = __builtin_amdgcn_mfma_f32_16x16x32_f16(alo, b8, D, 0, 0, 0);
            // scale of (half h, t, 16-element half u): byte 8h + 2t + u of the 16, now byte 2t of its word
            const uint32_t word = scl[(8 * h + 2 * t) >> 2];
            const float sc = (float)((word >> (8 * ((2 * t) & 3))) & 255u) - 128.0f;
            if (t >= 2) { U16.x = fmaf(sc, D.x, U16.x); U16.y = fmaf(sc, D.y, U16.y); U16.z = fmaf(sc, D.z, U16.z); U16.w = fmaf(sc, D.w, U16.w); }
            else { U.x = fmaf(sc, D.x, U.x); U.y = fmaf(sc, D.y, U.y); U.z = fmaf(sc, D.z, U.z); U.w = fmaf(sc, D.w, U.w); }
        }
    }
    // U carries 2^-24 from the subnormal fields and the token's scale s; V carries s / 32
    const float4 inv = *(const float4*)(xinv_b + 4u * tq);
    const float d = half_bits_to_float(w.d);
    const float d24 = d * 16777216.0f, d1k = d * 1024.0f;
    tot.x += inv.x * fmaf(d24, fmaf(0.0625f, U16.x, U.x), -(d1k * V.x));
    tot.y += inv.y * fmaf(d24, fmaf(0.0625f, U16.y, U.y), -(d1k * V.y));
    tot.z += inv.z * fmaf(d24, fmaf(0.0625f, U16.z, U.z), -(d1k * V.z));
    tot.w += inv.w * fmaf(d24, fmaf(0.0625f, U16.w, U.w), -(d1k * V.w));
}

// Q6_K with 16 tokens: lane l holds tokens 4*(l/16) .. +3 of weight row l%16 as in the Q4_K kernel.  Every run of
// 32 elements is multiplied whole and with the second half of the weight operand zeroed (the lanes of k >= 16):
// D1 = sum over the first 16 elements, Dw - D1 = sum over the second, each with its own scale:
// sc1 * D1 + sc2 * (Dw - D1) = (sc1 - sc2) * D1 + sc2 * Dw.  xv_b: the sums of x per group of 16 as an operand.
__device__ __forceinline__ void q6k_mtile_block_wide(const Q6TileW& w, const uint8_t* xa_b, const uint8_t* xv_b,
                                                     const float* xinv_b, uint32_t lane, t_f32x4& tot)
{
    const uint32_t tq = lane >> 4;
    const uint32_t first = tq < 2u ? 0xFFFFFFFFu : 0u;   // this lane's k belong to the first half of a run
    const t_u32x4 scu = {w.sc.x ^ 0x80808080u, w.sc.y ^ 0x80808080u, w.sc.z ^ 0x80808080u, w.sc.w ^ 0x80808080u};
    const t_half8 vx = *(const t_half8*)(xv_b + (size_t)lane * 16u);
    t_f32x4 V = {0, 0, 0, 0};
    V = __builtin_amdgcn_mfma_f32_16x16x32_f16(vx, q6k_scale_operand(scu, tq), V, 0, 0, 0);
    t_f32x4 U = {0, 0, 0, 0}, U16 = {0, 0, 0, 0};   // U16: the runs whose fields sit four bits up
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        t_u32x4 bq[4];   // B operands of runs t = 0..3 of this half
#pragma unroll
        for (int wd = 0; wd < 2; ++wd) {
            const uint32_t A = w.ql[h][0][wd], B = w.ql[h][1][wd], H = w.qh[h][wd];
            const uint32_t A8 = A >> 8, B8 = B >> 8;
            const uint32_t Hl4 = H << 4, Hl2 = H << 2, Hr4 = H >> 4, Hr6 = H >> 6;
            bq[0][2 * wd] = (A & 0x000F000Fu) | (Hl4 & 0x00300030u);
            bq[0][2 * wd + 1] = (A8 & 0x000F000Fu) | (Hr4 & 0x00300030u);
            bq[1][2 * wd] = (B & 0x000F000Fu) | (Hl2 & 0x00300030u);
            bq[1][2 * wd + 1] = (B8 & 0x000F000Fu) | (Hr6 & 0x00300030u);
            bq[2][2 * wd] = (A & 0x00F000F0u) | (Hl4 & 0x03000300u);
            bq[2][2 * wd + 1] = (A8 & 0x00F000F0u) | (Hr4 & 0x03000300u);
            bq[3][2 * wd] = (B & 0x00F000F0u) | (Hl2 & 0x03000300u);
            bq[3][2 * wd + 1] = (B8 & 0x00F000F0u) | (Hr6 & 0x03000300u);
        }
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int run = 4 * h + t;
            const uint8_t* ap = xa_b + (size_t)run * MT_XA_PITCH + mt_xa_pos(lane & 15u, lane >> 4) * 16u;
            const t_half8 ahi = *(const t_half8*)ap;
            const t_half8 alo = *(const t_half8*)(ap + 1024);
            const t_u32x4 b1 = {bq[t].x & first, bq[t].y & first, bq[t].z & first, bq[t].w & first};
            const t_half8 bw8 = __builtin_bit_cast(t_half8, bq[t]);
            const t_half8 b18 = __builtin_bit_cast(t_half8, b1);
            t_f32x4 Dw = {0, 0, 0, 0}, D1 = {0, 0, 0, 0};
            Dw = __builtin_amdgcn_mfma_f32_16x16x32_f16(ahi, bw8, Dw, 0, 0, 0);
            D1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(ahi, b18, D1, 0, 0, 0);
            Dw = __builtin_amdgcn_mfma_f32_16x16x32_f16(alo, bw8, Dw, 0, 0, 0);
            D1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(alo, b18, D1, 0, 0, 0);
            // scales of (half h, t): bytes 8h + 2t (first 16 elements) and 8h + 2t + 1 of the 16; the 128 added to
            // both leaves their difference
            const uint32_t word = scu[(8 * h + 2 * t) >> 2];
            const int sh = 8 * ((2 * t) & 3);
            const float u1 = (float)((word >> sh) & 255u), u2 = (float)((word >> (sh + 8)) & 255u);
            const float s2 = u2 - 128.0f, s12 = u1 - u2;
            if (t >= 2) {
                U16.x = fmaf(s12, D1.x, fmaf(s2, Dw.x, U16.x)); U16.y = fmaf(s12, D1.y, fmaf(s2, Dw.y, U16.y));
                U16.z = fmaf(s12, D1.z, fmaf(s2, Dw.z, U16.z)); U16.w = fmaf(s12, D1.w, fmaf(s2, Dw.w, U16.w));
            } else {
                U.x = fmaf(s12, D1.x, fmaf(s2, Dw.x, U.x)); U.y = fmaf(s12, D1.y, fmaf(s2, Dw.y, U.y));
                U.z = fmaf(s12, D1.z, fmaf(s2, Dw.z, U.z)); U.w = fmaf(s12, D1.w, fmaf(s2, Dw.w, U.w));
            }
        }
    }
    const float4 inv = *(const float4*)(xinv_b + 4u * tq);
    const float d = half_bits_to_float(w.d);
    const float d24 = d * 16777216.0f, d1k = d * 1024.0f;
    tot.x += inv.x * fmaf(d24, fmaf(0.0625f, U16.x, U.x), -(d1k * V.x));
    tot.y += inv.y * fmaf(d24, fmaf(0.0625f, U16.y, U.y), -(d1k * V.y));
    tot.z += inv.z * fmaf(d24, fmaf(0.0625f, U16.z, U.z), -(d1k * V.z));
    tot.w += inv.w * fmaf(d24, fmaf(0.0625f, U16.w, U.w), -(d1k * V.w));
}

// Weights travel HBM -> registers -> LDS in 16-byte units that are consecutive along a row, so every cache
// line is fetched once and whole (a lane fetching only the 8-byte pieces its operands need makes each line
// cross the L2 -> L1 path five times).  A wave stages SPAN bytes of each of its 16 rows in a private LDS
// window (row pitch PITCH, chosen so that the 16 rows start in different banks) and then reads its operand
// pieces from there.
template <int SPAN, int PITCH>
struct MtileWStage {
    static constexpr int UPR = (SPAN + 15) / 16;            // units per row
    static constexpr int NU = (16 * UPR + 63) / 64;         // units per lane
    const uint8_t* base;        // the tile's first row (the same for all lanes)
    uint32_t src[NU];           // byte offset of the unit's row from there (16 rows: fits 32 bits)
    uint32_t dst[NU], col[NU];
    t_u32x4 raw[NU];
    __device__ __forceinline__ void init(const uint8_t* wmat, uint32_t row0, uint32_t N, uint32_t row_stride, uint32_t lane)
    {
        const uint32_t first = min(row0, N - 1u);
        base = wmat + (size_t)first * row_stride;
#pragma unroll
        for (int i = 0; i < NU; ++i) {
            const uint32_t u = min((uint32_t)i * 64u + lane, 16u * UPR - 1u);   // spare lanes repeat the last unit
            const uint32_t r = u / UPR, c = u - r * UPR;
            src[i] = (min(row0 + r, N - 1u) - first) * row_stride;
            col[i] = c * 16u;
            dst[i] = r * PITCH + c * 16u;
        }
    }
    // requests bytes [off, off + SPAN) of every row; a unit that would start at or beyond row_bytes reads
    // the row's last 16 bytes instead (it belongs to superblocks that do not exist and are not multiplied)
    __device__ __forceinline__ void load(uint32_t off, uint32_t row_bytes)
    {
#pragma unroll
        for (int i = 0; i < NU; ++i) {
            const uint32_t o = off + col[i];
            __builtin_memcpy(&raw[i], base + (src[i] + (o < row_bytes ? o : row_bytes - 16u)), 16);
        }
    }
    __device__ __forceinline__ void store(uint8_t* window) const
    {
#pragma unroll
        for (int i = 0; i < NU; ++i) *(t_u32x4*)(window + dst[i]) = raw[i];
    }
};

// STAGED: weights through the LDS windows described above (dense calls).  Grouped calls walk one or two
// chunks per workgroup and run thousands of workgroups: there the windows' LDS (one workgroup per CU instead
// of two) costs more than the line re-fetches, so they load each lane's pieces straight from global memory.
// (the grouped Q4_K kernel is held to 128 registers so that two of its workgroups share a CU)
// FUSED: residual and pair epilogue; PRO: the prologue (1 RMSNorm, 2 act(gate) * up)
template <int TYPE, int NW, int R, bool STAGED, int TOK, bool FUSED = false, int PRO = 0, bool HL8 = false, bool DUAL = false>
__device__ __forceinline__ void mtile_body(const MtileParams& p)
// (Q5_K: the Q4_K code with blocks of 176 bytes — header, 32 bytes of fifth bits, quants — and one more
// 8-byte piece per lane and superblock)
{
    static_assert(R == NW || R == 1, "a wave owns a tile, or all waves share one");
    extern __shared__ __align__(16) uint8_t smem[];
    uint8_t* xa = smem;
    float* xs = (float*)(smem + MT_XA_BYTES);
    float* xinv = xs + MT_XS_FLOATS;
    uint8_t* xv = (uint8_t*)(xinv + MT_INV_FLOATS);
    float* red = (float*)smem;   // reused after the last chunk

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // grouped mode: this workgroup's tokens are the pairs of one record, its weights one expert's rows
    const uint32_t* rec = nullptr;
    uint32_t count = p.M;
    const uint8_t* wmat = p.W;
    if (p.tiles) {
        if (blockIdx.y >= *p.n_tiles) return;   // whole workgroup
        rec = p.tiles + (size_t)blockIdx.y * p.tile_stride;
        // a record may hold more pairs than a pass of this kernel has token slots: blockIdx.z takes a slice
        const uint32_t slots = TYPE == KQ_TYPE_Q6_K ? 8u : 16u;   // (the 16-token Q6_K kernel has its own code: 16)
        const uint32_t first = blockIdx.z * slots;
        if (first >= rec[1]) return;            // whole workgroup
        count = min(rec[1] - first, slots);
        wmat += (size_t)rec[0] * p.N * p.row_stride_bytes;
        rec += first;                           // rec[2 + token] is now the slice's pair
    }
    static_assert(!FUSED || (R == NW && STAGED), "the fused forms come with a wave per tile, weights staged");
    static_assert(FUSED || PRO == 0, "prologues belong to the fused kernels");
    static_assert(!HL8 || (STAGED && (TYPE == KQ_TYPE_Q4_K || TYPE == KQ_TYPE_Q5_K)), "hi / lo slots: dense Q4_K / Q5_K");
    bool has_tile = R == 1 || wave < p.tiles_per_wg;
    uint32_t tile = R == 1 ? blockIdx.x : blockIdx.x * p.tiles_per_wg + wave;
    const bool pairs = FUSED && p.epi != 0;
    const uint32_t half_waves = p.tiles_per_wg >> 1;
    if (pairs) {
        // waves 0 .. h-1: gate tiles g*h .. +h-1; waves h .. 2h-1: the up tiles of the same outputs
        const uint32_t gate = blockIdx.x * half_waves + (wave < half_waves ? wave : wave - half_waves);
        has_tile = wave < p.tiles_per_wg && gate < p.pair_tile0;
        tile = wave < half_waves ? gate : p.pair_tile0 + gate;
    }
    const uint32_t row = has_tile ? tile * 16u + (lane & 15u) : p.N;
    const uint32_t kq = lane >> 4;

    // Q6: the block format; Q6S: the 8-token kernel whose tokens take two slots each; Q6W: the 16-token one
    constexpr bool Q6W = TYPE == MT_TYPE_Q6K_WIDE, Q6S = TYPE == KQ_TYPE_Q6_K, Q6 = Q6W || Q6S, Q5 = TYPE == KQ_TYPE_Q5_K;
    // lanes l and l + 32 hold two addends of the same outputs (Q6_K's 16-element halves, or hi and lo parts)
    constexpr bool HALVES = Q6S || HL8;
    constexpr uint32_t BB = Q6 ? KQ_Q6K_BYTES : Q5 ? KQ_Q5K_BYTES : KQ_Q4K_BYTES;
    constexpr uint32_t QOFF = Q5 ? 48u : 16u;   // where the quants start inside a block
    // A wave with a tile of its own stages two superblocks of its 16 rows at a time (two passes per chunk);
    // waves that share a tile stage the one superblock of the chunk that is theirs.
    constexpr int HB = R == 1 ? 1 : 2;                        // superblocks per staging pass
    constexpr int SPAN = HB * BB;
    constexpr int PITCH = Q6 ? (HB == 1 ? 240 : 464) : Q5 ? (HB == 1 ? 176 : 368) : (HB == 1 ? 160 : 304);
    constexpr int PASSES = R == 1 ? 1 : MT_KC / HB;
    using WStage = MtileWStage<SPAN, PITCH>;
    static_assert(PITCH >= WStage::UPR * 16 && PITCH % 16 == 0, "window row holds the staged units");
    uint8_t* wwin = smem + MT_STAGE_BYTES + wave * (16 * PITCH);
    const uint32_t row_bytes = p.n_blocks * BB;
    WStage ws[PASSES];
#pragma unroll
    for (int h = 0; h < PASSES; ++h) ws[h].init(wmat, has_tile ? tile * 16u : 0u, p.N, p.row_stride_bytes, lane);
    // first superblock of staging pass h of the chunk at c0
    auto pass_block = [&](uint32_t c0, int h) { return c0 + (R == 1 ? wave : (uint32_t)h * HB); };

    const uint32_t c_begin = (p.tiles ? 0u : blockIdx.z) * p.chunks_per_split * MT_KC;
    const uint32_t c_end = min(p.n_blocks, c_begin + p.chunks_per_split * MT_KC);

    MtileStager<64 * NW, Q6S, TOK, STAGED && !Q6, Q6W, PRO, HL8> stager;
    stager.init(p, rec, count);
    stager.fetch(p, c_begin);
    // norm prologue: the sums of squares per token are gathered while X is converted and meet here at the end
    // (16 floats behind the staging area); the outputs are scaled, not the activations
    float* rinv = (float*)(smem + MT_STAGE_BYTES + NW * (16 * PITCH));
    static_assert(!FUSED || (NW == 8 && TOK == 16), "a token's 32 converting threads are half a wave");
    // ... and the norm weights of a chunk (4 x 256 floats) are shared by all tokens: 256 threads bring them two
    // chunks ahead into registers and one chunk ahead into one of two LDS buffers behind the sums
    float* nwbuf = rinv + 16;
    float4 nwv = {0.0f, 0.0f, 0.0f, 0.0f};
    auto nw_fetch = [&](uint32_t c0) {
        if constexpr (PRO == 1) {
            if (threadIdx.x < 256u) {
                const uint32_t b = min(c0 + (threadIdx.x >> 6), p.n_blocks - 1u);
                nwv = *(const float4*)(p.norm_w + (size_t)b * KQ_QK + (threadIdx.x & 63u) * 4u);
            }
        }
    };
    auto nw_park = [&](uint32_t parity) {
        if constexpr (PRO == 1) {
            if (threadIdx.x < 256u) *(float4*)(nwbuf + parity * (MT_KC * KQ_QK) + threadIdx.x * 4u) = nwv;
        }
    };
    uint32_t nw_parity = 0;
    nw_fetch(c_begin);
    nw_park(0);
    nw_fetch(c_begin + MT_KC);
    t_f32x4 tot = {0, 0, 0, 0};
    // a finished tile: lane l holds tokens 4*(l/16) .. +3 of weight row row_t
    auto put_tile = [&](uint32_t row_t, const t_f32x4& t) {
        if (row_t < p.N && (!HALVES || kq < 2u)) {
            const float bias = p.bias ? p.bias[row_t] : 0.0f;
            const float t4[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const uint32_t token = 4u * kq + r;
                if (token < count) {
                    const uint32_t yrow = rec ? rec[2u + token] : token;
                    const size_t at = (size_t)yrow * p.ldy + p.y_offset + row_t;
                    float y = t4[r] + bias;
                    if constexpr (FUSED) {
                        if (p.residual) y += p.residual[at];
                    }
                    p.Y[at] = y;
                }
            }
        }
    };
    auto store_tile = [&](uint32_t row_t, t_f32x4 t) {
        if constexpr (HALVES) {   // lanes l and l + 32 hold two addends of the same tokens
            t.x += __shfl_xor(t.x, 32, 64);
            t.y += __shfl_xor(t.y, 32, 64);
            t.z += __shfl_xor(t.z, 32, 64);
            t.w += __shfl_xor(t.w, 32, 64);
        }
        put_tile(row_t, t);
    };
    if constexpr (STAGED) {
#pragma unroll
    for (int h = 0; h < PASSES; ++h) ws[h].load(pass_block(c_begin, h) * BB, row_bytes);
    // slots of tokens beyond M, and for Q6_K the halves that must read as zero, are cleared once
    for (uint32_t i = threadIdx.x; i < MT_STAGE_BYTES / 16; i += 64 * NW)
        ((t_u32x4*)smem)[i] = t_u32x4{0, 0, 0, 0};
    __syncthreads();

    // HL8 leaves the second plane of every operand pair unused: consecutive chunks alternate between the planes
    // (the token scales between xinv and the unused xs), so a chunk is parked while slower waves still multiply
    // the one before, and one barrier per chunk is enough.
    uint32_t plane = 0;
    for (uint32_t c0 = c_begin; c0 < c_end; c0 += MT_KC) {
        uint8_t* xa_c = xa + (HL8 ? plane * 1024u : 0u);
        uint8_t* xv_c = xv + (HL8 ? plane * 1024u : 0u);
        float* xinv_c = HL8 && plane ? xs : xinv;
        stager.prologue(p, c0 + stager.bb < c_end, nwbuf + nw_parity * (MT_KC * KQ_QK));
        stager.park(xa_c, xs, xinv_c, xv_c);
        nw_parity ^= 1u;
        nw_park(nw_parity);           // the next chunk's norm weights (this buffer was last read one barrier ago)
        ws[0].store(wwin);
        __syncthreads();
        // the next chunk of X and of the weights travels while this one is multiplied
        stager.fetch(p, c0 + MT_KC);
        nw_fetch(c0 + 2u * MT_KC);
        ws[0].load(pass_block(c0 + MT_KC, 0) * BB, row_bytes);
#pragma unroll
        for (int h = 0; h < PASSES; ++h) {
            if (h > 0) {
                wave_window_fence();          // this wave's reads of the previous pass are done
                ws[h].store(wwin);
                ws[h].load(pass_block(c0 + MT_KC, h) * BB, row_bytes);
                wave_window_fence();
            }
#pragma unroll
            for (int i = 0; i < HB; ++i) {
                const uint32_t bb = R == 1 ? wave : (uint32_t)(h * HB + i);
                if (has_tile && bb < MT_KC && c0 + bb < c_end) {
                    const uint8_t* blk = wwin + (lane & 15u) * PITCH + i * BB;
                    if constexpr (Q6) {
                        Q6TileW w6;
                        q6k_mtile_load(blk, kq, w6);
                        if constexpr (Q6W)
                            q6k_mtile_block_wide(w6, xa + (size_t)bb * (8 * MT_XA_PITCH), xv + (size_t)bb * 2048, xinv + bb * 16, lane, tot);
                        else
                            q6k_mtile_block(w6, xa + (size_t)bb * (8 * MT_XA_PITCH), xv + (size_t)bb * 2048, xinv + bb * 16, lane, tot);
                    } else {
                        const t_u32x4 hdr = *(const t_u32x4*)blk;
                        t_u32x2 w[4], qhw = {0, 0};
#pragma unroll
                        for (int g = 0; g < 4; ++g) w[g] = *(const t_u32x2*)(blk + QOFF + 32u * g + 8u * kq);
                        if constexpr (Q5) qhw = *(const t_u32x2*)(blk + 16u + 8u * kq);
                        q4k_mtile_block<Q5, HL8>(hdr, w, qhw, xa_c + (size_t)bb * (8 * MT_XA_PITCH), xv_c + (size_t)bb * 2048, xinv_c + bb * 16, lane, tot);
                    }
                }
            }
        }
        if constexpr (HL8) {
            plane ^= 1u;
            wave_window_fence();   // this wave's reads of its window are done before the next chunk is stored there
        } else {
            __syncthreads();
        }
    }
    } else {
    for (uint32_t i = threadIdx.x; i < MT_STAGE_BYTES / 16; i += 64 * NW)
        ((t_u32x4*)smem)[i] = t_u32x4{0, 0, 0, 0};
    __syncthreads();
    if constexpr (DUAL) {
        // Gate and up of a routed expert in one walk: a chunk of the record's X is converted once and multiplied
        // with the wave's tile of W, then with the same tile of W2; one set of weight registers, refilled block by
        // block with what is multiplied next (W2's blocks of this chunk, then W's of the next), and
        // silu(W x) * (W2 x) is what gets stored.
        static_assert(R == NW && !STAGED && !FUSED, "a grouped kernel, a wave per tile");
        constexpr int NBLK = MT_KC;
        const uint8_t* wrow_g = wmat + (size_t)min(row, p.N - 1u) * p.row_stride_bytes;
        const uint8_t* wrow_u = p.W2 + (wrow_g - p.W);
        t_u32x4 hdr[NBLK];
        t_u32x2 w[NBLK][4], qhw[NBLK];
        Q6TileW w6[NBLK];
        auto load_block = [&](const uint8_t* wrow, uint32_t c0, int i) {
            const uint8_t* blk = wrow + (size_t)min(c0 + (uint32_t)i, p.n_blocks - 1u) * BB;
            if constexpr (Q6) {
                q6k_mtile_load(blk, kq, w6[i]);
            } else {
                hdr[i] = *(const t_u32x4*)blk;
#pragma unroll
                for (int g = 0; g < 4; ++g) w[i][g] = *(const t_u32x2*)(blk + QOFF + 32u * g + 8u * kq);
                qhw[i] = t_u32x2{0, 0};
                if constexpr (Q5) qhw[i] = *(const t_u32x2*)(blk + 16u + 8u * kq);
            }
        };
        auto mul_block = [&](int i, t_f32x4& t) {
            if constexpr (Q6W)
                q6k_mtile_block_wide(w6[i], xa + (size_t)i * (8 * MT_XA_PITCH), xv + (size_t)i * 2048, xinv + i * 16, lane, t);
            else if constexpr (Q6)
                q6k_mtile_block(w6[i], xa + (size_t)i * (8 * MT_XA_PITCH), xv + (size_t)i * 2048, xinv + i * 16, lane, t);
            else
                q4k_mtile_block_compact<Q5>(hdr[i], w[i], qhw[i], xa + (size_t)i * (8 * MT_XA_PITCH), xs + i * 128, xinv + i * 16, lane, t);
        };
#pragma unroll
        for (int i = 0; i < NBLK; ++i) load_block(wrow_g, c_begin, i);
        t_f32x4 tot2 = {0, 0, 0, 0};
        for (uint32_t c0 = c_begin; c0 < c_end; c0 += MT_KC) {
            stager.park(xa, xs, xinv, xv);
            __syncthreads();
            if (c0 + MT_KC < c_end) stager.fetch(p, c0 + MT_KC);   // the next chunk of X travels while this one is multiplied
#pragma unroll
            for (int i = 0; i < NBLK; ++i) {
                if (has_tile && c0 + i < c_end) mul_block(i, tot);
                load_block(wrow_u, c0, i);
            }
#pragma unroll
            for (int i = 0; i < NBLK; ++i) {
                if (has_tile && c0 + i < c_end) mul_block(i, tot2);
                load_block(wrow_g, c0 + MT_KC, i);   // (past the end: the last block again, never multiplied)
            }
            __syncthreads();
        }
        if constexpr (HALVES) {   // lanes l and l + 32 hold two addends of the same tokens
            tot.x += __shfl_xor(tot.x, 32, 64); tot.y += __shfl_xor(tot.y, 32, 64);
            tot.z += __shfl_xor(tot.z, 32, 64); tot.w += __shfl_xor(tot.w, 32, 64);
            tot2.x += __shfl_xor(tot2.x, 32, 64); tot2.y += __shfl_xor(tot2.y, 32, 64);
            tot2.z += __shfl_xor(tot2.z, 32, 64); tot2.w += __shfl_xor(tot2.w, 32, 64);
        }
        if (row < p.N && (!HALVES || kq < 2u)) {
            const float g4[4] = {tot.x, tot.y, tot.z, tot.w}, u4[4] = {tot2.x, tot2.y, tot2.z, tot2.w};
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const uint32_t token = 4u * kq + r;
                if (token < count) {
                    const uint32_t yrow = rec ? rec[2u + token] : token;
                    // the formula of the separate activation kernel, so that the two ways agree to the bit
                    p.Y[(size_t)yrow * p.ldy + p.y_offset + row] = g4[r] / (expf(-g4[r]) + 1.0f) * u4[r];
                }
            }
        }
        return;
    }
    // A grouped call whose K fits one chunk stages the record's X once and lets every wave walk `iters` tiles
    // with it (no barrier after the first): such workgroups are otherwise mostly set-up.
    const uint32_t iters = (R == NW && p.tiles) ? p.tile_iters : 1u;
    constexpr int BPC = R == 1 ? (MT_KC + NW - 1) / NW : MT_KC;   // superblocks of a chunk this wave takes
    if constexpr (R == NW && Q6) {   // (the grouped Q4_K kernel is held to 128 registers: no room for this)
        if (iters > 1u) {
            // (iters is 2, 4 or 8.)  One set of weight registers, refilled block by block: as soon as a superblock
            // of tile it has been multiplied its registers are requested again for tile it + 1, so the loads of a
            // tile travel under the products of the blocks after them and of the next tile's blocks before them.
            // A second whole set (the next tile requested at once) took the kernel past 256 registers, to one
            // wave per SIMD; with this it keeps two workgroups on a CU.
            auto tile_row = [&](uint32_t it) {
                const uint32_t tile_i = (blockIdx.x * iters + it) * p.tiles_per_wg + wave;
                return has_tile ? tile_i * 16u + (lane & 15u) : p.N;
            };
            auto block_at = [&](uint32_t it, int i) {   // (past the last tile: that tile again, cache hits, never multiplied)
                const uint8_t* wrow = wmat + (size_t)min(tile_row(min(it, iters - 1u)), p.N - 1u) * p.row_stride_bytes;
                return wrow + (size_t)min(c_begin + (uint32_t)i, p.n_blocks - 1u) * BB;
            };
            const uint32_t nb = min(c_end - c_begin, (uint32_t)BPC);
            Q6TileW w6[BPC];
#pragma unroll
            for (int i = 0; i < BPC; ++i)
                if ((uint32_t)i < nb) q6k_mtile_load(block_at(0u, i), kq, w6[i]);
            stager.park(xa, xs, xinv, xv);
            __syncthreads();
            for (uint32_t it = 0; it < iters; ++it) {
                t_f32x4 tt = {0, 0, 0, 0};
#pragma unroll
                for (int i = 0; i < BPC; ++i) {
                    if ((uint32_t)i < nb) {
                        if (has_tile) {
                            if constexpr (Q6W)
                                q6k_mtile_block_wide(w6[i], xa + (size_t)i * (8 * MT_XA_PITCH), xv + (size_t)i * 2048, xinv + i * 16, lane, tt);
                            else
                                q6k_mtile_block(w6[i], xa + (size_t)i * (8 * MT_XA_PITCH), xv + (size_t)i * 2048, xinv + i * 16, lane, tt);
                        }
                        q6k_mtile_load(block_at(it + 1u, i), kq, w6[i]);
                    }
                }
                store_tile(tile_row(it), tt);
            }
            return;
        }
    }
    for (uint32_t it = 0; it < iters; ++it) {
    const uint32_t tile_i = iters > 1u ? (blockIdx.x * iters + it) * p.tiles_per_wg + wave : tile;
    const uint32_t row_i = has_tile ? tile_i * 16u + (lane & 15u) : p.N;
    if (iters > 1u) tot = t_f32x4{0, 0, 0, 0};
    const uint8_t* wrow = wmat + (size_t)min(row_i, p.N - 1u) * p.row_stride_bytes;
    for (uint32_t c0 = c_begin; c0 < c_end; c0 += MT_KC) {
        // the chunk's weights are requested first, so that their latency runs under the conversion of X
        t_u32x4 hdr[BPC];
        t_u32x2 w[BPC][4], qhw[BPC];
        Q6TileW w6[BPC];
#pragma unroll
        for (int i = 0; i < BPC; ++i) {
            const uint32_t bb = R == 1 ? wave + i * NW : i;
            const uint32_t b = min(c0 + bb, p.n_blocks - 1u);
            const uint8_t* blk = wrow + (size_t)b * BB;
            if constexpr (Q6) {
                q6k_mtile_load(blk, kq, w6[i]);
            } else {
                hdr[i] = *(const t_u32x4*)blk;
#pragma unroll
                for (int g = 0; g < 4; ++g) w[i][g] = *(const t_u32x2*)(blk + QOFF + 32u * g + 8u * kq);
                qhw[i] = t_u32x2{0, 0};
                if constexpr (Q5) qhw[i] = *(const t_u32x2*)(blk + 16u + 8u * kq);
            }
        }
        if (it == 0u) {
            stager.park(xa, xs, xinv, xv);
            __syncthreads();
            if (c0 + MT_KC < c_end) stager.fetch(p, c0 + MT_KC);   // the next chunk of X travels while this one is multiplied
        }
        if (has_tile) {
#pragma unroll
            for (int i = 0; i < BPC; ++i) {
                const uint32_t bb = R == 1 ? wave + i * NW : i;
                if (bb < MT_KC && c0 + bb < c_end) {
                    if constexpr (Q6W)
                        q6k_mtile_block_wide(w6[i], xa + (size_t)bb * (8 * MT_XA_PITCH), xv + (size_t)bb * 2048, xinv + bb * 16, lane, tot);
                    else if constexpr (Q6)
                        q6k_mtile_block(w6[i], xa + (size_t)bb * (8 * MT_XA_PITCH), xv + (size_t)bb * 2048, xinv + bb * 16, lane, tot);
                    else
                        q4k_mtile_block_compact<Q5>(hdr[i], w[i], qhw[i], xa + (size_t)bb * (8 * MT_XA_PITCH), xs + bb * 128, xinv + bb * 16, lane, tot);
                }
            }
        }
        if (iters == 1u) __syncthreads();   // (with iters > 1 there is one chunk and X stays where it is)
    }
    if (iters > 1u) store_tile(row_i, tot);
    }
    if (iters > 1u) return;
    }

    if (R == 1) {
        // fold the waves' partial tiles in wave order
        *(t_f32x4*)(red + (wave * 64u + lane) * 4u) = tot;
        __syncthreads();
        if (wave != 0) return;
#pragma unroll
        for (int w2 = 1; w2 < NW; ++w2) {
            const t_f32x4 o = *(const t_f32x4*)(red + (w2 * 64u + lane) * 4u);
            tot.x += o.x; tot.y += o.y; tot.z += o.z; tot.w += o.w;
        }
    }
    if constexpr (HALVES) {
        // lanes l and l + 32 hold the two addends of tokens 4*(l/16) .. +3: add them
        tot.x += __shfl_xor(tot.x, 32, 64);
        tot.y += __shfl_xor(tot.y, 32, 64);
        tot.z += __shfl_xor(tot.z, 32, 64);
        tot.w += __shfl_xor(tot.w, 32, 64);
    }
    constexpr bool normed = PRO == 1;
    if constexpr (PRO == 1) {
        if (normed) {
            // thread t converted for token t / 32: the sums of this workgroup's part of K, per token
            float ss = stager.ss;
            ss += group_partner<1>(ss); ss += group_partner<2>(ss); ss += group_partner<4>(ss);
            ss += group_partner<8>(ss);          // (DPP moves inside the row of 16 ...
            ss += __shfl_xor(ss, 16, 64);        //  ... and one exchange between the token's two rows)
            if ((threadIdx.x & 31u) == 0u) rinv[threadIdx.x >> 5] = ss;
            __syncthreads();
        }
    }
    if (R == NW && p.n_splits > 1) {   // (only the wave-per-tile kernels are launched with splits)
        // Same hand-over as the split GEMV: partial sums go out as agent-scope stores, the workgroup takes a
        // ticket once they are acknowledged, and the last one in reads all of them back past the
        // non-coherent cache levels and adds them in split order.
        const size_t plane = (size_t)gridDim.x * p.tiles_per_wg * 16u;   // rows of all tiles
        const bool mine = has_tile && (!HALVES || kq < 2u);
        const uint32_t prow = (blockIdx.x * p.tiles_per_wg + wave) * 16u + (lane & 15u);
        if (mine) {
            const float t4[4] = {tot.x, tot.y, tot.z, tot.w};
#pragma unroll
            for (int r = 0; r < 4; ++r)
                __hip_atomic_store(p.partial + ((size_t)blockIdx.z * 16u + 4u * kq + r) * plane + prow, t4[r], __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
        }
        // (norm prologue: the splits' sums of squares travel the same way, behind the partial tiles)
        float* ssq = p.partial + (size_t)p.n_splits * 16u * plane + (size_t)blockIdx.x * p.n_splits * 16u;
        if (normed && threadIdx.x < 16u)
            __hip_atomic_store(ssq + blockIdx.z * 16u + threadIdx.x, rinv[threadIdx.x], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        uint32_t* ticket = (uint32_t*)(smem + 16);
        if (threadIdx.x == 0)
            *ticket = __hip_atomic_fetch_add(&p.counters[blockIdx.x], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (*ticket != p.n_splits - 1u) return;   // whole workgroup
        if (mine) {
            // eight splits' partials are requested before the first is added (one round trip, not one per
            // split); the sums still run in split order
            float t4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            for (uint32_t z0 = 0; z0 < p.n_splits; z0 += 8u) {
                float v[8][4];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const uint32_t z = min(z0 + (uint32_t)j, p.n_splits - 1u);
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        v[j][r] = __hip_atomic_load(p.partial + ((size_t)z * 16u + 4u * kq + r) * plane + prow, __ATOMIC_RELAXED,
                                                    __HIP_MEMORY_SCOPE_AGENT);
                }
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    if (z0 + (uint32_t)j < p.n_splits) {
#pragma unroll
                        for (int r = 0; r < 4; ++r) t4[r] += v[j][r];
                    }
            }
            tot = t_f32x4{t4[0], t4[1], t4[2], t4[3]};
        }
        if (normed) {
            if (threadIdx.x < 16u) {
                float t = 0.0f;
                for (uint32_t z0 = 0; z0 < p.n_splits; z0 += 8u) {   // (as above: eight loads in flight, sums in split order)
                    float v[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        v[j] = __hip_atomic_load(ssq + min(z0 + (uint32_t)j, p.n_splits - 1u) * 16u + threadIdx.x, __ATOMIC_RELAXED,
                                                 __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        if (z0 + (uint32_t)j < p.n_splits) t += v[j];
                }
                rinv[threadIdx.x] = t;
            }
            __syncthreads();
        }
        if (threadIdx.x == 0) __hip_atomic_store(&p.counters[blockIdx.x], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if constexpr (PRO == 1) {
        if (normed) {
            const float4 q = *(const float4*)(rinv + 4u * kq);
            const float k1 = 1.0f / (float)p.K;
            tot.x *= 1.0f / sqrtf(fmaf(q.x, k1, p.eps)); tot.y *= 1.0f / sqrtf(fmaf(q.y, k1, p.eps));
            tot.z *= 1.0f / sqrtf(fmaf(q.z, k1, p.eps)); tot.w *= 1.0f / sqrtf(fmaf(q.w, k1, p.eps));
        }
    }
    if constexpr (FUSED) {
        if (pairs) {
            // the up waves hand their tiles (bias added) to the gate waves of the same outputs
            __syncthreads();   // the staging area is free
            const float b = (has_tile && p.bias) ? p.bias[row] : 0.0f;
            if (wave >= half_waves && wave < p.tiles_per_wg)
                *(t_f32x4*)(red + ((wave - half_waves) * 64u + lane) * 4u) = t_f32x4{tot.x + b, tot.y + b, tot.z + b, tot.w + b};
            __syncthreads();
            if (wave >= half_waves || !has_tile || (HALVES && kq >= 2u)) return;
            const t_f32x4 up = *(const t_f32x4*)(red + (wave * 64u + lane) * 4u);
            const float g4[4] = {tot.x + b, tot.y + b, tot.z + b, tot.w + b}, u4[4] = {up.x, up.y, up.z, up.w};
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const uint32_t token = 4u * kq + r;
                if (token < count)
                    p.Y[(size_t)token * p.ldy + p.y_offset + row] = p.epi == 2 ? mtile_act<2>(g4[r], u4[r]) : mtile_act<3>(g4[r], u4[r]);
            }
            return;
        }
    }
    put_tile(row, tot);
}

// Kernel entry.  What the first instructions need travels as scalars (KQ_KERNARG_PRELOAD: 14 dwords arrive in
// scalar registers with the wave), the rest as a struct that is fetched when it is used.
struct MtileRest {
    const float* bias;
    float* Y;
    uint32_t y_offset, ldy;
    float* partial;
    uint32_t* counters;
    int pro, epi;
    float eps;
    const float* norm_w;
    const float* residual;
    uint32_t pair_tile0;
    const uint32_t* n_tiles;
    uint32_t tile_iters, tile_stride, k_slots;
    int x_per_slot;
    const uint8_t* W2;
};

template <int TYPE, int NW, int R, bool STAGED, int TOK, bool FUSED = false, int PRO = 0, bool HL8 = false, bool DUAL = false>
__global__ __launch_bounds__(64 * NW, (!STAGED && TYPE == KQ_TYPE_Q4_K) ? 4 : (!STAGED && NW == 4) ? 2 : 1) void mtile_kernel(
    const uint8_t* W, const float* X, const uint32_t* tiles, uint32_t M, uint32_t N, uint32_t K, uint32_t n_blocks,
    uint32_t row_stride_bytes, uint32_t tiles_per_wg, uint32_t chunks_per_split, uint32_t n_splits, uint32_t x_stride,
    MtileRest r)
{
    MtileParams p;
    p.W2 = nullptr;
    p.X = X; p.W = W; p.bias = r.bias; p.Y = r.Y;
    p.M = M; p.N = N; p.K = K; p.n_blocks = n_blocks; p.row_stride_bytes = row_stride_bytes;
    p.y_offset = r.y_offset; p.ldy = r.ldy;
    p.tiles_per_wg = tiles_per_wg; p.n_splits = n_splits; p.chunks_per_split = chunks_per_split;
    p.partial = r.partial; p.counters = r.counters;
    p.pro = r.pro; p.epi = r.epi; p.eps = r.eps; p.norm_w = r.norm_w; p.residual = r.residual;
    p.x_stride = x_stride; p.pair_tile0 = r.pair_tile0;
    p.tiles = tiles; p.n_tiles = r.n_tiles; p.tile_iters = r.tile_iters; p.tile_stride = r.tile_stride;
    p.k_slots = r.k_slots; p.x_per_slot = r.x_per_slot; p.W2 = r.W2;
    mtile_body<TYPE, NW, R, STAGED, TOK, FUSED, PRO, HL8, DUAL>(p);
}

bool mtile_supported(const MatmulArgs& a)
{
    // dense calls of more than 16 tokens run as groups of 16 (8 for Q6_K), each reading the weights again:
    // meant for the few dozen tokens between a verify batch and a prefill, not for prefill itself (whose entry
    // point is the bf16 GEMM); any fp32 token count is served this way rather than by the generic kernel
    if (!a.expert_idx && (a.M < 1 || a.M > 65536u)) return false;   // grouped calls bring their tokens in records
    if (((uintptr_t)a.X & 15u)) return false;
    if (a.type == KQ_TYPE_Q4_K || a.type == KQ_TYPE_Q5_K) return !(((uintptr_t)a.W & 15u) || (a.row_stride_bytes & 15u));
    if (a.type == KQ_TYPE_Q6_K) return !(((uintptr_t)a.W & 1u) || (a.row_stride_bytes & 1u));
    return false;
}

template <int TYPE, int NW, int R, bool STAGED = true, int TOK = 16, bool FUSED = false, int PRO = 0, bool HL8 = false, bool DUAL = false>
static hipError_t launch_mtile_one(const MtileParams& p, uint32_t wgs, uint32_t wgs_y, hipStream_t s, uint32_t wgs_z = 1)
{
    constexpr bool Q6 = TYPE == KQ_TYPE_Q6_K || TYPE == MT_TYPE_Q6K_WIDE, Q5 = TYPE == KQ_TYPE_Q5_K;
    constexpr int PITCH = Q6 ? (R == 1 ? 240 : 464) : Q5 ? (R == 1 ? 176 : 368) : (R == 1 ? 160 : 304);   // as in the kernel
    // + the sums of squares per token and two chunks of norm weights
    constexpr size_t shmem = MT_STAGE_BYTES + (STAGED ? (size_t)NW * 16 * PITCH : 0) + (FUSED ? 64 : 0) +
                             (PRO == 1 ? 2 * MT_KC * KQ_QK * 4 : 0);
    auto kern = mtile_kernel<TYPE, NW, R, STAGED, TOK, FUSED, PRO, HL8, DUAL>;
    static bool raised = false;   // per instantiation
    if (!raised) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
        if (e != hipSuccess) return e;
        raised = true;
    }
    const MtileRest r{p.bias, p.Y, p.y_offset, p.ldy, p.partial, p.counters, p.pro, p.epi, p.eps, p.norm_w, p.residual,
                      p.pair_tile0, p.n_tiles, p.tile_iters, p.tile_stride, p.k_slots, p.x_per_slot, p.W2};
    hipLaunchKernelGGL(kern, dim3(wgs, wgs_y, wgs_z), dim3(64 * NW), shmem, s, p.W, p.X, p.tiles, p.M, p.N, p.K, p.n_blocks,
                       p.row_stride_bytes, p.tiles_per_wg, p.chunks_per_split, p.n_splits, p.x_stride, r);
    return hipGetLastError();
}

uint32_t mtile_group_cap(int) { return 16u; }

// The grouped call can take a twin matrix W2 (a.W2) and store silu(W x) * (W2 x): where K spans more than one chunk
// of four superblocks (a single chunk runs the form that walks several tiles per wave with X staged once).
bool mtile_grouped_dual_supported(const MatmulArgs& a)
{
    return mtile_supported(a) && a.n_blocks > (uint32_t)MT_KC && !(((uintptr_t)a.W2) & (a.type == KQ_TYPE_Q6_K ? 1u : 15u));
}

hipError_t launch_mtile_grouped(const MatmulArgs& a, const uint32_t* tiles, const uint32_t* n_tiles,
                                uint32_t tiles_bound, uint32_t cap, hipStream_t s)
{
    // records of up to cap pairs: Q6_K runs its 8-token kernel for records of up to 8, the 16-token one beyond
    const bool q6_wide = a.type == KQ_TYPE_Q6_K && cap > 8u;
    const uint32_t slices = 1;
    if (cap == 0 || cap > 16u || tiles_bound == 0 || tiles_bound > 65535u) return hipErrorInvalidValue;
    MtileParams p;
    p.W2 = nullptr;
    p.X = (const float*)a.X;
    p.W = a.W;
    p.bias = nullptr;
    p.Y = a.Y;
    p.M = cap; p.N = a.N; p.K = a.K;
    p.n_blocks = a.n_blocks;
    p.row_stride_bytes = a.row_stride_bytes;
    p.y_offset = 0;
    p.ldy = a.ldy;
    p.tiles = tiles;
    p.n_tiles = n_tiles;
    p.W2 = nullptr;
    p.tile_stride = 2u + cap;
    p.n_splits = 1; p.chunks_per_split = (a.n_blocks + MT_KC - 1) / MT_KC; p.partial = nullptr; p.counters = nullptr;
    p.k_slots = a.k_slots;
    p.x_per_slot = a.x_per_slot;
    p.pro = 0; p.epi = 0; p.eps = 0.0f; p.norm_w = nullptr; p.residual = nullptr; p.x_stride = a.K; p.pair_tile0 = 0;
    // a wave per 16-row tile of the expert, X of the record converted once per workgroup.  These workgroups walk
    // one or two chunks and are bound by their latencies, so two must share a CU: Q4_K runs 8 tiles per
    // workgroup at 128 registers, Q6_K (160 registers) 4 tiles per workgroup of 4 waves.
    const uint32_t row_tiles = (a.N + 15u) / 16u;
    const uint32_t tpw = a.type == KQ_TYPE_Q6_K ? 4u : 8u;
    p.tiles_per_wg = tpw;
    // one chunk of K: every wave walks up to 8 tiles with the record's X staged once, as long as a record
    // still spreads over four workgroups
    p.tile_iters = 1;
    if (p.chunks_per_split == 1u) {
        const uint32_t groups = (row_tiles + tpw - 1u) / tpw;
        p.tile_iters = groups >= 32u ? 8u : groups >= 16u ? 4u : groups >= 8u ? 2u : 1u;
        // ... and as long as the launch's workgroups fill whole rounds over the two a CU holds at once: the record
        // count is only known on the device, so it is estimated for pairs spread evenly over the experts, and a
        // workgroup is priced at 1.2 tiles for its conversion of X plus the tiles a wave walks.  (128 experts,
        // 2048 x 768: 2048 pairs are about 186 records; walking 8 tiles these are 744 workgroups on 512 places,
        // 115 us, walking 4 they are 1488, 103 us; 1024 pairs, 128 records, 512 workgroups: 8 tiles lead by 7 us.)
        if (a.tile_iters) p.tile_iters = min(p.tile_iters, a.tile_iters);
        else if (tiles_bound < a.M) {   // (the bound is pairs / cap + experts)
            const double records = moe_expected_records(a.M, tiles_bound - a.M / cap, cap);
            const double places = 2.0 * (double)device_cu_count();
            double best = 0.0;
            uint32_t best_iters = p.tile_iters;
            for (uint32_t it = p.tile_iters; it >= 1u; it >>= 1) {
                const double wg_per_record = (double)((groups + it - 1u) / it);
                // (a few workgroups more than a whole number of rounds do not make a round)
                const double cost = std::ceil(records * wg_per_record / places - 0.05) * (1.2 + (double)it);
                if (best == 0.0 || cost < best) { best = cost; best_iters = it; }
            }
            p.tile_iters = best_iters;
        }
    }
    const uint32_t wgs = (row_tiles + tpw * p.tile_iters - 1u) / (tpw * p.tile_iters);
    if (a.W2) {
        // gate and up in one walk, the activation in its store (several chunks of K: see mtile_grouped_dual_supported)
        if (!mtile_grouped_dual_supported(a)) return hipErrorInvalidValue;
        p.W2 = a.W2;
        if (q6_wide) return launch_mtile_one<MT_TYPE_Q6K_WIDE, 4, 4, false, 16, false, 0, false, true>(p, wgs, tiles_bound, s, slices);
        if (a.type == KQ_TYPE_Q6_K) return launch_mtile_one<KQ_TYPE_Q6_K, 4, 4, false, 16, false, 0, false, true>(p, wgs, tiles_bound, s, slices);
        if (a.type == KQ_TYPE_Q5_K) return launch_mtile_one<KQ_TYPE_Q5_K, 8, 8, false, 16, false, 0, false, true>(p, wgs, tiles_bound, s, slices);
        return launch_mtile_one<KQ_TYPE_Q4_K, 8, 8, false, 16, false, 0, false, true>(p, wgs, tiles_bound, s, slices);
    }
    if (q6_wide) return launch_mtile_one<MT_TYPE_Q6K_WIDE, 4, 4, false>(p, wgs, tiles_bound, s, slices);
    if (a.type == KQ_TYPE_Q6_K) return launch_mtile_one<KQ_TYPE_Q6_K, 4, 4, false>(p, wgs, tiles_bound, s, slices);
    if (a.type == KQ_TYPE_Q5_K) return launch_mtile_one<KQ_TYPE_Q5_K, 8, 8, false>(p, wgs, tiles_bound, s, slices);
    return launch_mtile_one<KQ_TYPE_Q4_K, 8, 8, false>(p, wgs, tiles_bound, s, slices);
}

hipError_t launch_mtile(const MatmulArgs& a, const SplitScratch& sc, hipStream_t s)
{
    const bool q6 = a.type == KQ_TYPE_Q6_K;
    // Q6_K: up to 8 tokens on the kernel whose tokens take two slots each, more on the 16-token kernel
    const bool q6_wide = q6 && a.M > 8u;
    const uint32_t group = 16u;
    const uint32_t tiles = (a.N + 15u) / 16u;
    const uint32_t n_chunks = (a.n_blocks + MT_KC - 1) / MT_KC;
    const uint32_t cus = device_cu_count();

    // Work split.  A wave per tile, tpw tiles per workgroup (they share the conversion of X), and K cut into
    // n_splits runs of whole chunks when the rows alone give too few workgroups.  Candidates are priced as
    // rounds x (chunks walked + 1.5 for launch, prologue and fold), a partly idle last round costing half its
    // idle share extra; one tile per workgroup with the waves taking different superblocks is the fallback
    // for matrices of a few rows.
    uint32_t best_tpw = 0, best_splits = 1, best_cps = n_chunks;
    float best_cost = 1e30f;
    for (uint32_t tpw = 8; tpw >= 4; --tpw) {
        const uint32_t groups = (tiles + tpw - 1u) / tpw;
        for (uint32_t splits = 1; splits <= n_chunks && splits <= 16u; ++splits) {
            const uint32_t cps = (n_chunks + splits - 1u) / splits;
            if ((splits - 1u) * cps >= n_chunks) continue;   // a split would be empty
            if (splits > 1u && ((size_t)splits * 16u * groups * tpw * 16u > sc.capacity_floats || groups > sc.n_counters)) continue;
            const uint32_t wgs = groups * splits, rounds = (wgs + cus - 1u) / cus;
            const float idle = 1.0f - (float)wgs / (float)(rounds * cus);
            const float cost = (float)rounds * ((float)cps + 1.5f) * (1.0f + 0.5f * idle);
            if (cost < best_cost) { best_cost = cost; best_tpw = tpw; best_splits = splits; best_cps = cps; }
        }
    }
    // one tile per workgroup of 4 waves, two workgroups per CU: every workgroup converts all of X itself
    const float shared_rounds = (float)((tiles + 2u * cus - 1u) / (2u * cus));
    const bool shared_tile = shared_rounds * ((float)n_chunks * 1.25f + 1.5f) < best_cost;

    for (uint32_t m0 = 0; m0 < a.M; m0 += group) {
        MtileParams p;
        p.W2 = nullptr;
        p.X = (const float*)a.X + (size_t)m0 * a.K;
        p.W = a.W;
        p.bias = a.bias;
        p.Y = a.Y + (size_t)m0 * a.ldy;
        p.M = a.M - m0 < group ? a.M - m0 : group;
        p.N = a.N; p.K = a.K;
        p.n_blocks = a.n_blocks;
        p.row_stride_bytes = a.row_stride_bytes;
        p.y_offset = a.y_offset;
        p.ldy = a.ldy;
        p.tiles_per_wg = 1;
        p.tiles = nullptr; p.n_tiles = nullptr; p.tile_stride = 0; p.tile_iters = 1; p.k_slots = 1; p.x_per_slot = 0;
        p.n_splits = 1; p.chunks_per_split = n_chunks; p.partial = sc.partial; p.counters = sc.counters;
        p.pro = 0; p.epi = 0; p.eps = 0.0f; p.norm_w = nullptr; p.residual = nullptr; p.x_stride = a.K; p.pair_tile0 = 0;
        hipError_t e;
        const bool q5 = a.type == KQ_TYPE_Q5_K;
        if (shared_tile) {
            e = q6_wide ? launch_mtile_one<MT_TYPE_Q6K_WIDE, 4, 1>(p, tiles, 1, s)
                : q6 ? launch_mtile_one<KQ_TYPE_Q6_K, 4, 1>(p, tiles, 1, s)
                : q5 ? launch_mtile_one<KQ_TYPE_Q5_K, 4, 1>(p, tiles, 1, s) : launch_mtile_one<KQ_TYPE_Q4_K, 4, 1>(p, tiles, 1, s);
        } else {
            p.tiles_per_wg = best_tpw;
            p.n_splits = best_splits;
            p.chunks_per_split = best_cps;
            const uint32_t wgs = (tiles + best_tpw - 1u) / best_tpw;
            // 5..8 tokens: the conversion of X is spread over twice the threads per (token, superblock), so
            // that all waves take part (measured +2-3 %; with 4 tokens or fewer the wider exchange costs more)
            // Q4_K / Q5_K with at most 8 tokens: hi and lo parts as token slots of one matrix instruction
            if (p.M > 4u && p.M <= 8u)
                e = q6 ? launch_mtile_one<KQ_TYPE_Q6_K, 8, 8, true, 8>(p, wgs, 1, s, best_splits)
                    : q5 ? launch_mtile_one<KQ_TYPE_Q5_K, 8, 8, true, 8, false, 0, true>(p, wgs, 1, s, best_splits)
                         : launch_mtile_one<KQ_TYPE_Q4_K, 8, 8, true, 8, false, 0, true>(p, wgs, 1, s, best_splits);
            else if (p.M <= 4u && !q6)
                e = q5 ? launch_mtile_one<KQ_TYPE_Q5_K, 8, 8, true, 16, false, 0, true>(p, wgs, 1, s, best_splits)
                       : launch_mtile_one<KQ_TYPE_Q4_K, 8, 8, true, 16, false, 0, true>(p, wgs, 1, s, best_splits);
            else
                e = q6_wide ? launch_mtile_one<MT_TYPE_Q6K_WIDE, 8, 8, true, 16>(p, wgs, 1, s, best_splits)
                    : q6 ? launch_mtile_one<KQ_TYPE_Q6_K, 8, 8, true, 16>(p, wgs, 1, s, best_splits)
                    : q5 ? launch_mtile_one<KQ_TYPE_Q5_K, 8, 8, true, 16>(p, wgs, 1, s, best_splits)
                         : launch_mtile_one<KQ_TYPE_Q4_K, 8, 8, true, 16>(p, wgs, 1, s, best_splits);
        }
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

// The fused forms of the decode matvec for verify batches (3..16 tokens; one or two as well where the
// lanes-along-K kernel declines): prologue in the conversion of X, residual in the store, act(gate) * up between
// the waves of a workgroup.  One launch, a wave per tile.
bool mtile_fused_supported(const MatmulArgs& a)
{
    if (a.expert_idx || a.M < 1 || a.M > 16 || !mtile_supported(a)) return false;
    if (a.pro == 1 && ((uintptr_t)a.norm_w & 15u)) return false;
    if (a.pro >= 2 && a.type == KQ_TYPE_Q6_K && a.M > 8u) return false;   // no registers for up beside 16 Q6_K token slots
    if (a.epi && (a.N & 31u)) return false;   // gate and up tiles of 16 rows each
    return true;
}

hipError_t launch_mtile_fused(const MatmulArgs& a, const SplitScratch& sc, hipStream_t s)
{
    const bool q6 = a.type == KQ_TYPE_Q6_K, q5 = a.type == KQ_TYPE_Q5_K, q6_wide = q6 && a.M > 8u;
    const uint32_t tiles = (a.N + 15u) / 16u;
    const uint32_t n_chunks = (a.n_blocks + MT_KC - 1) / MT_KC;
    const uint32_t cus = device_cu_count();
    // the work split of launch_mtile; pairs take an even number of tiles per workgroup
    uint32_t best_tpw = 8, best_splits = 1, best_cps = n_chunks;
    float best_cost = 1e30f;
    for (uint32_t tpw = 8; tpw >= 4; tpw -= a.epi ? 2u : 1u) {
        const uint32_t groups = a.epi ? (tiles / 2u + tpw / 2u - 1u) / (tpw / 2u) : (tiles + tpw - 1u) / tpw;
        for (uint32_t splits = 1; splits <= n_chunks && splits <= 16u; ++splits) {
            const uint32_t cps = (n_chunks + splits - 1u) / splits;
            if ((splits - 1u) * cps >= n_chunks) continue;   // a split would be empty
            // (partial tiles, then 16 sums of squares per workgroup for the norm prologue)
            if (splits > 1u && ((size_t)splits * 16u * groups * (tpw * 16u + 1u) > sc.capacity_floats || groups > sc.n_counters)) continue;
            const uint32_t wgs = groups * splits, rounds = (wgs + cus - 1u) / cus;
            const float idle = 1.0f - (float)wgs / (float)(rounds * cus);
            const float cost = (float)rounds * ((float)cps + 1.5f) * (1.0f + 0.5f * idle);
            if (cost < best_cost) { best_cost = cost; best_tpw = tpw; best_splits = splits; best_cps = cps; }
        }
    }
    MtileParams p;
    p.W2 = nullptr;
    p.X = (const float*)a.X;
    p.W = a.W;
    p.bias = a.bias;
    p.Y = a.Y;
    p.M = a.M; p.N = a.N; p.K = a.K;
    p.n_blocks = a.n_blocks;
    p.row_stride_bytes = a.row_stride_bytes;
    p.y_offset = a.y_offset;
    p.ldy = a.ldy;
    p.tiles_per_wg = best_tpw;
    p.tiles = nullptr; p.n_tiles = nullptr; p.tile_stride = 0; p.tile_iters = 1; p.k_slots = 1; p.x_per_slot = 0;
    p.n_splits = best_splits; p.chunks_per_split = best_cps; p.partial = sc.partial; p.counters = sc.counters;
    p.pro = a.pro; p.epi = a.epi; p.eps = a.eps; p.norm_w = a.norm_w; p.residual = a.residual;
    p.x_stride = a.pro >= 2 ? 2u * a.K : a.K;
    p.pair_tile0 = tiles / 2u;
    const uint32_t wgs = a.epi ? (tiles / 2u + best_tpw / 2u - 1u) / (best_tpw / 2u) : (tiles + best_tpw - 1u) / best_tpw;
    const bool hl8 = !q6 && a.M <= 8u;   // hi and lo parts as token slots of one matrix instruction
    if (a.pro == 1) {
        if (q6_wide) return launch_mtile_one<MT_TYPE_Q6K_WIDE, 8, 8, true, 16, true, 1>(p, wgs, 1, s, best_splits);
        if (q6) return launch_mtile_one<KQ_TYPE_Q6_K, 8, 8, true, 16, true, 1>(p, wgs, 1, s, best_splits);
        if (q5) return hl8 ? launch_mtile_one<KQ_TYPE_Q5_K, 8, 8, true, 16, true, 1, true>(p, wgs, 1, s, best_splits)
                           : launch_mtile_one<KQ_TYPE_Q5_K, 8, 8, true, 16, true, 1>(p, wgs, 1, s, best_splits);
        return hl8 ? launch_mtile_one<KQ_TYPE_Q4_K, 8, 8, true, 16, true, 1, true>(p, wgs, 1, s, best_splits)
                   : launch_mtile_one<KQ_TYPE_Q4_K, 8, 8, true, 16, true, 1>(p, wgs, 1, s, best_splits);
    }
    if (a.pro != 0) {
        // (the 16-slot Q6_K kernel has no registers for a second operand: mtile_fused_supported declines)
        if (q6) return launch_mtile_one<KQ_TYPE_Q6_K, 8, 8, true, 16, true, 2>(p, wgs, 1, s, best_splits);
        if (q5) return hl8 ? launch_mtile_one<KQ_TYPE_Q5_K, 8, 8, true, 16, true, 2, true>(p, wgs, 1, s, best_splits)
                           : launch_mtile_one<KQ_TYPE_Q5_K, 8, 8, true, 16, true, 2>(p, wgs, 1, s, best_splits);
        return hl8 ? launch_mtile_one<KQ_TYPE_Q4_K, 8, 8, true, 16, true, 2, true>(p, wgs, 1, s, best_splits)
                   : launch_mtile_one<KQ_TYPE_Q4_K, 8, 8, true, 16, true, 2>(p, wgs, 1, s, best_splits);
    }
    if (q6_wide) return launch_mtile_one<MT_TYPE_Q6K_WIDE, 8, 8, true, 16, true>(p, wgs, 1, s, best_splits);
    if (q6) return launch_mtile_one<KQ_TYPE_Q6_K, 8, 8, true, 16, true>(p, wgs, 1, s, best_splits);
    if (q5) return hl8 ? launch_mtile_one<KQ_TYPE_Q5_K, 8, 8, true, 16, true, 0, true>(p, wgs, 1, s, best_splits)
                       : launch_mtile_one<KQ_TYPE_Q5_K, 8, 8, true, 16, true>(p, wgs, 1, s, best_splits);
    return hl8 ? launch_mtile_one<KQ_TYPE_Q4_K, 8, 8, true, 16, true, 0, true>(p, wgs, 1, s, best_splits)
               : launch_mtile_one<KQ_TYPE_Q4_K, 8, 8, true, 16, true>(p, wgs, 1, s, best_splits);
}

}  // namespace kq
