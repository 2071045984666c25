// kq_mrow.hip — fused dequant-matvec for M = 1..16 on the matrix cores, one weight
// row per lane.  Serves decode (M = 1), speculative verify (M = 2..16) and, in
// grouped mode, the MoE expert matvec over ragged token lists.
//
// Weights.  As in the row-per-lane scheme, a wave copies the bytes of one
// superblock column of 64 rows HBM -> VGPR -> LDS with coalesced 128-bit loads
// and each lane reads its own row back.  A masked 4- or 6-bit field left in the
// low mantissa bits of an fp16 lane is the subnormal q*2^-24 (q*2^-20 four bits
// up): the matrix cores multiply subnormals exactly, so five bit-ops turn one
// 32-bit word into the B operands of two v_mfma_f32_4x4x4_16B_f16.
//
// Activations.  That MFMA computes 16 independent 4x4x4 products; lane 4b+j holds
// column j of block b.  With B = weights, lane = row, and the A operand taken
// from block 0 and broadcast to all 16 blocks (CBSZ = 4), one instruction
// multiplies 64 rows x 4 k by 4 activation "slots".  A token of fp32 X occupies
// two slots: hi = fp16(x*s), lo = fp16(x*s - hi) with s a power of two chosen per
// 256-element block so the largest element sits just below 2^15 — 22 bits of x,
// no overflow, no reduction across lanes.  Each wave converts the X of its own
// superblock (64 lanes x 4 elements) and parks it in LDS in operand order; only
// lanes 0..3 read it back.
//
// Scales.  Every 32-element sub-block has its own accumulator chain; its sum is
// multiplied by the 6-bit scale (Q4_K) / int8 scale (Q6_K) in fp32, the block
// scale d, and the power of two.  Q4_K minima and the Q6_K -32 offset are
// applied against sums of x computed while staging.
//
// Workgroups, K split and the cross-workgroup fold are those of kq_gemv.hip.
#include "kq_format.h"
#include "kq_kernels.h"

namespace kq {

typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr float M_TWO24 = 16777216.0f;
constexpr float M_TWO20 = 1048576.0f;
constexpr int Q6W_PIECES = 14;    // 224-byte window per row
constexpr int Q6W_LDS_ROW = 240;  // odd multiple of 16 bytes

struct MrowParams {
    const float* X;
    const uint8_t* W;
    const float* bias;
    float* Y;
    uint32_t M, N, K, n_blocks, row_stride_bytes, y_offset, ldy;
    uint32_t blocks_per_split, n_splits;
    float* partial;
    uint32_t* counters;
    // grouped mode (tiles != nullptr): blockIdx.z walks tiles of up to 2*SETS
    // (token, slot) pairs that share an expert; tile t = {expert, count, pairs...}
    const uint32_t* tiles;
    const uint32_t* n_tiles;
    uint32_t tile_stride;   // words per tile record
    uint32_t k_slots;
    int x_per_slot;
};

__device__ __forceinline__ void mrow_lds_fence()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

template <int CTRL>
__device__ __forceinline__ float dpp_f(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

// butterflies inside a row of 16 lanes: quad xor 1, xor 2, half-row mirror, row mirror
__device__ __forceinline__ float sum4(float v) { v += dpp_f<0xB1>(v); v += dpp_f<0x4E>(v); return v; }
__device__ __forceinline__ float sum8(float v) { v = sum4(v); v += dpp_f<0x141>(v); return v; }

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u(uint32_t v)
{
    return (uint32_t)__builtin_amdgcn_mov_dpp((int)v, CTRL, 0xF, 0xF, true);
}

// Largest bit pattern of a non-negative float across the wave (orders like the
// floats themselves, and needs no NaN canonicalisation).  Uniform result.
__device__ __forceinline__ uint32_t wave_max_bits(uint32_t v)
{
    v = max(v, dpp_u<0xB1>(v));
    v = max(v, dpp_u<0x4E>(v));
    v = max(v, dpp_u<0x141>(v));
    v = max(v, dpp_u<0x140>(v));
    const uint32_t a = (uint32_t)__builtin_amdgcn_readlane((int)v, 0);
    const uint32_t b = (uint32_t)__builtin_amdgcn_readlane((int)v, 16);
    const uint32_t c = (uint32_t)__builtin_amdgcn_readlane((int)v, 32);
    const uint32_t d = (uint32_t)__builtin_amdgcn_readlane((int)v, 48);
    return max(max(a, b), max(c, d));
}

// Converts this lane's four consecutive activations of one token into the hi/lo
// fp16 A-operand words and writes them, plus the sub-block sums, to LDS.
//   xa:  [64 records][4 slots][16 bytes]; record = 4 consecutive k; the 16 bytes
//        of a slot hold the operand for MFMA "phase" 0 and 1 (see callers)
//   returns the power of two that undoes the scaling
template <int SEG>
__device__ __forceinline__ float stage_token(const float4 x, uint32_t lane, uint32_t rec, uint32_t phase,
                                             uint32_t slot_hi, uint8_t* xa, float* xs)
{
    const uint32_t m01 = max(__builtin_bit_cast(uint32_t, x.x) & 0x7FFFFFFFu, __builtin_bit_cast(uint32_t, x.y) & 0x7FFFFFFFu);
    const uint32_t m23 = max(__builtin_bit_cast(uint32_t, x.z) & 0x7FFFFFFFu, __builtin_bit_cast(uint32_t, x.w) & 0x7FFFFFFFu);
    uint32_t e = wave_max_bits(max(m01, m23)) >> 23;          // biased exponent of the largest |x|
    e = e < 15u ? 15u : e;
    const float s = __builtin_bit_cast(float, (268u - e) << 23);      // 2^(141-e): amax*s in [2^14, 2^15)
    const float inv = __builtin_bit_cast(float, (e - 14u) << 23);     // 2^(e-141)
    const float a0 = x.x * s, a1 = x.y * s, a2 = x.z * s, a3 = x.w * s;
    // operand order along k is (0, 2, 1, 3): the weight unpack yields bytes 0,2 then 1,3
    const half2_t h02 = {(_Float16)a0, (_Float16)a2};
    const half2_t h13 = {(_Float16)a1, (_Float16)a3};
    const half2_t l02 = {(_Float16)(a0 - (float)h02.x), (_Float16)(a2 - (float)h02.y)};
    const half2_t l13 = {(_Float16)(a1 - (float)h13.x), (_Float16)(a3 - (float)h13.y)};
    uint8_t* dst = xa + (rec * 4u + slot_hi) * 16u + phase * 8u;
    *(u32x2*)dst = u32x2{__builtin_bit_cast(uint32_t, h02), __builtin_bit_cast(uint32_t, h13)};
    *(u32x2*)(dst + 16) = u32x2{__builtin_bit_cast(uint32_t, l02), __builtin_bit_cast(uint32_t, l13)};
    // sums of the unscaled x over aligned runs of SEG elements
    const float part = (x.x + x.y) + (x.z + x.w);
    const float tot = SEG == 32 ? sum8(part) : sum4(part);
    constexpr uint32_t LPS = SEG / 4;
    if ((lane % LPS) == 0) xs[lane / LPS] = tot;
    return inv;
}

// ---------------------------------------------------------------------------
template <int TYPE, int SETS, int NW>
__global__ __launch_bounds__(64 * NW) void mrow_kernel(MrowParams p)
{
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr int MT = 2 * SETS;                                   // tokens per pass
    constexpr int BB = TYPE == KQ_TYPE_Q4_K ? KQ_Q4K_BYTES : KQ_Q6K_BYTES;
    constexpr int NPIECE = TYPE == KQ_TYPE_Q4_K ? 9 : Q6W_PIECES;
    constexpr int LROW = TYPE == KQ_TYPE_Q4_K ? KQ_Q4K_BYTES : Q6W_LDS_ROW;
    constexpr int SEG = TYPE == KQ_TYPE_Q4_K ? 32 : 16;
    constexpr int NSEG = 256 / SEG;
    constexpr int TILE = 64 * LROW;
    constexpr int XA = SETS * 4096;                                // 64 records x 4 slots x 16 B per set
    constexpr int XS = MT * NSEG * 4;
    constexpr int WAVE_LDS = TILE + XA + XS;

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t row0 = blockIdx.x * 64u;
    const uint32_t b_begin = blockIdx.y * p.blocks_per_split;
    const uint32_t b_end = min(p.n_blocks, b_begin + p.blocks_per_split);

    uint8_t* tile = smem + wave * WAVE_LDS;
    uint8_t* xa = tile + TILE;
    float* xs = (float*)(xa + XA);
    float* red = (float*)smem;

    // ---- which rows of X, Y and W this workgroup works on
    const uint8_t* wmat = p.W;
    const float* xrow[MT];
    float* yrow[MT];
    uint32_t count = p.M;
    if (p.tiles) {
        if (blockIdx.z >= *p.n_tiles) return;
        const uint32_t* t = p.tiles + (size_t)blockIdx.z * p.tile_stride;
        const uint32_t expert = t[0];
        count = t[1];
        wmat += (size_t)expert * p.N * p.row_stride_bytes;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const uint32_t pair = t[2 + ((uint32_t)m < count ? m : 0)];
            xrow[m] = p.X + (size_t)(p.x_per_slot ? pair : pair / p.k_slots) * p.K;
            yrow[m] = p.Y + (size_t)pair * p.ldy;
        }
    } else {
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const uint32_t mm = (uint32_t)m < count ? m : 0;
            xrow[m] = p.X + (size_t)mm * p.K;
            yrow[m] = p.Y + (size_t)mm * p.ldy + p.y_offset;
        }
    }

    // ---- weight pieces: piece i*64+lane -> (row r, 16-byte segment s)
    uint32_t goff[NPIECE], loff[NPIECE];
#pragma unroll
    for (int i = 0; i < NPIECE; ++i) {
        const uint32_t pc = i * 64u + lane;
        const uint32_t r = pc / NPIECE, s = pc - r * NPIECE;
        const uint32_t row = min(row0 + r, p.N - 1u);
        goff[i] = (row - row0) * p.row_stride_bytes + s * 16u;
        loff[i] = r * LROW + s * 16u;
    }
    const uint8_t* wbase = wmat + (size_t)row0 * p.row_stride_bytes;
    // Q6_K: the 224-byte window starts at the block (even b), 14 bytes before it
    // (odd b), or 12 bytes before it (even b closing a row with an odd block count)
    const uint32_t last_even = (p.n_blocks & 1u) ? p.n_blocks - 1u : 0xFFFFFFFFu;
    auto wofs = [&](uint32_t b) -> size_t {
        if (TYPE == KQ_TYPE_Q4_K) return (size_t)b * BB;
        return (size_t)b * BB - ((b & 1u) ? 14u : (b == last_even ? 12u : 0u));
    };

    float acc[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[m] = 0.0f;

    // Two superblocks per wave are in flight at any time (register double buffer).
    u32x4 v0[NPIECE], v1[NPIECE];
    float4 xv0[MT], xv1[MT];
    auto prefetch = [&](u32x4 (&v)[NPIECE], float4 (&xv)[MT], uint32_t b) {
#pragma unroll
        for (int i = 0; i < NPIECE; ++i)
            v[i] = __builtin_nontemporal_load((const u32x4*)(wbase + goff[i] + wofs(b)));
#pragma unroll
        for (int m = 0; m < MT; ++m) xv[m] = ((const float4*)(xrow[m] + (size_t)b * KQ_QK))[lane];
    };

    auto step = [&](u32x4 (&v)[NPIECE], float4 (&xv)[MT], uint32_t b) {
        // ---- park weights and activations of this superblock in LDS
#pragma unroll
        for (int i = 0; i < NPIECE; ++i) *(u32x4*)(tile + loff[i]) = v[i];
        float inv[MT];
        {
            // lane holds k = 4*lane .. 4*lane+3 of the block
            uint32_t rec, phase;
            if (TYPE == KQ_TYPE_Q4_K) {
                // sub-block sb = lane/8, word w = lane%8: record (sb/2)*8 + w, phase = sb&1
                rec = (lane >> 4) * 8u + (lane & 7u);
                phase = (lane >> 3) & 1u;
            } else {
                // element 128h + 32t + 4u: h = lane/32, t = (lane/8)%4, u = lane%8:
                // record (h*8 + u)*2 + t/2, phase = t&1
                rec = ((lane >> 5) * 8u + (lane & 7u)) * 2u + ((lane >> 4) & 1u);
                phase = (lane >> 3) & 1u;
            }
#pragma unroll
            for (int m = 0; m < MT; ++m)
                inv[m] = stage_token<SEG>(xv[m], lane, rec, phase, (m & 1) * 2, xa + (m >> 1) * 4096, xs + m * NSEG);
        }
        const uint32_t bn = b + 2 * NW;
        if (bn < b_end) prefetch(v, xv, bn);
        mrow_lds_fence();

        // ---- this lane's row
        const uint8_t* mine = tile + lane * LROW;
        float d;

        if (TYPE == KQ_TYPE_Q4_K) {
            const u32x4 hdr = *(const u32x4*)mine;
            d = half_bits_to_float(hdr.x & 0xFFFFu);
            const float dmin = half_bits_to_float(hdr.x >> 16);
            const uint32_t scA = hdr.y & 0x3F3F3F3Fu;
            const uint32_t mnA = hdr.z & 0x3F3F3F3Fu;
            const uint32_t scB = (hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u);
            const uint32_t mnB = ((hdr.w >> 4) & 0x0F0F0F0Fu) | ((hdr.z >> 2) & 0x30303030u);
            f32x4 sE[SETS], sO[SETS];
#pragma unroll
            for (int s = 0; s < SETS; ++s) { sE[s] = f32x4{0, 0, 0, 0}; sO[s] = f32x4{0, 0, 0, 0}; }
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                f32x4 dE[SETS], dO[SETS];
#pragma unroll
                for (int s = 0; s < SETS; ++s) { dE[s] = f32x4{0, 0, 0, 0}; dO[s] = f32x4{0, 0, 0, 0}; }
                const u32x4 q0 = *(const u32x4*)(mine + 16 + g * 32);
                const u32x4 q1 = *(const u32x4*)(mine + 32 + g * 32);
                const uint32_t wds[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
                // A operands of WB words at a time, fetched by lanes 0..3 only
                constexpr int WB = SETS == 1 ? 4 : SETS <= 4 ? 2 : 1;
#pragma unroll
                for (int w0 = 0; w0 < 8; w0 += WB) {
                    u32x4 aop[WB][SETS];
#pragma unroll
                    for (int i = 0; i < WB; ++i)
#pragma unroll
                        for (int s = 0; s < SETS; ++s) aop[i][s] = __builtin_nondeterministic_value(aop[i][s]);
                    if (lane < 4) {
#pragma unroll
                        for (int i = 0; i < WB; ++i)
#pragma unroll
                            for (int s = 0; s < SETS; ++s)
                                aop[i][s] = *(const u32x4*)(xa + s * 4096 + ((g * 8 + w0 + i) * 4 + lane) * 16);
                    }
#pragma unroll
                    for (int i = 0; i < WB; ++i) {
                        const uint32_t wv = wds[w0 + i], t8 = wv >> 8;
                        const u32x2 bE = {wv & 0x000F000Fu, t8 & 0x000F000Fu};
                        const u32x2 bO = {wv & 0x00F000F0u, t8 & 0x00F000F0u};
#pragma unroll
                        for (int s = 0; s < SETS; ++s) {
                            const half4_t aE = __builtin_bit_cast(half4_t, u32x2{aop[i][s].x, aop[i][s].y});
                            const half4_t aO = __builtin_bit_cast(half4_t, u32x2{aop[i][s].z, aop[i][s].w});
                            dE[s] = __builtin_amdgcn_mfma_f32_4x4x4f16(aE, __builtin_bit_cast(half4_t, bE), dE[s], 4, 0, 0);
                            dO[s] = __builtin_amdgcn_mfma_f32_4x4x4f16(aO, __builtin_bit_cast(half4_t, bO), dO[s], 4, 0, 0);
                        }
                    }
                }
                const uint32_t scw = g < 2 ? scA : scB;
                const float scE = (float)((scw >> (8 * ((2 * g) & 3))) & 255u);
                const float scO = (float)((scw >> (8 * ((2 * g + 1) & 3))) & 255u);
#pragma unroll
                for (int s = 0; s < SETS; ++s) {
                    sE[s] += scE * dE[s];
                    sO[s] += scO * dO[s];
                }
            }
            // minima: sum_sb mn_sb * sum(x over sb)
            float mnf[8];
#pragma unroll
            for (int sb = 0; sb < 8; ++sb) mnf[sb] = (float)(((sb < 4 ? mnA : mnB) >> (8 * (sb & 3))) & 255u);
#pragma unroll
            for (int m = 0; m < MT; ++m) {
                const f32x4 e = sE[m >> 1], o = sO[m >> 1];
                const int h = (m & 1) * 2;
                const float body = fmaf(e[h] + e[h + 1], M_TWO24, (o[h] + o[h + 1]) * M_TWO20) * inv[m];
                float ms = 0.0f;
#pragma unroll
                for (int sb = 0; sb < 8; ++sb) ms = fmaf(mnf[sb], xs[m * NSEG + sb], ms);
                acc[m] = fmaf(d, body, acc[m]);
                acc[m] = fmaf(-dmin, ms, acc[m]);
            }
        } else {
            // 53 words of the block; odd blocks sit 14 bytes into the window
            // (2 bytes off a word), the closing even block of an odd row 12 bytes
            const uint32_t shift = (b & 1u) ? 14u : (b == last_even ? 12u : 0u);
            uint32_t wq[53];
            {
                u32x4 raw[Q6W_PIECES];
#pragma unroll
                for (int s = 0; s < Q6W_PIECES; ++s) raw[s] = *(const u32x4*)(mine + s * 16);
                if (shift == 14u) {
#pragma unroll
                    for (int j = 0; j < 53; ++j) {
                        const int lo = 3 + j, hi = 4 + j;
                        const uint32_t wl = raw[lo >> 2][lo & 3];
                        const uint32_t wh = hi < 56 ? raw[hi >> 2][hi & 3] : 0u;
                        wq[j] = __builtin_amdgcn_alignbit(wh, wl, 16);
                    }
                } else if (shift == 12u) {
#pragma unroll
                    for (int j = 0; j < 53; ++j) wq[j] = raw[(j + 3) >> 2][(j + 3) & 3];
                } else {
#pragma unroll
                    for (int j = 0; j < 53; ++j) wq[j] = raw[j >> 2][j & 3];
                }
            }
            d = half_bits_to_float(wq[52] & 0xFFFFu);
            float tot[MT];
#pragma unroll
            for (int m = 0; m < MT; ++m) tot[m] = 0.0f;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
#pragma unroll
                for (int uq = 0; uq < 2; ++uq) {
                    f32x4 dd[4][SETS];
#pragma unroll
                    for (int t = 0; t < 4; ++t)
#pragma unroll
                        for (int s = 0; s < SETS; ++s) dd[t][s] = f32x4{0, 0, 0, 0};
#pragma unroll
                    for (int uu = 0; uu < 4; ++uu) {
                        const int u = uq * 4 + uu;
                        const uint32_t A = wq[16 * h + u], B = wq[16 * h + 8 + u], H = wq[32 + 8 * h + u];
                        const uint32_t A8 = A >> 8, B8 = B >> 8;
                        const uint32_t Hl4 = H << 4, Hl2 = H << 2, Hr4 = H >> 4, Hr6 = H >> 6;
                        u32x2 bq[4];
                        bq[0] = u32x2{(A & 0x000F000Fu) | (Hl4 & 0x00300030u), (A8 & 0x000F000Fu) | (Hr4 & 0x00300030u)};
                        bq[1] = u32x2{(B & 0x000F000Fu) | (Hl2 & 0x00300030u), (B8 & 0x000F000Fu) | (Hr6 & 0x00300030u)};
                        bq[2] = u32x2{(A & 0x00F000F0u) | (Hl4 & 0x03000300u), (A8 & 0x00F000F0u) | (Hr4 & 0x03000300u)};
                        bq[3] = u32x2{(B & 0x00F000F0u) | (Hl2 & 0x03000300u), (B8 & 0x00F000F0u) | (Hr6 & 0x03000300u)};
                        // records (h*8+u)*2 + {0,1}: t = 0,1 then t = 2,3
                        u32x4 aop[2][SETS];
#pragma unroll
                        for (int s = 0; s < SETS; ++s) {
                            aop[0][s] = __builtin_nondeterministic_value(aop[0][s]);
                            aop[1][s] = __builtin_nondeterministic_value(aop[1][s]);
                        }
                        if (lane < 4) {
#pragma unroll
                            for (int s = 0; s < SETS; ++s) {
                                const uint8_t* r0 = xa + s * 4096 + (((h * 8 + u) * 2) * 4 + lane) * 16;
                                aop[0][s] = *(const u32x4*)r0;
                                aop[1][s] = *(const u32x4*)(r0 + 64);
                            }
                        }
#pragma unroll
                        for (int t = 0; t < 4; ++t)
#pragma unroll
                            for (int s = 0; s < SETS; ++s) {
                                const u32x4 ao = aop[t >> 1][s];
                                const half4_t a = __builtin_bit_cast(half4_t, (t & 1) ? u32x2{ao.z, ao.w} : u32x2{ao.x, ao.y});
                                dd[t][s] = __builtin_amdgcn_mfma_f32_4x4x4f16(a, __builtin_bit_cast(half4_t, bq[t]), dd[t][s], 4, 0, 0);
                            }
                    }
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const int j = 8 * h + 2 * t + uq;
                        const float sc = (float)(int)(int8_t)((wq[48 + (j >> 2)] >> (8 * (j & 3))) & 255u);
                        const float f = t < 2 ? M_TWO24 : M_TWO20;
#pragma unroll
                        for (int m = 0; m < MT; ++m) {
                            const f32x4 r = dd[t][m >> 1];
                            const int hh = (m & 1) * 2;
                            const float s = fmaf((r[hh] + r[hh + 1]) * f, inv[m], -32.0f * xs[m * NSEG + j]);
                            tot[m] = fmaf(sc, s, tot[m]);
                        }
                    }
                }
            }
#pragma unroll
            for (int m = 0; m < MT; ++m) acc[m] = fmaf(d, tot[m], acc[m]);
        }
        mrow_lds_fence();
    };

    uint32_t b = b_begin + wave;
    if (b < b_end) prefetch(v0, xv0, b);
    if (b + NW < b_end) prefetch(v1, xv1, b + NW);
    for (; b < b_end; b += 2 * NW) {
        step(v0, xv0, b);
        if (b + NW < b_end) step(v1, xv1, b + NW);
    }

    // ---- fold across the waves of the workgroup, then across workgroups
    __syncthreads();
#pragma unroll
    for (int m = 0; m < MT; ++m) red[(wave * MT + m) * 64 + lane] = acc[m];
    __syncthreads();
    if (wave != 0) return;
    float tot[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        float t = red[m * 64 + lane];
#pragma unroll
        for (int w = 1; w < NW; ++w) t += red[(w * MT + m) * 64 + lane];
        tot[m] = t;
    }
    if (p.n_splits > 1) {
        const size_t plane = (size_t)gridDim.x * 64u;
        float* mine = p.partial + (size_t)blockIdx.y * MT * plane + (size_t)blockIdx.x * 64u + lane;
#pragma unroll
        for (int m = 0; m < MT; ++m)
            __hip_atomic_store(mine + m * plane, tot[m], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        uint32_t ticket = 0;
        if (lane == 0)
            ticket = __hip_atomic_fetch_add(&p.counters[blockIdx.x], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        ticket = __builtin_amdgcn_readfirstlane(ticket);
        if (ticket != p.n_splits - 1) return;
        asm volatile("" ::: "memory");
        const float* base = p.partial + (size_t)blockIdx.x * 64u + lane;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            float t = 0.0f;
            for (uint32_t s = 0; s < p.n_splits; ++s)
                t += __hip_atomic_load(base + ((size_t)s * MT + m) * plane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            tot[m] = t;
        }
        if (lane == 0)
            __hip_atomic_store(&p.counters[blockIdx.x], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    const uint32_t row = row0 + lane;
    if (row < p.N) {
        const float bias = p.bias ? p.bias[row] : 0.0f;
#pragma unroll
        for (int m = 0; m < MT; ++m)
            if ((uint32_t)m < count) yrow[m][row] = tot[m] + bias;
    }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
struct MrowPlan { int nw; uint32_t bps, splits; };

static int sets_of(uint32_t M) { return M <= 2 ? 1 : M <= 4 ? 2 : M <= 8 ? 4 : 8; }

static size_t mrow_wave_lds(int type, int sets)
{
    const size_t lrow = type == KQ_TYPE_Q4_K ? KQ_Q4K_BYTES : Q6W_LDS_ROW;
    const size_t nseg = type == KQ_TYPE_Q4_K ? 8 : 16;
    return 64 * lrow + (size_t)sets * 4096 + 2 * (size_t)sets * nseg * 4;
}

static MrowPlan plan_mrow(const MatmulArgs& a, const GemvTuning& t, bool grouped, int sets)
{
    MrowPlan pl;
    const uint32_t groups = (a.N + 63u) / 64u;
    pl.nw = t.waves > 0 ? t.waves : 4;
    while (pl.nw > 2 && (size_t)pl.nw * mrow_wave_lds(a.type, sets) > 160u * 1024u) pl.nw /= 2;
    uint32_t want = grouped ? 1u : t.splits > 0 ? (uint32_t)t.splits : (512u + groups - 1u) / groups;
    const uint32_t max_splits = (a.n_blocks + pl.nw - 1u) / pl.nw;
    if (want > max_splits) want = max_splits;
    if (want < 1u) want = 1u;
    uint32_t bps = (a.n_blocks + want - 1u) / want;
    bps = (bps + pl.nw - 1u) / pl.nw * pl.nw;
    pl.bps = bps;
    pl.splits = (a.n_blocks + bps - 1u) / bps;
    return pl;
}

bool mrow_supported(const MatmulArgs& a)
{
    if (a.type != KQ_TYPE_Q4_K && a.type != KQ_TYPE_Q6_K) return false;
    if (a.M < 1) return false;
    if (!a.expert_idx && a.M > 16) return false;
    if (((uintptr_t)a.X & 15u) || (a.K & 3u)) return false;
    if ((uintptr_t)a.W & 3u) return false;
    if (a.type == KQ_TYPE_Q4_K && (((uintptr_t)a.W & 15u) || (a.row_stride_bytes & 15u))) return false;
    // Q6_K windows borrow up to 14 bytes from a neighbouring block of the same row
    if (a.type == KQ_TYPE_Q6_K && a.n_blocks < 2) return false;
    if ((size_t)64 * a.row_stride_bytes > 0x7FFFFFFFull) return false;
    return true;
}

size_t mrow_scratch_floats(const MatmulArgs& a, const GemvTuning& t)
{
    const MrowPlan pl = plan_mrow(a, t, a.expert_idx != nullptr, sets_of(a.M));
    if (pl.splits <= 1) return 0;
    return (size_t)pl.splits * 2 * sets_of(a.M) * ((a.N + 63u) / 64u) * 64u;
}

template <int TYPE, int SETS, int NW>
static hipError_t launch_mrow_one(const MrowParams& p, uint32_t tiles_bound, hipStream_t s)
{
    const uint32_t groups = (p.N + 63u) / 64u;
    constexpr size_t lrow = TYPE == KQ_TYPE_Q4_K ? KQ_Q4K_BYTES : Q6W_LDS_ROW;
    constexpr size_t nseg = TYPE == KQ_TYPE_Q4_K ? 8 : 16;
    constexpr size_t wave_lds = 64 * lrow + SETS * 4096 + 2 * SETS * nseg * 4;
    constexpr size_t red = (size_t)NW * 2 * SETS * 64 * sizeof(float);
    constexpr size_t shmem = NW * wave_lds > red ? NW * wave_lds : red;
    if constexpr (shmem > 160 * 1024) {
        return hipErrorInvalidValue;   // plan_mrow never picks such a shape
    } else {
    auto kern = mrow_kernel<TYPE, SETS, NW>;
    if (shmem > 64u * 1024u) {
        static bool raised = false;
        if (!raised) {
            hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
            if (e != hipSuccess) return e;
            raised = true;
        }
    }
    hipLaunchKernelGGL(kern, dim3(groups, p.n_splits, tiles_bound), dim3(64 * NW), shmem, s, p);
    return hipGetLastError();
    }
}

template <int TYPE, int NW>
static hipError_t launch_mrow_sets(const MrowParams& p, int sets, uint32_t tiles_bound, hipStream_t s)
{
    switch (sets) {
    case 1: return launch_mrow_one<TYPE, 1, NW>(p, tiles_bound, s);
    case 2: return launch_mrow_one<TYPE, 2, NW>(p, tiles_bound, s);
    case 4: return launch_mrow_one<TYPE, 4, NW>(p, tiles_bound, s);
    default: return launch_mrow_one<TYPE, 8, NW>(p, tiles_bound, s);
    }
}

// Dense call (a.expert_idx == nullptr, M <= 16) or grouped call: tiles/n_tiles
// come from the MoE grouping kernel, tiles_bound bounds the grid, sets fixes the
// tile capacity (2*sets pairs per tile).
hipError_t launch_mrow(const MatmulArgs& a, const SplitScratch& sc, const GemvTuning& t, const uint32_t* tiles,
                       const uint32_t* n_tiles, uint32_t tiles_bound, int sets, hipStream_t s)
{
    const bool grouped = tiles != nullptr;
    if (!grouped) {
        sets = sets_of(a.M);
        tiles_bound = 1;
    }
    const MrowPlan pl = plan_mrow(a, t, grouped, sets);
    MrowParams p{};
    p.X = (const float*)a.X;
    p.W = a.W;
    p.bias = a.bias;
    p.Y = a.Y;
    p.M = a.M; p.N = a.N; p.K = a.K;
    p.n_blocks = a.n_blocks;
    p.row_stride_bytes = a.row_stride_bytes;
    p.y_offset = a.y_offset;
    p.ldy = a.ldy;
    p.blocks_per_split = pl.bps;
    p.n_splits = pl.splits;
    p.partial = sc.partial;
    p.counters = sc.counters;
    p.tiles = tiles;
    p.n_tiles = n_tiles;
    p.k_slots = a.k_slots ? a.k_slots : 1u;
    p.x_per_slot = a.x_per_slot;
    p.tile_stride = 2u + 2u * (uint32_t)sets;
    if (pl.splits > 1) {
        const uint32_t groups = (a.N + 63u) / 64u;
        if (mrow_scratch_floats(a, t) > sc.capacity_floats || groups > sc.n_counters) return hipErrorOutOfMemory;
    }
    const bool q4 = a.type == KQ_TYPE_Q4_K;
    switch (pl.nw) {
    case 2: return q4 ? launch_mrow_sets<KQ_TYPE_Q4_K, 2>(p, sets, tiles_bound, s) : launch_mrow_sets<KQ_TYPE_Q6_K, 2>(p, sets, tiles_bound, s);
    case 4: return q4 ? launch_mrow_sets<KQ_TYPE_Q4_K, 4>(p, sets, tiles_bound, s) : launch_mrow_sets<KQ_TYPE_Q6_K, 4>(p, sets, tiles_bound, s);
    case 8: return q4 ? launch_mrow_sets<KQ_TYPE_Q4_K, 8>(p, sets, tiles_bound, s) : launch_mrow_sets<KQ_TYPE_Q6_K, 8>(p, sets, tiles_bound, s);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace kq
