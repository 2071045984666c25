// kq_gemv.hip — decode GEMV (M = 1..4) for Q4_K and Q6_K, one output row per lane.
//
// Data flow, per wavefront, per superblock column b of a 64-row group:
//   HBM --global_load_dwordx4, lanes sweep the 64 rows' block bytes--> VGPRs
//       --ds_write_b128--> LDS (wave-private tile, a byte copy of 64 blocks)
//       --ds_read_b128, lane r reads row r--> VGPRs --> unpack + fp32 FMAs.
// Because every lane of a wave is at the same k, the activations are wave-
// uniform: they are fetched with scalar loads and fed to the FMAs as scalar
// operands, so X costs no vector registers, no LDS traffic and no cross-lane
// reduction.  4-bit / 6-bit quants are never converted with v_cvt: a masked
// field sitting in the low mantissa bits of an fp16 lane *is* the subnormal
// q * 2^-24 (or q * 2^-20 four bits up), which v_fma_mix_f32 multiplies with the
// fp32 activation exactly; the power of two is folded into the block scale.
// The per-sub-block minimum (Q4_K) and the -32 offset (Q6_K) are applied once
// per sub-block against sums of X computed by the workgroup into LDS.
//
// A workgroup is NW waves that share a 64-row group and take interleaved
// superblock columns; their per-row sums are folded through LDS in wave order.
// When a matrix has too few row groups to fill 256 CUs the K range is also
// split across workgroups: each writes its 64 partial sums to scratch with
// write-through stores, and the last to arrive (one atomic counter per row
// group) adds them in split order, so results do not depend on scheduling.
#include "kq_format.h"
#include "kq_kernels.h"

namespace kq {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ half2_t as_half2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }

// acc + (float)h * x with h an fp16 lane: selected as v_fma_mix_f32.
__device__ __forceinline__ float fma_h(_Float16 h, float x, float acc)
{
    return __builtin_fmaf((float)h, x, acc);
}

// LDS traffic between lanes of one wave needs ordering but no s_barrier.
__device__ __forceinline__ void wave_lds_fence()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

constexpr float TWO24 = 16777216.0f;
constexpr float TWO20 = 1048576.0f;

struct GemvParams {
    const float* X;
    const uint8_t* W;
    const float* bias;
    float* Y;
    uint32_t M, N, K, n_blocks, row_stride_bytes, y_offset, ldy;
    uint32_t blocks_per_split, n_splits;
    float* partial;       // [n_splits][MT][groups*64]
    uint32_t* counters;   // [groups], zero between launches
};

// Sums of X over every aligned run of SEG elements of the workgroup's K range,
// for each of the MT rows, into LDS: xs[(m*nblk + blk) * (256/SEG) + j].
template <int MT, int SEG, int NT>
__device__ __forceinline__ void stage_x_sums(const float* __restrict__ X, uint32_t K, uint32_t M,
                                             uint32_t b_begin, uint32_t nblk, float* xs)
{
    constexpr int LANES = SEG / 4;       // lanes holding one run, one float4 each
    const uint32_t chunks = nblk * 64u;  // float4 chunks per row of X
    for (int m = 0; m < MT; ++m) {
        const float4* x4 = (const float4*)(X + (size_t)(m < (int)M ? m : 0) * K + (size_t)b_begin * KQ_QK);
        for (uint32_t c0 = 0; c0 < chunks; c0 += NT) {
            const uint32_t c = c0 + threadIdx.x;
            float s = 0.0f;
            if (c < chunks) {
                const float4 v = x4[c];
                s = (v.x + v.y) + (v.z + v.w);
            }
#pragma unroll
            for (int off = 1; off < LANES; off <<= 1) s += __shfl_xor(s, off, 64);
            if (c < chunks && (threadIdx.x % LANES) == 0) xs[(size_t)m * nblk * (256 / SEG) + c / LANES] = s;
        }
    }
}

// Cross-wave fold, optional cross-workgroup fold, bias and store.
//
// The cross-workgroup step uses no device-wide fence (on this part a fence
// writes back and invalidates the whole L2 of the XCD, once per workgroup).
// Partial sums are stored write-through at agent scope, the wave waits for the
// stores to be acknowledged, then takes a ticket with an agent-scope atomic;
// the last arriver reads the partials with agent-scope loads, which miss the
// non-coherent cache levels.  Counters are re-armed by the last arriver.
template <int MT, int NW>
__device__ __forceinline__ void finish_rows(const GemvParams& p, float (&acc)[MT], float* red,
                                            uint32_t row0, uint32_t lane, uint32_t wave)
{
    __syncthreads();  // tiles are dead: red may alias them
#pragma unroll
    for (int m = 0; m < MT; ++m) red[(wave * MT + m) * 64 + lane] = acc[m];
    __syncthreads();
    if (wave != 0) return;
    const uint32_t row = row0 + lane;
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
    if (row < p.N) {
        const float b = p.bias ? p.bias[row] : 0.0f;
#pragma unroll
        for (int m = 0; m < MT; ++m)
            if ((uint32_t)m < p.M) p.Y[(size_t)m * p.ldy + p.y_offset + row] = tot[m] + b;
    }
}

// ---------------------------------------------------------------------------
// Q4_K: 144-byte blocks = 9 pieces of 16 bytes; tile = 64 rows x 9 pieces.
// ---------------------------------------------------------------------------
template <int MT>
__device__ __forceinline__ void q4k_block_dot(const u32x4& hdr, const u32x4 (&q)[8], const float* __restrict__ X,
                                              uint32_t K, uint32_t M, uint32_t k0, const float* xsum,
                                              uint32_t xsum_stride, float (&acc)[MT])
{
    const float d = half_bits_to_float(hdr.x & 0xFFFFu);
    const float dmin = half_bits_to_float(hdr.x >> 16);
    // packed 6-bit fields, one per byte: sc0..3, mn0..3, sc4..7, mn4..7
    const uint32_t scA = hdr.y & 0x3F3F3F3Fu;
    const uint32_t mnA = hdr.z & 0x3F3F3F3Fu;
    const uint32_t scB = (hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u);
    const uint32_t mnB = ((hdr.w >> 4) & 0x0F0F0F0Fu) | ((hdr.z >> 2) & 0x30303030u);
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const float* __restrict__ x = X + (size_t)(m < (int)M ? m : 0) * K + k0;
        float sumE = 0.0f, sumO = 0.0f, sumM = 0.0f;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            float aE = 0.0f, aO = 0.0f;
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) {
                const u32x4 qq = q[2 * g + hf];
                const uint32_t wds[4] = {qq.x, qq.y, qq.z, qq.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t wv = wds[j];
                    const uint32_t t8 = wv >> 8;
                    const half2_t e02 = as_half2(wv & 0x000F000Fu);
                    const half2_t o02 = as_half2(wv & 0x00F000F0u);
                    const half2_t e13 = as_half2(t8 & 0x000F000Fu);
                    const half2_t o13 = as_half2(t8 & 0x00F000F0u);
                    const int i = hf * 16 + j * 4;
                    const float* xe = x + (2 * g) * 32 + i;
                    const float* xo = x + (2 * g + 1) * 32 + i;
                    aE = fma_h(e02.x, xe[0], aE);
                    aE = fma_h(e13.x, xe[1], aE);
                    aE = fma_h(e02.y, xe[2], aE);
                    aE = fma_h(e13.y, xe[3], aE);
                    aO = fma_h(o02.x, xo[0], aO);
                    aO = fma_h(o13.x, xo[1], aO);
                    aO = fma_h(o02.y, xo[2], aO);
                    aO = fma_h(o13.y, xo[3], aO);
                }
            }
            const uint32_t scw = g < 2 ? scA : scB;
            const uint32_t mnw = g < 2 ? mnA : mnB;
            const int be = (2 * g) & 3, bo = (2 * g + 1) & 3;
            const float scE = (float)((scw >> (8 * be)) & 255u);
            const float scO = (float)((scw >> (8 * bo)) & 255u);
            const float mnE = (float)((mnw >> (8 * be)) & 255u);
            const float mnO = (float)((mnw >> (8 * bo)) & 255u);
            sumE = fmaf(scE, aE, sumE);
            sumO = fmaf(scO, aO, sumO);
            sumM = fmaf(mnE, xsum[m * xsum_stride + 2 * g], sumM);
            sumM = fmaf(mnO, xsum[m * xsum_stride + 2 * g + 1], sumM);
        }
        const float body = fmaf(sumE, TWO24, sumO * TWO20);
        acc[m] = fmaf(d, body, acc[m]);
        acc[m] = fmaf(-dmin, sumM, acc[m]);
    }
}

// Q6_K block: 53 words, delivered through `word(j)`.
template <int MT, typename WordFn>
__device__ __forceinline__ void q6k_block_dot(WordFn word, const float* __restrict__ X, uint32_t K, uint32_t M,
                                              uint32_t k0, const float* xsum, uint32_t xsum_stride, float (&acc)[MT])
{
    const float d = half_bits_to_float(word(52) & 0xFFFFu);
    uint32_t scw[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) scw[i] = word(48 + i);
    float tot[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) tot[m] = 0.0f;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        uint32_t ql[16], qh[8];
#pragma unroll
        for (int i = 0; i < 16; ++i) ql[i] = word(16 * h + i);
#pragma unroll
        for (int i = 0; i < 8; ++i) qh[i] = word(32 + 8 * h + i);
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const float* __restrict__ x = X + (size_t)(m < (int)M ? m : 0) * K + k0 + 128 * h;
#pragma unroll
            for (int uq = 0; uq < 2; ++uq) {
                float a[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int uu = 0; uu < 4; ++uu) {
                    const int u = uq * 4 + uu;
                    const uint32_t A = ql[u], B = ql[8 + u], H = qh[u];
                    const uint32_t A8 = A >> 8, B8 = B >> 8;
                    const uint32_t Hl4 = H << 4, Hl2 = H << 2, Hr4 = H >> 4, Hr6 = H >> 6;
                    // [t][pair]: pair a holds l, l+2; pair b holds l+1, l+3
                    const half2_t q0a = as_half2((A & 0x000F000Fu) | (Hl4 & 0x00300030u));
                    const half2_t q2a = as_half2((A & 0x00F000F0u) | (Hl4 & 0x03000300u));
                    const half2_t q1a = as_half2((B & 0x000F000Fu) | (Hl2 & 0x00300030u));
                    const half2_t q3a = as_half2((B & 0x00F000F0u) | (Hl2 & 0x03000300u));
                    const half2_t q0b = as_half2((A8 & 0x000F000Fu) | (Hr4 & 0x00300030u));
                    const half2_t q2b = as_half2((A8 & 0x00F000F0u) | (Hr4 & 0x03000300u));
                    const half2_t q1b = as_half2((B8 & 0x000F000Fu) | (Hr6 & 0x00300030u));
                    const half2_t q3b = as_half2((B8 & 0x00F000F0u) | (Hr6 & 0x03000300u));
                    const float* xl = x + 4 * u;
                    a[0] = fma_h(q0a.x, xl[0], a[0]);
                    a[0] = fma_h(q0b.x, xl[1], a[0]);
                    a[0] = fma_h(q0a.y, xl[2], a[0]);
                    a[0] = fma_h(q0b.y, xl[3], a[0]);
                    a[1] = fma_h(q1a.x, xl[32], a[1]);
                    a[1] = fma_h(q1b.x, xl[33], a[1]);
                    a[1] = fma_h(q1a.y, xl[34], a[1]);
                    a[1] = fma_h(q1b.y, xl[35], a[1]);
                    a[2] = fma_h(q2a.x, xl[64], a[2]);
                    a[2] = fma_h(q2b.x, xl[65], a[2]);
                    a[2] = fma_h(q2a.y, xl[66], a[2]);
                    a[2] = fma_h(q2b.y, xl[67], a[2]);
                    a[3] = fma_h(q3a.x, xl[96], a[3]);
                    a[3] = fma_h(q3b.x, xl[97], a[3]);
                    a[3] = fma_h(q3a.y, xl[98], a[3]);
                    a[3] = fma_h(q3b.y, xl[99], a[3]);
                }
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const int j = 8 * h + 2 * t + uq;   // scale / 16-element group index
                    const float sc = (float)(int)(int8_t)((scw[j >> 2] >> (8 * (j & 3))) & 255u);
                    const float s = fmaf(a[t], t < 2 ? TWO24 : TWO20, -32.0f * xsum[m * xsum_stride + j]);
                    tot[m] = fmaf(sc, s, tot[m]);
                }
            }
        }
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[m] = fmaf(d, tot[m], acc[m]);
}

// ---------------------------------------------------------------------------
// The kernel.  Q4_K: 144-byte blocks = 9 pieces of 16 bytes, the LDS tile is a
// byte copy of 64 blocks.  Q6_K: 210-byte blocks; the wave copies a 224-byte
// window per row (14 pieces) that starts at the block (even b), 14 bytes before
// it (odd b) or 12 bytes before it (an even block that closes a row of an odd
// number of blocks), so the window is always 4-byte aligned and never leaves the
// row; LDS rows are 240 bytes apart (an odd number of 16-byte slots).  A block
// then starts `base` words into its LDS row, `sh` bits into that word, and
// every word is recovered with one v_alignbit (sh = 0 returns the word as is).
//
// Each wave keeps the pieces of up to DEPTH of its superblocks in registers and
// issues those loads before anything else, so that for the usual case (a wave
// owns <= DEPTH blocks) every HBM request of the launch is in flight within the
// first microsecond; the ring is refilled as blocks are consumed.
// ---------------------------------------------------------------------------
constexpr int Q6_WIN_PIECES = 14;
constexpr int Q6_LDS_ROW = 240;

template <int TYPE, int MT, int NW, int DEPTH>
__global__ __launch_bounds__(64 * NW) void gemv_rows_kernel(GemvParams p)
{
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr bool Q4 = TYPE == KQ_TYPE_Q4_K;
    constexpr int BB = Q4 ? KQ_Q4K_BYTES : KQ_Q6K_BYTES;
    constexpr int NPIECE = Q4 ? 9 : Q6_WIN_PIECES;
    constexpr int LROW = Q4 ? KQ_Q4K_BYTES : Q6_LDS_ROW;
    constexpr int SEG = Q4 ? 32 : 16;
    constexpr int NSEG = 256 / SEG;
    constexpr int TILE = 64 * LROW;

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t row0 = blockIdx.x * 64u;
    const uint32_t b_begin = blockIdx.y * p.blocks_per_split;
    const uint32_t b_end = min(p.n_blocks, b_begin + p.blocks_per_split);
    const uint32_t nblk = b_end - b_begin;

    uint8_t* tile = smem + wave * TILE;
    float* xs = (float*)(smem + NW * TILE);   // [MT][nblk][NSEG]
    float* red = (float*)smem;                // reused at the end

    // ---- piece i*64+lane of the tile: row r, 16-byte segment s (64 = 7*9+1 = 4*14+8)
    uint32_t goff[NPIECE], loff[NPIECE];
    {
        uint32_t r = lane / NPIECE, sg = lane - r * NPIECE;
#pragma unroll
        for (int i = 0; i < NPIECE; ++i) {
            const uint32_t row = min(row0 + r, p.N - 1u);
            goff[i] = (row - row0) * p.row_stride_bytes + sg * 16u;
            loff[i] = r * LROW + sg * 16u;
            r += 64 / NPIECE;
            sg += 64 % NPIECE;
            if (sg >= (uint32_t)NPIECE) { sg -= NPIECE; r += 1; }
        }
    }
    const uint8_t* wbase = p.W + (size_t)row0 * p.row_stride_bytes;
    const uint32_t last_even = (p.n_blocks & 1u) ? p.n_blocks - 1u : 0xFFFFFFFFu;
    auto back = [&](uint32_t b) -> uint32_t {   // bytes the Q6_K window starts before the block
        return Q4 ? 0u : (b & 1u) ? 14u : (b == last_even ? 12u : 0u);
    };

    // ---- all of this wave's first DEPTH blocks go in flight now
    u32x4 v[DEPTH][NPIECE];
#pragma unroll
    for (int dpt = 0; dpt < DEPTH; ++dpt) {
        const uint32_t b = b_begin + wave + dpt * NW;
        if (b < b_end) {
            const size_t o = (size_t)b * BB - back(b);
#pragma unroll
            for (int i = 0; i < NPIECE; ++i)
                v[dpt][i] = __builtin_nontemporal_load((const u32x4*)(wbase + goff[i] + o));
        }
    }

    stage_x_sums<MT, SEG, 64 * NW>(p.X, p.K, p.M, b_begin, nblk, xs);

    float acc[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[m] = 0.0f;
    __syncthreads();  // xs ready

    uint32_t it = 0;
    for (uint32_t b = b_begin + wave; b < b_end; b += NW, ++it) {
        // ---- ring slot it % DEPTH -> LDS, then refill it with block b + DEPTH*NW
        const uint32_t slot = it % DEPTH;
        const uint32_t bn = b + DEPTH * NW;
#pragma unroll
        for (int dpt = 0; dpt < DEPTH; ++dpt) {
            if (slot == (uint32_t)dpt) {
#pragma unroll
                for (int i = 0; i < NPIECE; ++i) *(u32x4*)(tile + loff[i]) = v[dpt][i];
                if (bn < b_end) {
                    const size_t o = (size_t)bn * BB - back(bn);
#pragma unroll
                    for (int i = 0; i < NPIECE; ++i)
                        v[dpt][i] = __builtin_nontemporal_load((const u32x4*)(wbase + goff[i] + o));
                }
            }
        }
        wave_lds_fence();
        const uint8_t* mine = tile + lane * LROW;
        if (Q4) {
            const u32x4 hdr = *(const u32x4*)mine;
            u32x4 q[8];
#pragma unroll
            for (int sgm = 0; sgm < 8; ++sgm) q[sgm] = *(const u32x4*)(mine + 16 + sgm * 16);
            wave_lds_fence();
            q4k_block_dot<MT>(hdr, q, p.X, p.K, p.M, b * KQ_QK, xs + (size_t)(b - b_begin) * NSEG, nblk * NSEG, acc);
        } else {
            const uint32_t bk = back(b);
            const uint32_t* rw = (const uint32_t*)(mine + (bk & ~3u));   // 0 or 12 bytes in
            const uint32_t sh = (bk & 2u) * 8u;                            // 0 or 16 bits
            auto word = [&](int j) -> uint32_t { return __builtin_amdgcn_alignbit(rw[j + 1], rw[j], sh); };
            q6k_block_dot<MT>(word, p.X, p.K, p.M, b * KQ_QK, xs + (size_t)(b - b_begin) * NSEG, nblk * NSEG, acc);
            wave_lds_fence();
        }
    }
    finish_rows<MT, NW>(p, acc, red, row0, lane, wave);
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
struct GemvPlan {
    int nw;             // waves per workgroup
    int depth;          // superblocks a wave keeps in flight
    uint32_t bps;       // superblock columns per workgroup
    uint32_t splits;    // workgroups along K
};

// Enough workgroups to cover 256 CUs a few times over, never fewer than one
// superblock column per wave, whole rounds of the NW waves per workgroup.
static GemvPlan plan_gemv(const MatmulArgs& a, const GemvTuning& t)
{
    GemvPlan pl;
    const uint32_t groups = (a.N + 63u) / 64u;
    pl.nw = t.waves > 0 ? t.waves : 4;
    // measured on MI355X: about 450 workgroups of 4 waves is the sweet spot for
    // every Llama-3-8B shape (more splits pay the cross-workgroup fold, fewer
    // leave CUs idle)
    uint32_t want = t.splits > 0 ? (uint32_t)t.splits : (448u + groups - 1u) / groups;
    const uint32_t max_splits = (a.n_blocks + pl.nw - 1u) / pl.nw;
    if (want > max_splits) want = max_splits;
    if (want < 1u) want = 1u;
    uint32_t bps = (a.n_blocks + want - 1u) / want;
    bps = (bps + pl.nw - 1u) / pl.nw * pl.nw;
    pl.bps = bps;
    pl.splits = (a.n_blocks + bps - 1u) / bps;
    const uint32_t per_wave = bps / pl.nw;
    const int max_depth = a.type == KQ_TYPE_Q4_K ? 4 : 2;
    // deeper rings cost registers (occupancy) and measured slower: default 1
    pl.depth = t.depth > 0 ? t.depth : 1;
    if (pl.depth > max_depth) pl.depth = max_depth;
    (void)per_wave;
    return pl;
}

bool gemv_rows_supported(const MatmulArgs& a)
{
    if (a.expert_idx) return false;
    if (a.M < 1 || a.M > 4) return false;
    if (a.type != KQ_TYPE_Q4_K && a.type != KQ_TYPE_Q6_K) return false;
    if (((uintptr_t)a.W & 15u) || (a.row_stride_bytes & 15u)) return false;
    if (((uintptr_t)a.X & 15u) || (a.K & 3u)) return false;
    // Q6_K windows borrow up to 14 bytes from a neighbouring block of the same row
    if (a.type == KQ_TYPE_Q6_K && a.n_blocks < 2) return false;
    if ((size_t)64 * a.row_stride_bytes > 0x7FFFFFFFull) return false;
    return true;
}

static int mt_of(uint32_t M) { return M <= 1 ? 1 : M <= 2 ? 2 : 4; }

size_t gemv_rows_scratch_floats(const MatmulArgs& a, const GemvTuning& t)
{
    const GemvPlan pl = plan_gemv(a, t);
    if (pl.splits <= 1) return 0;
    return (size_t)pl.splits * mt_of(a.M) * ((a.N + 63u) / 64u) * 64u;
}

template <int TYPE, int MT, int NW, int DEPTH>
static hipError_t launch_one(const GemvParams& p, hipStream_t s)
{
    const uint32_t groups = (p.N + 63u) / 64u;
    constexpr size_t tile = TYPE == KQ_TYPE_Q4_K ? 64 * KQ_Q4K_BYTES : 64 * Q6_LDS_ROW;
    constexpr size_t per_blk = TYPE == KQ_TYPE_Q4_K ? 8 : 16;
    const size_t tiles = (size_t)NW * tile;
    const size_t xs = (size_t)MT * p.blocks_per_split * per_blk * sizeof(float);
    const size_t red = (size_t)NW * MT * 64 * sizeof(float);
    const size_t shmem = tiles + xs > red ? tiles + xs : red;
    if (shmem > 160u * 1024u) return hipErrorInvalidValue;
    auto kern = gemv_rows_kernel<TYPE, MT, NW, DEPTH>;
    static size_t raised = 64u * 1024u;   // per instantiation
    if (shmem > raised) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
        if (e != hipSuccess) return e;
        raised = shmem;
    }
    hipLaunchKernelGGL(kern, dim3(groups, p.n_splits), dim3(64 * NW), shmem, s, p);
    return hipGetLastError();
}

template <int TYPE, int MT, int NW>
static hipError_t launch_depth(const GemvParams& p, int depth, hipStream_t s)
{
    if constexpr (TYPE == KQ_TYPE_Q4_K) {
        if (depth >= 4) return launch_one<TYPE, MT, NW, 4>(p, s);
    }
    if (depth >= 2) return launch_one<TYPE, MT, NW, 2>(p, s);
    return launch_one<TYPE, MT, NW, 1>(p, s);
}

template <int TYPE, int NW>
static hipError_t launch_mt(const GemvParams& p, int depth, hipStream_t s)
{
    switch (mt_of(p.M)) {
    case 1: return launch_depth<TYPE, 1, NW>(p, depth, s);
    case 2: return launch_depth<TYPE, 2, NW>(p, depth, s);
    default: return launch_depth<TYPE, 4, NW>(p, depth, s);
    }
}

hipError_t launch_gemv_rows(const MatmulArgs& a, const SplitScratch& sc, const GemvTuning& t, hipStream_t s)
{
    const GemvPlan pl = plan_gemv(a, t);
    GemvParams p;
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
    if (pl.splits > 1) {
        const uint32_t groups = (a.N + 63u) / 64u;
        if (gemv_rows_scratch_floats(a, t) > sc.capacity_floats || groups > sc.n_counters)
            return hipErrorOutOfMemory;
    }
    const bool q4 = a.type == KQ_TYPE_Q4_K;
    switch (pl.nw) {
    case 2: return q4 ? launch_mt<KQ_TYPE_Q4_K, 2>(p, pl.depth, s) : launch_mt<KQ_TYPE_Q6_K, 2>(p, pl.depth, s);
    case 4: return q4 ? launch_mt<KQ_TYPE_Q4_K, 4>(p, pl.depth, s) : launch_mt<KQ_TYPE_Q6_K, 4>(p, pl.depth, s);
    case 8: return q4 ? launch_mt<KQ_TYPE_Q4_K, 8>(p, pl.depth, s) : launch_mt<KQ_TYPE_Q6_K, 8>(p, pl.depth, s);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace kq
