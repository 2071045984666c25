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
#include "kq_wave.h"

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

#ifdef KQ_NT_LOADS
#define KQ_WLOAD(ptr) __builtin_nontemporal_load(ptr)
#else
#define KQ_WLOAD(ptr) (*(ptr))
#endif

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
    ArgmaxFold am;        // am.out_idx != nullptr: the greedy pick over the outputs rides along
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
            // (DPP moves inside the group of 4 or 8 lanes: an LDS-routed shuffle costs a hundred cycles)
            static_assert(LANES == 4 || LANES == 8, "a run is held by 4 or 8 lanes");
            s += group_partner<1>(s);
            s += group_partner<2>(s);
            if (LANES > 4) s += group_partner<4>(s);
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
    const float b = (row < p.N && p.bias) ? p.bias[row] : 0.0f;
    if (row < p.N) {
#pragma unroll
        for (int m = 0; m < MT; ++m)
            if ((uint32_t)m < p.M) p.Y[(size_t)m * p.ldy + p.y_offset + row] = tot[m] + b;
    }
    if (!p.am.out_idx) return;
    // The greedy pick (argmax + argmax_reduce behind lm_head, runtime/model_runner.cpp:2441-2453): this wave's
    // best per token goes out as a partial, the last workgroup to take the ticket reduces them all.
    const uint32_t groups = gridDim.x;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        if ((uint32_t)m >= p.M) break;
        float v = tot[m] + b;
        uint32_t i = row;
        if (!(row < p.N && v > -1e30f)) { v = -1e30f; i = 0xFFFFFFFFu; }   // "none": any real index is lower
        wave_best(v, i);
        if (lane == 0) {
            __hip_atomic_store(&p.am.part_val[(size_t)m * groups + blockIdx.x], v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(&p.am.part_idx[(size_t)m * groups + blockIdx.x], i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    // (as in the fold above: write-through stores acknowledged before the ticket, agent-scope loads by the last
    // arriver; no fence, which would write back and invalidate the XCD's L2 once per workgroup)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    uint32_t ticket = 0;
    if (lane == 0)
        ticket = __hip_atomic_fetch_add(p.am.ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    ticket = __builtin_amdgcn_readfirstlane(ticket);
    if (ticket != groups - 1u) return;
    asm volatile("" ::: "memory");
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        if ((uint32_t)m >= p.M) break;
        float v = -1e30f;
        uint32_t i = 0xFFFFFFFFu;
        // eight partials per lane in flight at a time (each load travels past the non-coherent cache levels)
        for (uint32_t q0 = lane; q0 < groups; q0 += 8u * 64u) {
            float pv[8];
            uint32_t pi[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const uint32_t q = min(q0 + 64u * (uint32_t)u, groups - 1u);   // (a repeated partial changes nothing)
                pv[u] = __hip_atomic_load(&p.am.part_val[(size_t)m * groups + q], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                pi[u] = __hip_atomic_load(&p.am.part_idx[(size_t)m * groups + q], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) best_of(v, i, pv[u], pi[u]);
        }
        wave_best(v, i);
        if (lane == 0) {
            p.am.out_idx[m] = i == 0xFFFFFFFFu ? 0 : (int32_t)i;
            if (p.am.out_val) p.am.out_val[m] = v;
        }
    }
    if (lane == 0) __hip_atomic_store(p.am.ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // re-armed
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

template <int MT, int NW>
__global__ __launch_bounds__(64 * NW) void q4k_gemv_kernel(GemvParams p)
{
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr int TILE = 64 * KQ_Q4K_BYTES;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t row0 = blockIdx.x * 64u;
    const uint32_t b_begin = blockIdx.y * p.blocks_per_split;
    const uint32_t b_end = min(p.n_blocks, b_begin + p.blocks_per_split);
    const uint32_t nblk = b_end - b_begin;

    u32x4* tile = (u32x4*)(smem + wave * TILE);   // 576 pieces of 16 B
    float* xs = (float*)(smem + NW * TILE);         // [MT][nblk][8]
    float* red = (float*)smem;                      // reused at the end

    stage_x_sums<MT, 32, 64 * NW>(p.X, p.K, p.M, b_begin, nblk, xs);

    // piece i*64+lane of the wave's 64x144-byte tile: row r, 16-byte segment s
    uint32_t goff[9];
#pragma unroll
    for (int i = 0; i < 9; ++i) {
        const uint32_t pc = i * 64u + lane;
        const uint32_t r = pc / 9u, s = pc - r * 9u;
        const uint32_t row = min(row0 + r, p.N - 1u);
        goff[i] = (row - row0) * p.row_stride_bytes + s * 16u;
    }
    const uint8_t* wbase = p.W + (size_t)row0 * p.row_stride_bytes;

    float acc[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[m] = 0.0f;

    u32x4 v[9];
    uint32_t b = b_begin + wave;
    if (b < b_end) {
#pragma unroll
        for (int i = 0; i < 9; ++i)
            v[i] = KQ_WLOAD((const u32x4*)(wbase + goff[i] + (size_t)b * KQ_Q4K_BYTES));
    }
    __syncthreads();  // xs ready

    for (; b < b_end; b += NW) {
#pragma unroll
        for (int i = 0; i < 9; ++i) tile[i * 64 + lane] = v[i];
        const uint32_t bn = b + NW;
        if (bn < b_end) {
#pragma unroll
            for (int i = 0; i < 9; ++i)
                v[i] = KQ_WLOAD((const u32x4*)(wbase + goff[i] + (size_t)bn * KQ_Q4K_BYTES));
        }
        wave_lds_fence();
        const u32x4 hdr = tile[lane * 9];
        u32x4 q[8];
#pragma unroll
        for (int s = 0; s < 8; ++s) q[s] = tile[lane * 9 + 1 + s];
        wave_lds_fence();
        q4k_block_dot<MT>(hdr, q, p.X, p.K, p.M, b * KQ_QK, xs + (size_t)(b - b_begin) * 8, nblk * 8, acc);
    }
    finish_rows<MT, NW>(p, acc, red, row0, lane, wave);
}

// ---------------------------------------------------------------------------
// Q6_K: 210-byte blocks.  The wave copies a 224-byte window per row (14 pieces)
// that starts at the block for even b and 14 bytes before it for odd b, so the
// window always begins 4-byte aligned and never leaves the row; in LDS rows
// are 240 bytes apart (odd multiple of 16: conflict-free 128-bit reads).
// Odd blocks sit 2 bytes off a word boundary and are realigned with one
// v_alignbit per word.
// ---------------------------------------------------------------------------
constexpr int Q6_WIN_PIECES = 14;
constexpr int Q6_LDS_ROW = 240;

// 32 x 16 elements of one (half, 16-lane quarter) chunk: words A (ql[l]),
// B (ql[l+32]), H (qh[l]) for l = 16*uq .. 16*uq+15, four words each.
template <int MT>
__device__ __forceinline__ void q6k_block_dot(const uint32_t (&w)[53], const float* __restrict__ X, uint32_t K,
                                              uint32_t M, uint32_t k0, const float* xsum, uint32_t xsum_stride,
                                              float (&acc)[MT])
{
    const float d = half_bits_to_float(w[52] & 0xFFFFu);
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const float* __restrict__ x = X + (size_t)(m < (int)M ? m : 0) * K + k0;
        float tot = 0.0f;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int uq = 0; uq < 2; ++uq) {
                float a[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int uu = 0; uu < 4; ++uu) {
                    const int u = uq * 4 + uu;
                    const uint32_t A = w[16 * h + u], B = w[16 * h + 8 + u], H = w[32 + 8 * h + u];
                    const uint32_t A8 = A >> 8, B8 = B >> 8;
                    const uint32_t Hl4 = H << 4, Hl2 = H << 2, Hr4 = H >> 4, Hr6 = H >> 6;
                    // [t][pair]: pair 0 holds l, l+2; pair 1 holds l+1, l+3
                    const half2_t q0a = as_half2((A & 0x000F000Fu) | (Hl4 & 0x00300030u));
                    const half2_t q2a = as_half2((A & 0x00F000F0u) | (Hl4 & 0x03000300u));
                    const half2_t q1a = as_half2((B & 0x000F000Fu) | (Hl2 & 0x00300030u));
                    const half2_t q3a = as_half2((B & 0x00F000F0u) | (Hl2 & 0x03000300u));
                    const half2_t q0b = as_half2((A8 & 0x000F000Fu) | (Hr4 & 0x00300030u));
                    const half2_t q2b = as_half2((A8 & 0x00F000F0u) | (Hr4 & 0x03000300u));
                    const half2_t q1b = as_half2((B8 & 0x000F000Fu) | (Hr6 & 0x00300030u));
                    const half2_t q3b = as_half2((B8 & 0x00F000F0u) | (Hr6 & 0x03000300u));
                    const float* xl = x + 128 * h + 4 * u;
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
                    const float sc = (float)(int)(int8_t)((w[48 + (j >> 2)] >> (8 * (j & 3))) & 255u);
                    const float s = fmaf(a[t], t < 2 ? TWO24 : TWO20, -32.0f * xsum[m * xsum_stride + j]);
                    tot = fmaf(sc, s, tot);
                }
            }
        }
        acc[m] = fmaf(d, tot, acc[m]);
    }
}

template <int MT, int NW>
__global__ __launch_bounds__(64 * NW) void q6k_gemv_kernel(GemvParams p)
{
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr int TILE = 64 * Q6_LDS_ROW;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t row0 = blockIdx.x * 64u;
    const uint32_t b_begin = blockIdx.y * p.blocks_per_split;
    const uint32_t b_end = min(p.n_blocks, b_begin + p.blocks_per_split);
    const uint32_t nblk = b_end - b_begin;

    uint8_t* tile = smem + wave * TILE;
    float* xs = (float*)(smem + NW * TILE);   // [MT][nblk][16]
    float* red = (float*)smem;

    stage_x_sums<MT, 16, 64 * NW>(p.X, p.K, p.M, b_begin, nblk, xs);

    // piece i*64+lane of the 64x224-byte window: row r, segment s
    uint32_t goff[Q6_WIN_PIECES], loff[Q6_WIN_PIECES];
#pragma unroll
    for (int i = 0; i < Q6_WIN_PIECES; ++i) {
        const uint32_t pc = i * 64u + lane;
        const uint32_t r = pc / Q6_WIN_PIECES, s = pc - r * Q6_WIN_PIECES;
        const uint32_t row = min(row0 + r, p.N - 1u);
        goff[i] = (row - row0) * p.row_stride_bytes + s * 16u;
        loff[i] = r * Q6_LDS_ROW + s * 16u;
    }
    const uint8_t* wbase = p.W + (size_t)row0 * p.row_stride_bytes;

    float acc[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[m] = 0.0f;

    // window start of block b relative to the row: 210*b for even b, 210*b - 14 for odd b
    auto win = [](uint32_t b) { return (size_t)b * KQ_Q6K_BYTES - ((b & 1u) ? 14u : 0u); };

    u32x4 v[Q6_WIN_PIECES];
    uint32_t b = b_begin + wave;
    if (b < b_end) {
#pragma unroll
        for (int i = 0; i < Q6_WIN_PIECES; ++i)
            v[i] = KQ_WLOAD((const u32x4*)(wbase + goff[i] + win(b)));
    }
    __syncthreads();  // xs ready

    for (; b < b_end; b += NW) {
#pragma unroll
        for (int i = 0; i < Q6_WIN_PIECES; ++i) *(u32x4*)(tile + loff[i]) = v[i];
        const uint32_t bn = b + NW;
        if (bn < b_end) {
#pragma unroll
            for (int i = 0; i < Q6_WIN_PIECES; ++i)
                v[i] = KQ_WLOAD((const u32x4*)(wbase + goff[i] + win(bn)));
        }
        wave_lds_fence();
        u32x4 raw[Q6_WIN_PIECES];
#pragma unroll
        for (int s = 0; s < Q6_WIN_PIECES; ++s) raw[s] = *(const u32x4*)(tile + lane * Q6_LDS_ROW + s * 16);
        wave_lds_fence();

        // 53 block words: bytes 0..211 of the block (the last half-word unused)
        uint32_t w[53];
        if (b & 1u) {
            // the block starts at byte 14 of the window: word j = bytes 14+4j .. 17+4j
#pragma unroll
            for (int j = 0; j < 53; ++j) {
                const int lo = 3 + j, hi = 4 + j;
                const uint32_t wl = raw[lo >> 2][lo & 3];
                const uint32_t wh = hi < 56 ? raw[hi >> 2][hi & 3] : 0u;
                w[j] = __builtin_amdgcn_alignbit(wh, wl, 16);
            }
        } else {
#pragma unroll
            for (int j = 0; j < 53; ++j) w[j] = raw[j >> 2][j & 3];
        }
        q6k_block_dot<MT>(w, p.X, p.K, p.M, b * KQ_QK, xs + (size_t)(b - b_begin) * 16, nblk * 16, acc);
    }
    finish_rows<MT, NW>(p, acc, red, row0, lane, wave);
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
struct GemvPlan {
    int nw;             // waves per workgroup
    uint32_t bps;       // superblock columns per workgroup
    uint32_t splits;    // workgroups along K
};

// Enough workgroups to cover 256 CUs a few times over, never fewer than one
// superblock column per wave, whole rounds of the NW waves per workgroup.
static GemvPlan plan_gemv(const MatmulArgs& a, const GemvTuning& t)
{
    GemvPlan pl;
    const uint32_t groups = (a.N + 63u) / 64u;
    // measured on MI355X: long Q4_K grids like 8 waves sharing a row group,
    // everything else 4; about 450 workgroups keep 256 CUs fed
    pl.nw = t.waves > 0 ? t.waves : (a.type == KQ_TYPE_Q4_K && groups >= 256u) ? 8 : 4;
    uint32_t want = t.splits > 0 ? (uint32_t)t.splits : (448u + groups - 1u) / groups;
    const uint32_t max_splits = (a.n_blocks + pl.nw - 1u) / pl.nw;
    if (want > max_splits) want = max_splits;
    if (want < 1u) want = 1u;
    uint32_t bps = (a.n_blocks + want - 1u) / want;
    bps = (bps + pl.nw - 1u) / pl.nw * pl.nw;
    pl.bps = bps;
    pl.splits = (a.n_blocks + bps - 1u) / bps;
    return pl;
}

bool gemv_rows_supported(const MatmulArgs& a)
{
    if (a.expert_idx) return false;
    if (a.M < 1 || a.M > 4) return false;
    if (a.type != KQ_TYPE_Q4_K && a.type != KQ_TYPE_Q6_K) return false;
    if (((uintptr_t)a.W & 15u) || (a.row_stride_bytes & 15u)) return false;
    if (((uintptr_t)a.X & 15u) || (a.K & 3u)) return false;
    // Q6_K windows reach 14 bytes into the neighbouring block of the same row:
    // rows must hold an even number of blocks so that odd blocks end the row
    if (a.type == KQ_TYPE_Q6_K && (a.n_blocks & 1u)) return false;
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

template <int TYPE, int MT, int NW>
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
    auto kern = TYPE == KQ_TYPE_Q4_K ? q4k_gemv_kernel<MT, NW> : q6k_gemv_kernel<MT, NW>;
    static size_t raised = 64u * 1024u;   // per instantiation
    if (shmem > raised) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
        if (e != hipSuccess) return e;
        raised = shmem;
    }
    hipLaunchKernelGGL(kern, dim3(groups, p.n_splits), dim3(64 * NW), shmem, s, p);
    return hipGetLastError();
}

template <int TYPE, int NW>
static hipError_t launch_mt(const GemvParams& p, hipStream_t s)
{
    switch (mt_of(p.M)) {
    case 1: return launch_one<TYPE, 1, NW>(p, s);
    case 2: return launch_one<TYPE, 2, NW>(p, s);
    default: return launch_one<TYPE, 4, NW>(p, s);
    }
}

bool gemv_rows_can_fold(const MatmulArgs& a, const ArgmaxFold& f)
{
    // one partial per token and group of 64 rows; the kernels hold up to four tokens
    return a.M >= 1 && a.M <= 4 && a.y_offset == 0 && (uint64_t)a.M * ((a.N + 63u) / 64u) <= f.cells;
}

hipError_t launch_gemv_rows(const MatmulArgs& a, const SplitScratch& sc, const GemvTuning& t, hipStream_t s,
                            const ArgmaxFold* fold)
{
    const GemvPlan pl = plan_gemv(a, t);
    GemvParams p;
    p.am = ArgmaxFold{nullptr, nullptr, nullptr, nullptr, nullptr, 0};
    if (fold) {
        if (!gemv_rows_can_fold(a, *fold)) return hipErrorInvalidValue;
        p.am = *fold;
    }
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
    case 2: return q4 ? launch_mt<KQ_TYPE_Q4_K, 2>(p, s) : launch_mt<KQ_TYPE_Q6_K, 2>(p, s);
    case 4: return q4 ? launch_mt<KQ_TYPE_Q4_K, 4>(p, s) : launch_mt<KQ_TYPE_Q6_K, 4>(p, s);
    case 8: return q4 ? launch_mt<KQ_TYPE_Q4_K, 8>(p, s) : launch_mt<KQ_TYPE_Q6_K, 8>(p, s);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace kq
