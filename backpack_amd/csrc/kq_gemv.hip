// kq_gemv.hip — decode GEMV (M = 1..4) for Q4_K and Q6_K, one output row per lane.
//
// Data flow, per wavefront, per superblock column b of a 64-row group:
//   HBM --global_load_dwordx4, lanes sweep the 64 rows' block bytes--> VGPRs
//       --ds_write_b128, linear--> LDS (wave-private tile, an exact byte copy)
//       --ds_read, lane r reads row r--> VGPRs --> unpack + fp32 FMAs.
// Because every lane of a wave is at the same k, the activations are wave-
// uniform: they are fetched with scalar loads and fed to the FMAs as scalar
// operands, so X costs no vector registers, no LDS traffic and no cross-lane
// reduction.  4-bit / 6-bit quants are never converted with v_cvt: a masked
// nibble sitting in the low mantissa bits of an fp16 lane *is* the subnormal
// q * 2^-24 (or q * 2^-20 four bits up), which v_fma_mix_f32 multiplies with the
// fp32 activation exactly; the power of two is folded into the block scale.
// The per-sub-block minimum (Q4_K) and the -32 offset (Q6_K) are applied once
// per sub-block against sums of X computed by the workgroup into LDS.
//
// A workgroup is 4 waves that share a 64-row group and take interleaved
// superblock columns; their per-row sums are folded through LDS in wave order.
// When a matrix has too few row groups to fill 256 CUs the K range is also
// split across workgroups: each writes its 64 partial sums to scratch, and the
// last to arrive (one atomic counter per row group) adds them in split order,
// so results do not depend on scheduling.
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

constexpr int GEMV_WAVES = 4;
constexpr float TWO24 = 16777216.0f;
constexpr float TWO20 = 1048576.0f;

struct GemvParams {
    const float* X;
    const uint8_t* W;
    const float* bias;
    float* Y;
    uint32_t M, N, K, n_blocks, row_stride_bytes, y_offset, ldy;
    uint32_t blocks_per_split, n_splits;
    float* partial;       // [n_splits][M][groups*64]
    uint32_t* counters;   // [groups]
};

// Sums of X over every aligned run of SEG elements of the workgroup's K range,
// for each of the MT rows, into LDS: xs[(m*nblk + blk) * (256/SEG) + j].
template <int MT, int SEG>
__device__ __forceinline__ void stage_x_sums(const float* __restrict__ X, uint32_t K, uint32_t M,
                                             uint32_t b_begin, uint32_t nblk, float* xs)
{
    constexpr int LANES = SEG / 4;       // lanes holding one run, one float4 each
    const uint32_t chunks = nblk * 64u;  // float4 chunks per row of X
    for (int m = 0; m < MT; ++m) {
        const float4* x4 = (const float4*)(X + (size_t)(m < (int)M ? m : 0) * K + (size_t)b_begin * KQ_QK);
        for (uint32_t c0 = 0; c0 < chunks; c0 += 256u) {
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
template <int MT>
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
        for (int w = 1; w < GEMV_WAVES; ++w) t += red[(w * MT + m) * 64 + lane];
        tot[m] = t;
    }
    if (p.n_splits > 1) {
        const uint32_t groups = gridDim.x;
        const size_t plane = (size_t)groups * 64u;
#pragma unroll
        for (int m = 0; m < MT; ++m)
            p.partial[((size_t)blockIdx.y * MT + m) * plane + (size_t)blockIdx.x * 64u + lane] = tot[m];
        __threadfence();
        uint32_t ticket = 0;
        if (lane == 0) ticket = atomicAdd(&p.counters[blockIdx.x], 1u);
        ticket = __builtin_amdgcn_readfirstlane(ticket);
        if (ticket != p.n_splits - 1) return;
        __threadfence();
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            float t = 0.0f;
            for (uint32_t s = 0; s < p.n_splits; ++s)
                t += __builtin_nontemporal_load(
                    &p.partial[((size_t)s * MT + m) * plane + (size_t)blockIdx.x * 64u + lane]);
            tot[m] = t;
        }
        if (lane == 0) p.counters[blockIdx.x] = 0u;  // ready for the next launch
    }
    if (row < p.N) {
        const float b = p.bias ? p.bias[row] : 0.0f;
#pragma unroll
        for (int m = 0; m < MT; ++m)
            if ((uint32_t)m < p.M) p.Y[(size_t)m * p.ldy + p.y_offset + row] = tot[m] + b;
    }
}

// ---------------------------------------------------------------------------
// Q4_K
// ---------------------------------------------------------------------------
template <int MT>
__global__ __launch_bounds__(64 * GEMV_WAVES) void q4k_gemv_kernel(GemvParams p)
{
    extern __shared__ __align__(16) uint8_t smem[];
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t row0 = blockIdx.x * 64u;
    const uint32_t b_begin = blockIdx.y * p.blocks_per_split;
    const uint32_t b_end = min(p.n_blocks, b_begin + p.blocks_per_split);
    const uint32_t nblk = b_end - b_begin;

    u32x4* tile = (u32x4*)(smem + wave * (64 * KQ_Q4K_BYTES));       // 576 pieces of 16 B
    float* xs = (float*)(smem + GEMV_WAVES * 64 * KQ_Q4K_BYTES);      // [MT][nblk][8]
    float* red = (float*)smem;                                          // reused at the end

    stage_x_sums<MT, 32>(p.X, p.K, p.M, b_begin, nblk, xs);

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
            v[i] = __builtin_nontemporal_load((const u32x4*)(wbase + goff[i] + (size_t)b * KQ_Q4K_BYTES));
    }
    __syncthreads();  // xs ready

    for (; b < b_end; b += GEMV_WAVES) {
#pragma unroll
        for (int i = 0; i < 9; ++i) tile[i * 64 + lane] = v[i];
        const uint32_t bn = b + GEMV_WAVES;
        if (bn < b_end) {
#pragma unroll
            for (int i = 0; i < 9; ++i)
                v[i] = __builtin_nontemporal_load((const u32x4*)(wbase + goff[i] + (size_t)bn * KQ_Q4K_BYTES));
        }
        wave_lds_fence();
        const u32x4 hdr = tile[lane * 9];
        u32x4 q[8];
#pragma unroll
        for (int s = 0; s < 8; ++s) q[s] = tile[lane * 9 + 1 + s];
        wave_lds_fence();

        const float d = half_bits_to_float(hdr.x & 0xFFFFu);
        const float dmin = half_bits_to_float(hdr.x >> 16);
        // packed 6-bit fields, one per byte: sc0..3, mn0..3, sc4..7, mn4..7
        const uint32_t scA = hdr.y & 0x3F3F3F3Fu;
        const uint32_t mnA = hdr.z & 0x3F3F3F3Fu;
        const uint32_t scB = (hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u);
        const uint32_t mnB = ((hdr.w >> 4) & 0x0F0F0F0Fu) | ((hdr.z >> 2) & 0x30303030u);

        const uint32_t k0 = b * KQ_QK;
        const uint32_t lb = b - b_begin;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            const float* __restrict__ x = p.X + (size_t)(m < (int)p.M ? m : 0) * p.K + k0;
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
                const float* xsum = xs + ((size_t)m * nblk + lb) * 8 + 2 * g;
                sumM = fmaf(mnE, xsum[0], sumM);
                sumM = fmaf(mnO, xsum[1], sumM);
            }
            const float body = fmaf(sumE, TWO24, sumO * TWO20);
            acc[m] = fmaf(d, body, acc[m]);
            acc[m] = fmaf(-dmin, sumM, acc[m]);
        }
    }
    finish_rows<MT>(p, acc, red, row0, lane, wave);
}

template <int MT>
static hipError_t launch_q4k(const GemvParams& p, hipStream_t s)
{
    const uint32_t groups = (p.N + 63u) / 64u;
    const size_t tiles = (size_t)GEMV_WAVES * 64 * KQ_Q4K_BYTES;
    const size_t xs = (size_t)MT * p.blocks_per_split * 8 * sizeof(float);
    const size_t red = (size_t)GEMV_WAVES * MT * 64 * sizeof(float);
    const size_t shmem = tiles + xs > red ? tiles + xs : red;
    hipLaunchKernelGGL(q4k_gemv_kernel<MT>, dim3(groups, p.n_splits), dim3(64 * GEMV_WAVES), shmem, s, p);
    return hipGetLastError();
}

// Picks the K split: enough workgroups to cover the chip a few times over,
// never fewer than one superblock column per wave.
static void choose_split(uint32_t N, uint32_t n_blocks, int forced_splits, uint32_t& bps, uint32_t& splits)
{
    const uint32_t groups = (N + 63u) / 64u;
    uint32_t want = forced_splits > 0 ? (uint32_t)forced_splits : (1024u + groups - 1u) / groups;
    const uint32_t max_splits = (n_blocks + GEMV_WAVES - 1u) / GEMV_WAVES;
    if (want > max_splits) want = max_splits;
    if (want < 1u) want = 1u;
    bps = (n_blocks + want - 1u) / want;
    bps = (bps + GEMV_WAVES - 1u) / GEMV_WAVES * GEMV_WAVES;  // whole rounds of the 4 waves
    splits = (n_blocks + bps - 1u) / bps;
}

bool gemv_rows_supported(const MatmulArgs& a)
{
    if (a.expert_idx) return false;
    if (a.M < 1 || a.M > 4) return false;
    if (a.type != KQ_TYPE_Q4_K) return false;
    if (((uintptr_t)a.W & 15u) || (a.row_stride_bytes & 15u)) return false;
    if (((uintptr_t)a.X & 15u) || (a.K & 3u)) return false;
    if ((size_t)64 * a.row_stride_bytes > 0x7FFFFFFFull) return false;
    return true;
}

size_t gemv_rows_scratch_floats(const MatmulArgs& a, int forced_splits)
{
    uint32_t bps, splits;
    choose_split(a.N, a.n_blocks, forced_splits, bps, splits);
    if (splits <= 1) return 0;
    const size_t groups = (a.N + 63u) / 64u;
    const size_t mt = a.M <= 1 ? 1 : a.M <= 2 ? 2 : 4;
    return (size_t)splits * mt * groups * 64u;
}

hipError_t launch_gemv_rows(const MatmulArgs& a, const SplitScratch& sc, int forced_splits, hipStream_t s)
{
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
    choose_split(a.N, a.n_blocks, forced_splits, p.blocks_per_split, p.n_splits);
    p.partial = sc.partial;
    p.counters = sc.counters;
    if (p.n_splits > 1) {
        const uint32_t groups = (a.N + 63u) / 64u;
        if (gemv_rows_scratch_floats(a, forced_splits) > sc.capacity_floats || groups > sc.n_counters)
            return hipErrorOutOfMemory;
    }
    if (a.M <= 1) return launch_q4k<1>(p, s);
    if (a.M <= 2) return launch_q4k<2>(p, s);
    return launch_q4k<4>(p, s);
}

}  // namespace kq
