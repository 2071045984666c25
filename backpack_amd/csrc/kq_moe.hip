// kq_moe.hip — MoE expert path: on-GPU grouping of (token, slot) pairs by expert,
// the activation between gate/up and down, and the weighted combine.
//
// The reference dispatches one matvec per slot against offsets[slot] =
// expert * rowsPerExpert (compute_offsets.wgsl) and, for T > 1, one per token
// and slot with no reuse of an expert's weights between tokens.  Here the
// T*k pairs are bucketed by expert into tiles of up to CAP pairs; a tile is one
// grid.z slice of the row kernel, so an expert's rows are streamed once per
// tile and shared by its pairs.  Nothing returns to the host: tile count and
// contents stay in device memory and surplus grid slices exit at once.
#include <cmath>
#include "kq_format.h"
#include "kq_kernels.h"

namespace kq {

// One workgroup buckets all pairs.  tiles: records of (2 + cap) words
// {expert, count, pair ids...}; experts appear in ascending order, the pairs
// of an expert in arrival order (the per-pair results do not depend on it).
// One pass over the pairs: the LDS counter's old value is the pair's place inside its expert, and the
// first pairs of a thread stay in registers until the records' places are known; the first record of
// every expert comes from a scan over the workgroup (eight experts per thread, a wave scan, the waves'
// totals through LDS) instead of one thread walking all experts.
constexpr int MOE_GROUP_KEEP = 4;   // pairs per thread kept in registers (more are read again)
__global__ __launch_bounds__(1024) void moe_group_kernel(const uint32_t* __restrict__ expert_idx, uint32_t n_pairs,
                                                         uint32_t n_experts, uint32_t cap, uint32_t* __restrict__ tiles,
                                                         uint32_t* __restrict__ n_tiles)
{
    extern __shared__ uint32_t sm[];
    uint32_t* count = sm;                  // [n_experts]
    uint32_t* base = sm + n_experts;       // [n_experts] first tile of the expert
    uint32_t* fill = sm + 2 * n_experts;   // [n_experts] places taken by the kept pairs (more than 4096 pairs only)
    __shared__ uint32_t wave_total[16];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    for (uint32_t e = tid; e < n_experts; e += 1024u) count[e] = 0;
    __syncthreads();
    uint32_t my_e[MOE_GROUP_KEEP], my_pos[MOE_GROUP_KEEP];
#pragma unroll
    for (int i = 0; i < MOE_GROUP_KEEP; ++i) {
        const uint32_t p = tid + (uint32_t)i * 1024u;
        my_e[i] = p < n_pairs ? expert_idx[p] : 0xFFFFFFFFu;
    }
#pragma unroll
    for (int i = 0; i < MOE_GROUP_KEEP; ++i) {
        my_pos[i] = 0;
        if (my_e[i] < n_experts) my_pos[i] = atomicAdd(&count[my_e[i]], 1u);   // out-of-range ids are dropped
    }
    __syncthreads();
    const bool more = n_pairs > MOE_GROUP_KEEP * 1024u;   // (uniform)
    if (more) {
        // pairs beyond the kept ones: counted now, placed behind the kept ones by a second read below
        for (uint32_t e = tid; e < n_experts; e += 1024u) fill[e] = count[e];
        __syncthreads();
        for (uint32_t p = tid + MOE_GROUP_KEEP * 1024u; p < n_pairs; p += 1024u) {
            const uint32_t e = expert_idx[p];
            if (e < n_experts) atomicAdd(&count[e], 1u);
        }
        __syncthreads();
    }
    // exclusive scan of the experts' record counts: thread t owns experts 8t .. 8t+7
    uint32_t nt[8], mine = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const uint32_t e = tid * 8u + j;
        nt[j] = e < n_experts ? (count[e] + cap - 1u) / cap : 0u;
        mine += nt[j];
    }
    uint32_t incl = mine;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const uint32_t v = __shfl_up(incl, o, 64);
        if (lane >= (uint32_t)o) incl += v;
    }
    if (lane == 63u) wave_total[wave] = incl;
    __syncthreads();
    uint32_t before = 0, all = 0;
#pragma unroll
    for (int w = 0; w < 16; ++w) {
        const uint32_t v = wave_total[w];
        before += (uint32_t)w < wave ? v : 0u;
        all += v;
    }
    uint32_t run = before + incl - mine;
    const uint32_t stride = 2u + cap;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const uint32_t e = tid * 8u + j;
        if (e < n_experts) {
            base[e] = run;
            for (uint32_t i = 0; i < nt[j]; ++i) {
                uint32_t* rec = tiles + (size_t)(run + i) * stride;
                rec[0] = e;
                rec[1] = min(cap, count[e] - i * cap);
            }
            run += nt[j];
        }
    }
    if (tid == 0) *n_tiles = all;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < MOE_GROUP_KEEP; ++i) {
        const uint32_t e = my_e[i];
        if (e < n_experts) tiles[(size_t)(base[e] + my_pos[i] / cap) * stride + 2u + my_pos[i] % cap] = tid + (uint32_t)i * 1024u;
    }
    if (more) {
        for (uint32_t p = tid + MOE_GROUP_KEEP * 1024u; p < n_pairs; p += 1024u) {
            const uint32_t e = expert_idx[p];
            if (e >= n_experts) continue;
            const uint32_t pos = atomicAdd(&fill[e], 1u);
            tiles[(size_t)(base[e] + pos / cap) * stride + 2u + pos % cap] = p;
        }
    }
}

// act[p, i] = silu(gate[p, i]) * up[p, i] with silu(g) = g / (exp(-g) + 1)
__global__ __launch_bounds__(256) void moe_silu_mul_kernel(const float* __restrict__ gate, const float* __restrict__ up,
                                                           float* __restrict__ act, size_t n)
{
    const size_t i = (size_t)blockIdx.x * 256u + threadIdx.x;
    if (i >= n) return;
    const float g = gate[i];
    act[i] = g / (expf(-g) + 1.0f) * up[i];
}

// out[t, h] = sum over slots, in slot order, of wt[t, s] * down[(t*k + s), h]
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ down, const float* __restrict__ wt,
                                                          float* __restrict__ out, uint32_t k, uint32_t hidden)
{
    const uint32_t t = blockIdx.y;
    const uint32_t h = blockIdx.x * 256u + threadIdx.x;
    if (h >= hidden) return;
    float a = 0.0f;
    for (uint32_t s = 0; s < k; ++s) {
        const float v = wt[(size_t)t * k + s] * down[((size_t)t * k + s) * hidden + h];
        a = s == 0 ? v : a + v;
    }
    out[(size_t)t * hidden + h] = a;
}

int moe_sets_for(uint32_t n_pairs, uint32_t n_experts)
{
    const uint32_t per = (n_pairs + n_experts - 1u) / n_experts;
    return per <= 1u ? 1 : per <= 4u ? 2 : 4;
}

uint32_t moe_tiles_bound(uint32_t n_pairs, uint32_t n_experts, int sets)
{
    const uint32_t cap = 2u * (uint32_t)sets;
    const uint32_t a = n_pairs / cap + n_experts;   // every expert can add one partial tile
    return a < n_pairs ? a : n_pairs;
}

// Records that n_pairs pairs spread evenly (independently) over n_experts experts are expected to make at cap
// pairs per record: n_experts * E[ceil(n / cap)] for n ~ Poisson(n_pairs / n_experts).  Host arithmetic for launch
// shapes only; the device counts the real ones.
double moe_expected_records(uint32_t n_pairs, uint32_t n_experts, uint32_t cap)
{
    if (n_experts == 0u || cap == 0u) return 0.0;
    const double lambda = (double)n_pairs / (double)n_experts;
    if (lambda > 500.0) return (double)n_experts * (lambda / (double)cap + 0.5);
    double pmf = std::exp(-lambda), sum = 0.0;
    const uint32_t top = (uint32_t)(lambda + 12.0 * std::sqrt(lambda) + 24.0);
    for (uint32_t n = 1; n <= top; ++n) {
        pmf *= lambda / (double)n;
        sum += pmf * (double)((n + cap - 1u) / cap);
    }
    return (double)n_experts * sum;
}

size_t moe_tiles_words(uint32_t n_pairs, uint32_t n_experts, int sets)
{
    return (size_t)moe_tiles_bound(n_pairs, n_experts, sets) * (2u + 2u * (uint32_t)sets) + 1u;   // + n_tiles
}

hipError_t launch_moe_group(const uint32_t* expert_idx, uint32_t n_pairs, uint32_t n_experts, int sets, uint32_t* tiles,
                            uint32_t* n_tiles, hipStream_t s)
{
    if (n_experts > 8192u) return hipErrorInvalidValue;   // three LDS arrays of n_experts words, eight experts per thread
    hipLaunchKernelGGL(moe_group_kernel, dim3(1), dim3(1024), 3 * n_experts * sizeof(uint32_t), s, expert_idx, n_pairs,
                       n_experts, 2u * (uint32_t)sets, tiles, n_tiles);
    return hipGetLastError();
}

hipError_t launch_moe_silu_mul(const float* gate, const float* up, float* act, size_t n, hipStream_t s)
{
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(moe_silu_mul_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, gate, up, act, n);
    return hipGetLastError();
}

hipError_t launch_moe_combine(const float* down, const float* wt, float* out, uint32_t T, uint32_t k, uint32_t hidden,
                              hipStream_t s)
{
    for (uint32_t t0 = 0; t0 < T; t0 += 65535u) {
        const uint32_t tc = T - t0 < 65535u ? T - t0 : 65535u;
        hipLaunchKernelGGL(moe_combine_kernel, dim3((hidden + 255) / 256, tc), dim3(256), 0, s,
                           down + (size_t)t0 * k * hidden, wt + (size_t)t0 * k, out + (size_t)t0 * hidden, k, hidden);
    }
    return hipGetLastError();
}

}  // namespace kq
