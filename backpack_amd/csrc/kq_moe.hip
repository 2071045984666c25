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
#include "kq_format.h"
#include "kq_kernels.h"

namespace kq {

// One workgroup buckets all pairs.  tiles: records of (2 + cap) words
// {expert, count, pair ids...}; experts appear in ascending order, the pairs
// of an expert in arrival order (the per-pair results do not depend on it).
__global__ __launch_bounds__(1024) void moe_group_kernel(const uint32_t* __restrict__ expert_idx, uint32_t n_pairs,
                                                         uint32_t n_experts, uint32_t cap, uint32_t* __restrict__ tiles,
                                                         uint32_t* __restrict__ n_tiles)
{
    extern __shared__ uint32_t sm[];
    uint32_t* count = sm;                  // [n_experts]
    uint32_t* base = sm + n_experts;       // [n_experts] first tile of the expert
    uint32_t* fill = sm + 2 * n_experts;   // [n_experts]
    for (uint32_t e = threadIdx.x; e < n_experts; e += blockDim.x) { count[e] = 0; fill[e] = 0; }
    __syncthreads();
    for (uint32_t p = threadIdx.x; p < n_pairs; p += blockDim.x) {
        const uint32_t e = expert_idx[p];
        if (e < n_experts) atomicAdd(&count[e], 1u);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t t = 0;
        for (uint32_t e = 0; e < n_experts; ++e) {
            base[e] = t;
            t += (count[e] + cap - 1u) / cap;
        }
        *n_tiles = t;
    }
    __syncthreads();
    const uint32_t stride = 2u + cap;
    for (uint32_t e = threadIdx.x; e < n_experts; e += blockDim.x) {
        const uint32_t nt = (count[e] + cap - 1u) / cap;
        for (uint32_t i = 0; i < nt; ++i) {
            uint32_t* rec = tiles + (size_t)(base[e] + i) * stride;
            rec[0] = e;
            rec[1] = min(cap, count[e] - i * cap);
        }
    }
    for (uint32_t p = threadIdx.x; p < n_pairs; p += blockDim.x) {
        const uint32_t e = expert_idx[p];
        if (e >= n_experts) continue;   // out-of-range ids are dropped; their outputs stay untouched
        const uint32_t pos = atomicAdd(&fill[e], 1u);
        tiles[(size_t)(base[e] + pos / cap) * stride + 2u + pos % cap] = p;
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

size_t moe_tiles_words(uint32_t n_pairs, uint32_t n_experts, int sets)
{
    return (size_t)moe_tiles_bound(n_pairs, n_experts, sets) * (2u + 2u * (uint32_t)sets) + 1u;   // + n_tiles
}

hipError_t launch_moe_group(const uint32_t* expert_idx, uint32_t n_pairs, uint32_t n_experts, int sets, uint32_t* tiles,
                            uint32_t* n_tiles, hipStream_t s)
{
    if (n_experts > 8192u) return hipErrorInvalidValue;   // three LDS arrays of n_experts words
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
