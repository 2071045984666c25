// kq_generic.hip — shape-agnostic fused dequant-matmul.
//
// Serves every call the specialised kernels decline (rows that are not 16-byte
// aligned, ragged N, unusual K) and is the in-library cross-check for them.
// One wavefront per output row; each lane owns 4 consecutive elements of every
// superblock, accumulates in fp32 for up to 4 rows of X at once, and the 64
// partial sums are folded with cross-lane shuffles.  Weight bytes are read with
// byte loads, so only 4-byte alignment of W is assumed.
#include "kq_format.h"
#include "kq_kernels.h"

namespace kq {

__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

template <int TYPE, int MT, bool INDIRECT>
__global__ __launch_bounds__(256) void matmul_generic_kernel(MatmulArgs a)
{
    constexpr uint32_t BB = TYPE == KQ_TYPE_Q4_K ? KQ_Q4K_BYTES : TYPE == KQ_TYPE_Q5_K ? KQ_Q5K_BYTES : KQ_Q6K_BYTES;
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t n = blockIdx.x * 4u + (threadIdx.x >> 6);
    if (n >= a.N) return;  // whole wave leaves together

    uint32_t wrow = n, m0, mcount, xrow0;
    size_t yrow0;
    if (INDIRECT) {
        const uint32_t pair = blockIdx.y;
        wrow = a.expert_idx[pair] * a.N + n;
        m0 = 0;
        mcount = 1;
        xrow0 = a.x_per_slot ? pair : pair / a.k_slots;
        yrow0 = pair;
    } else {
        m0 = blockIdx.y * MT;
        mcount = a.M - m0 < (uint32_t)MT ? a.M - m0 : (uint32_t)MT;
        xrow0 = m0;
        yrow0 = m0;
    }
    const float* X = (const float*)a.X;
    const uint8_t* row = a.W + (size_t)wrow * a.row_stride_bytes;

    float acc[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[m] = 0.0f;

    for (uint32_t b = 0; b < a.n_blocks; ++b) {
        const uint8_t* blk = row + (size_t)b * BB;
        float w[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
            w[j] = kq_element<TYPE>(blk, lane * 4u + j);
        const size_t k0 = (size_t)b * KQ_QK + lane * 4u;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            if ((uint32_t)m < mcount) {
                const float* x = X + (size_t)(xrow0 + m) * a.K + k0;
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[m] = fmaf(x[j], w[j], acc[m]);
            }
        }
    }
    const float bias = a.bias ? a.bias[n] : 0.0f;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
        const float s = wave_sum(acc[m]);
        if ((uint32_t)m < mcount && lane == 0)
            a.Y[(yrow0 + m) * a.ldy + a.y_offset + n] = s + bias;
    }
}

hipError_t launch_matmul_generic(const MatmulArgs& a, hipStream_t s)
{
    if (a.M == 0 || a.N == 0) return hipSuccess;
    const uint32_t gx = (a.N + 3u) / 4u;
    if (a.expert_idx) {
        // one grid row per (token, slot) pair; M carries the pair count
        for (uint32_t p0 = 0; p0 < a.M; p0 += 65535u) {
            MatmulArgs c = a;
            const uint32_t pc = a.M - p0 < 65535u ? a.M - p0 : 65535u;
            // shift the pair-indexed arrays; token rows shift only per-slot X
            c.expert_idx = a.expert_idx + p0;
            c.Y = a.Y + (size_t)p0 * a.ldy;
            if (a.x_per_slot) c.X = (const float*)a.X + (size_t)p0 * a.K;
            else if (p0 % a.k_slots) return hipErrorInvalidValue;
            else c.X = (const float*)a.X + (size_t)(p0 / a.k_slots) * a.K;
            dim3 grid(gx, pc);
            if (a.type == KQ_TYPE_Q4_K)
                hipLaunchKernelGGL((matmul_generic_kernel<KQ_TYPE_Q4_K, 1, true>), grid, dim3(256), 0, s, c);
            else if (a.type == KQ_TYPE_Q5_K)
                hipLaunchKernelGGL((matmul_generic_kernel<KQ_TYPE_Q5_K, 1, true>), grid, dim3(256), 0, s, c);
            else
                hipLaunchKernelGGL((matmul_generic_kernel<KQ_TYPE_Q6_K, 1, true>), grid, dim3(256), 0, s, c);
        }
        return hipGetLastError();
    }
    constexpr int MT = 4;
    for (uint32_t m0 = 0; m0 < a.M; m0 += 65535u * MT) {
        MatmulArgs c = a;
        const uint32_t mc = a.M - m0 < 65535u * MT ? a.M - m0 : 65535u * MT;
        c.M = mc;
        c.X = (const float*)a.X + (size_t)m0 * a.K;
        c.Y = a.Y + (size_t)m0 * a.ldy;
        dim3 grid(gx, (mc + MT - 1) / MT);
        if (a.type == KQ_TYPE_Q4_K)
            hipLaunchKernelGGL((matmul_generic_kernel<KQ_TYPE_Q4_K, MT, false>), grid, dim3(256), 0, s, c);
        else if (a.type == KQ_TYPE_Q5_K)
            hipLaunchKernelGGL((matmul_generic_kernel<KQ_TYPE_Q5_K, MT, false>), grid, dim3(256), 0, s, c);
        else
            hipLaunchKernelGGL((matmul_generic_kernel<KQ_TYPE_Q6_K, MT, false>), grid, dim3(256), 0, s, c);
    }
    return hipGetLastError();
}

}  // namespace kq
