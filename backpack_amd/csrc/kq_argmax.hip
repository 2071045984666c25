// kq_argmax.hip — the greedy-sampling tail behind the lm_head matvec: index of the largest logit per row.
//
// Replaces the two dispatches argmax + argmax_reduce (runtime/kernels/.../argmax.wgsl: per-workgroup
// scan of a chunk with `v > best` from best = -1e30, index 0; argmax_reduce.wgsl: the same over the
// partials; wired in runtime/model_runner.cpp:2441-2453) by one launch: ARGMAX_PARTS workgroups per row
// leave a partial each, the last of them to arrive (a ticket per row) reduces the partials and re-arms
// the ticket.  Among equal maxima the lowest index is returned (the reference's butterfly leaves that
// to the lane order); a row with nothing above -1e30 yields index 0.
#include <hip/hip_runtime.h>

#include "kq_kernels.h"
#include "kq_wave.h"

namespace kq {

// Best of a workgroup of 256 lanes; valid in thread 0.
__device__ __forceinline__ void argmax_block(float& v, uint32_t& i, float (&sv)[4], uint32_t (&si)[4])
{
    wave_best(v, i);
    if ((threadIdx.x & 63u) == 0) { sv[threadIdx.x >> 6] = v; si[threadIdx.x >> 6] = i; }
    __syncthreads();
    if (threadIdx.x == 0) {
        v = sv[0]; i = si[0];
#pragma unroll
        for (int w = 1; w < 4; ++w) best_of(v, i, sv[w], si[w]);
    }
}

__global__ __launch_bounds__(256) void argmax_rows_kernel(const float* logits, uint32_t N, uint32_t ld, int32_t* out_idx,
                                                          float* out_val, float* part_val, uint32_t* part_idx,
                                                          uint32_t* tickets)
{
    __shared__ float sv[4];
    __shared__ uint32_t si[4];
    __shared__ bool last;
    const uint32_t row = blockIdx.y, parts = gridDim.x;
    const float* x = logits + (size_t)row * ld;
    const uint32_t chunk = (N + parts - 1u) / parts;
    const uint32_t begin = blockIdx.x * chunk, end = min(begin + chunk, N);
    float v = -1e30f;
    uint32_t i = 0xFFFFFFFFu;   // "none yet": any real index is lower
    for (uint32_t k = begin + threadIdx.x; k < end; k += 256u) {
        const float t = x[k];
        if (t > v) { v = t; i = k; }   // ascending k per lane: the first of equals stays
    }
    argmax_block(v, i, sv, si);
    if (threadIdx.x == 0) {
        const size_t cell = (size_t)row * parts + blockIdx.x;
        __hip_atomic_store(&part_val[cell], v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(&part_idx[cell], i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        // release: the partial is visible to whoever sees the ticket; acquire: the last one sees them all
        const uint32_t t = __hip_atomic_fetch_add(&tickets[row], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        last = t == parts - 1u;
    }
    __syncthreads();
    if (!last) return;
    v = -1e30f;
    i = 0xFFFFFFFFu;
    for (uint32_t q = threadIdx.x; q < parts; q += 256u) {
        const size_t cell = (size_t)row * parts + q;
        const float pv = __hip_atomic_load(&part_val[cell], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const uint32_t pi = __hip_atomic_load(&part_idx[cell], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        best_of(v, i, pv, pi);
    }
    __syncthreads();   // sv / si are reused
    argmax_block(v, i, sv, si);
    if (threadIdx.x == 0) {
        out_idx[row] = i == 0xFFFFFFFFu ? 0 : (int32_t)i;
        if (out_val) out_val[row] = v;
        __hip_atomic_store(&tickets[row], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // re-armed for the next launch
    }
}

// Scratch of the entry point that allocates nothing (bpk_argmax_rows_static): partial values | partial
// indices | tickets, the layout of the allocated scratch of bpk_argmax_rows, 132 096 bytes that every GPU
// the library runs on holds until the process ends.  Zero when the code object is loaded; the last
// workgroup of a row to arrive puts the row's ticket back to zero, so every launch finds its tickets
// cleared.  In host code this name stands for the array only as a symbol: its device address, one per
// GPU, comes from hipGetSymbolAddress below and is what launches are given.
static __device__ __align__(256) __attribute__((used)) uint32_t scratch[ARGMAX_STATIC_WORDS];

hipError_t argmax_static_scratch(uint32_t** out)
{
    void* ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));   // of the current device
    if (e != hipSuccess) return e;
    *out = (uint32_t*)ptr;
    return hipSuccess;
}

// scratch: ARGMAX_MAX_ROWS * ARGMAX_PARTS floats, as many words, ARGMAX_MAX_ROWS tickets (zero between launches)
hipError_t launch_argmax_rows(const float* logits, uint32_t M, uint32_t N, uint32_t ld, int32_t* out_idx,
                              float* out_val, float* part_val, uint32_t* part_idx, uint32_t* tickets, hipStream_t s)
{
    // a part is worth at least a few thousand logits
    uint32_t parts = (N + 4095u) / 4096u;
    parts = parts < 1u ? 1u : parts > ARGMAX_PARTS ? ARGMAX_PARTS : parts;
    for (uint32_t m0 = 0; m0 < M; m0 += ARGMAX_MAX_ROWS) {
        const uint32_t rows = M - m0 < ARGMAX_MAX_ROWS ? M - m0 : ARGMAX_MAX_ROWS;
        hipLaunchKernelGGL(argmax_rows_kernel, dim3(parts, rows), dim3(256), 0, s, logits + (size_t)m0 * ld, N, ld,
                           out_idx + m0, out_val ? out_val + m0 : nullptr, part_val, part_idx, tickets);
    }
    return hipGetLastError();
}

}  // namespace kq
