// kq_route.hip — the router stage in front of the MoE expert matvecs: router logits (fp32 matvec against
// the [n_experts, hidden] router matrix) and, per token, the k largest by iterated argmax with a softmax
// over the selected ones.
//
// Reference forms: runtime/kernels/moe/topk_softmax.wgsl:23-67 (k passes of argmax over the unmasked
// logits, `v > best` so the lowest index wins a tie, best starts at -3.4e38 with index 0; weights
// exp(v - max) over the selected, times 1/sum when the normalize flag is set and the sum is positive),
// dispatched per layer after the router matmul (runtime/model_runner.cpp:3532-3548).  The reference
// runs the selection on one thread of one workgroup per token; here a wave per token keeps the logits
// in registers and each pass is a lane-local scan and a six-step butterfly.
#include <hip/hip_runtime.h>

#include "kq_kernels.h"
#include "kq_wave.h"

namespace kq {

constexpr int ROUTE_MAX_PER_LANE = 16;   // n_experts <= 1024
constexpr float ROUTE_NEG_INF = -3.4e38f;

// One wave selects for one token.  vals[j] is the logit of expert 64*j + lane (-inf beyond n_experts).
// Lane s ends up holding the s-th pick.  The pass loop is a real loop: these kernels run their code once,
// and unrolled they spent their time fetching instructions (10 us for a few hundred operations).
template <int PER_LANE>
__device__ __forceinline__ void route_select(float (&vals)[PER_LANE], uint32_t lane, uint32_t n_experts, uint32_t k,
                                             int normalize, uint32_t* idx_out, float* wt_out)
{
    float my_v = ROUTE_NEG_INF;
    uint32_t my_i = 0;
    uint32_t taken = 0;   // bit j: the lane's j-th expert is masked
#pragma nounroll
    for (uint32_t s = 0; s < k; ++s) {
        // lane-local candidate among the unmasked experts; an expert only counts if it beats -3.4e38
        float bv = ROUTE_NEG_INF;
        uint32_t bi = 0xFFFFFFFFu;
#pragma unroll
        for (int j = 0; j < PER_LANE; ++j) {
            const uint32_t e = 64u * j + lane;
            const bool ok = e < n_experts && !((taken >> j) & 1u) && vals[j] > bv;   // ascending e: first wins
            bv = ok ? vals[j] : bv;
            bi = ok ? e : bi;
        }
        wave_best(bv, bi);
        // nothing above -3.4e38 left: the reference's scan leaves index 0 and that value
        if (bi == 0xFFFFFFFFu) bi = 0;
        else if ((bi & 63u) == lane) taken |= 1u << (bi >> 6);
        if (lane == s) { my_v = bv; my_i = bi; }
    }
    float mx = lane < k ? my_v : ROUTE_NEG_INF;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    const float ex = lane < k ? expf(my_v - mx) : 0.0f;
    float sum = ex;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) sum += __shfl_xor(sum, o);
    const float inv = (normalize && sum > 0.0f) ? 1.0f / sum : 1.0f;
    if (lane < k) {
        idx_out[lane] = my_i;
        wt_out[lane] = ex * inv;
    }
}

// Picks the scan width by the number of experts (wave-uniform): the lane-local scan is the larger half
// of a pass.
__device__ __forceinline__ void route_select_any(float (&vals)[ROUTE_MAX_PER_LANE], uint32_t lane, uint32_t n_experts,
                                                 uint32_t k, int normalize, uint32_t* idx_out, float* wt_out)
{
    if (n_experts <= 128u) {
        float v2[2] = {vals[0], vals[1]};
        route_select(v2, lane, n_experts, k, normalize, idx_out, wt_out);
    } else if (n_experts <= 256u) {
        float v4[4] = {vals[0], vals[1], vals[2], vals[3]};
        route_select(v4, lane, n_experts, k, normalize, idx_out, wt_out);
    } else {
        route_select(vals, lane, n_experts, k, normalize, idx_out, wt_out);
    }
}

// logits [T, n_experts] -> idx, wt [T, k]; a wave per token, four tokens per workgroup.
__global__ __launch_bounds__(256) void topk_softmax_kernel(const float* logits, uint32_t T, uint32_t n_experts,
                                                           uint32_t k, int normalize, uint32_t* idx, float* wt)
{
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t tok = blockIdx.x * 4u + (threadIdx.x >> 6);
    if (tok >= T) return;
    float vals[ROUTE_MAX_PER_LANE];
#pragma unroll
    for (int j = 0; j < ROUTE_MAX_PER_LANE; ++j) {
        const uint32_t e = 64u * j + lane;
        vals[j] = e < n_experts ? logits[(size_t)tok * n_experts + e] : ROUTE_NEG_INF;
    }
    route_select_any(vals, lane, n_experts, k, normalize, idx + (size_t)tok * k, wt + (size_t)tok * k);
}

// Logits of experts e0 .. e0+3 for one token: lanes along hidden, four independent load streams.
__device__ __forceinline__ void route_dot4(const float* x, const float* router_w, uint32_t hidden, uint32_t n_experts,
                                           uint32_t e0, uint32_t lane, float (&out)[4])
{
    const uint32_t h4 = hidden / 4u;   // hidden % 4 == 0 (checked by the caller)
    const float4* x4 = (const float4*)x;
    const float4* w4[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) w4[j] = (const float4*)(router_w + (size_t)min(e0 + j, n_experts - 1u) * hidden);
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (uint32_t i = lane; i < h4; i += 64u) {
        const float4 a = x4[i];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float4 b = w4[j][i];
            acc[j] = fmaf(a.x, b.x, acc[j]);
            acc[j] = fmaf(a.y, b.y, acc[j]);
            acc[j] = fmaf(a.z, b.z, acc[j]);
            acc[j] = fmaf(a.w, b.w, acc[j]);
        }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) acc[j] += __shfl_xor(acc[j], o);
        out[j] = acc[j];
    }
}

// Router matvec and selection in one launch: a workgroup of four waves per token.  Wave w computes the
// logits of experts 4w .. 4w+3, 4w+16 .., the logits meet in LDS, wave 0 selects.  router_w: f32
// [n_experts, hidden].  For many tokens (a workgroup each fills the machine).
__global__ __launch_bounds__(256) void route_kernel(const float* X, const float* router_w, uint32_t hidden,
                                                    uint32_t n_experts, uint32_t k, int normalize, float* logits_out,
                                                    uint32_t* idx, float* wt)
{
    __shared__ float lg[64 * ROUTE_MAX_PER_LANE];
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t tok = blockIdx.x;
    const float* x = X + (size_t)tok * hidden;
    for (uint32_t e0 = wave * 4u; e0 < n_experts; e0 += 16u) {
        float v[4];
        route_dot4(x, router_w, hidden, n_experts, e0, lane, v);
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (lane == (uint32_t)j && e0 + j < n_experts) {
                lg[e0 + j] = v[j];
                if (logits_out) logits_out[(size_t)tok * n_experts + e0 + j] = v[j];
            }
    }
    __syncthreads();
    if (wave != 0) return;
    float vals[ROUTE_MAX_PER_LANE];
#pragma unroll
    for (int j = 0; j < ROUTE_MAX_PER_LANE; ++j) {
        const uint32_t e = 64u * j + lane;
        vals[j] = e < n_experts ? lg[e] : ROUTE_NEG_INF;
    }
    route_select_any(vals, lane, n_experts, k, normalize, idx + (size_t)tok * k, wt + (size_t)tok * k);
}

// Few tokens: the experts are spread over workgroups (blockIdx.x takes 16 of them, blockIdx.y is the token)
// and the selection is a launch of its own.
__global__ __launch_bounds__(256) void route_logits_kernel(const float* X, const float* router_w, uint32_t hidden,
                                                           uint32_t n_experts, float* logits_out)
{
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t tok = blockIdx.y;
    const uint32_t e0 = blockIdx.x * 16u + wave * 4u;
    if (e0 >= n_experts) return;
    float v[4];
    route_dot4(X + (size_t)tok * hidden, router_w, hidden, n_experts, e0, lane, v);
#pragma unroll
    for (int j = 0; j < 4; ++j)
        if (lane == (uint32_t)j && e0 + j < n_experts) logits_out[(size_t)tok * n_experts + e0 + j] = v[j];
}

hipError_t launch_topk_softmax(const float* logits, uint32_t T, uint32_t n_experts, uint32_t k, int normalize,
                               uint32_t* idx, float* wt, hipStream_t s)
{
    hipLaunchKernelGGL(topk_softmax_kernel, dim3((T + 3u) / 4u), dim3(256), 0, s, logits, T, n_experts, k, normalize,
                       idx, wt);
    return hipGetLastError();
}

hipError_t launch_route(const float* X, const float* router_w, uint32_t T, uint32_t hidden, uint32_t n_experts,
                        uint32_t k, int normalize, float* logits_out, float* logits_scratch, uint32_t* idx, float* wt,
                        hipStream_t s)
{
    // logits_scratch holds ROUTE_SPREAD_TOKENS x 1024 floats: below that many tokens a workgroup per token
    // would leave most of the machine idle
    if (T < ROUTE_SPREAD_TOKENS && logits_scratch) {
        float* lg = logits_out ? logits_out : logits_scratch;
        hipLaunchKernelGGL(route_logits_kernel, dim3((n_experts + 15u) / 16u, T), dim3(256), 0, s, X, router_w, hidden,
                           n_experts, lg);
        return launch_topk_softmax(lg, T, n_experts, k, normalize, idx, wt, s);
    }
    hipLaunchKernelGGL(route_kernel, dim3(T), dim3(256), 0, s, X, router_w, hidden, n_experts, k, normalize,
                       logits_out, idx, wt);
    return hipGetLastError();
}

}  // namespace kq
