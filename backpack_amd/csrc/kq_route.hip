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
    // (the picks sit in lanes 0 .. k-1 of the first row of 16, k <= 16: DPP moves inside that row, lane 0 has the result)
    float mx = lane < k ? my_v : ROUTE_NEG_INF;
    mx = fmaxf(mx, group_partner<1>(mx)); mx = fmaxf(mx, group_partner<2>(mx));
    mx = fmaxf(mx, group_partner<4>(mx)); mx = fmaxf(mx, group_partner<8>(mx));
    mx = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, mx), 0));
    const float ex = lane < k ? expf(my_v - mx) : 0.0f;
    float sum = ex;
    sum += group_partner<1>(sum); sum += group_partner<2>(sum);
    sum += group_partner<4>(sum); sum += group_partner<8>(sum);
    sum = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, sum), 0));
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
        out[j] = wave_total(acc[j]);   // (DPP moves: an LDS-routed shuffle costs a hundred cycles)
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

// A workgroup takes TB tokens x 4 experts (many tokens: 8, so a router row is fetched once per 8 tokens instead of
// once per token); its four waves take every fourth step along hidden (lanes along hidden inside a step) and their
// sums meet in LDS, in wave order.  The selection is a launch of its own.  Tokens and experts beyond the end
// repeat the last one (their sums are dropped).
template <int TB>   // tokens per workgroup: 8, or 1 for a few tokens
__global__ __launch_bounds__(256) void route_logits_tiled_kernel(const float* X, const float* router_w, uint32_t T,
                                                                 uint32_t hidden, uint32_t n_experts, float* logits_out)
{
    __shared__ float part[4][4 * TB];
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t t0 = blockIdx.y * TB, e0 = blockIdx.x * 4u;
    const uint32_t h4 = hidden / 4u;
    const float4* x4[TB];
    const float4* w4[4];
#pragma unroll
    for (int t = 0; t < TB; ++t) x4[t] = (const float4*)(X + (size_t)min(t0 + t, T - 1u) * hidden);
#pragma unroll
    for (int j = 0; j < 4; ++j) w4[j] = (const float4*)(router_w + (size_t)min(e0 + j, n_experts - 1u) * hidden);
    float acc[4][TB];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int t = 0; t < TB; ++t) acc[j][t] = 0.0f;
    // (the next step's loads are in flight while this step is multiplied)
    float4 a[TB], b[4];
    auto fetch = [&](uint32_t i) {
        const uint32_t ic = min(i, h4 - 1u);
#pragma unroll
        for (int t = 0; t < TB; ++t) a[t] = x4[t][ic];
#pragma unroll
        for (int j = 0; j < 4; ++j) b[j] = w4[j][ic];
    };
    fetch(wave * 64u + lane);
    for (uint32_t i = wave * 64u + lane; i < h4; i += 256u) {
        float4 ca[TB], cb[4];
#pragma unroll
        for (int t = 0; t < TB; ++t) ca[t] = a[t];
#pragma unroll
        for (int j = 0; j < 4; ++j) cb[j] = b[j];
        fetch(i + 256u);
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int t = 0; t < TB; ++t) {
                acc[j][t] = fmaf(ca[t].x, cb[j].x, acc[j][t]);
                acc[j][t] = fmaf(ca[t].y, cb[j].y, acc[j][t]);
                acc[j][t] = fmaf(ca[t].z, cb[j].z, acc[j][t]);
                acc[j][t] = fmaf(ca[t].w, cb[j].w, acc[j][t]);
            }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int t = 0; t < TB; ++t) {
            const float v = wave_total(acc[j][t]);
            if (lane == (uint32_t)(j * TB + t)) part[wave][j * TB + t] = v;
        }
    __syncthreads();
    if (threadIdx.x < 4u * TB) {
        const uint32_t j = threadIdx.x / TB, t = threadIdx.x % TB;
        const float v = ((part[0][threadIdx.x] + part[1][threadIdx.x]) + part[2][threadIdx.x]) + part[3][threadIdx.x];
        if (e0 + j < n_experts && t0 + t < T) logits_out[(size_t)(t0 + t) * n_experts + e0 + j] = v;
    }
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
    // logits_scratch holds ROUTE_SCRATCH_FLOATS floats (at least ROUTE_SPREAD_TOKENS x 1024): below that many
    // tokens a workgroup per token would leave most of the machine idle
    if (T < ROUTE_SPREAD_TOKENS && logits_scratch) {
        float* lg = logits_out ? logits_out : logits_scratch;
        hipLaunchKernelGGL(route_logits_tiled_kernel<1>, dim3((n_experts + 3u) / 4u, T), dim3(256), 0, s, X, router_w, T,
                           hidden, n_experts, lg);
        return launch_topk_softmax(lg, T, n_experts, k, normalize, idx, wt, s);
    }
    // many tokens: logits by 8-token tiles, then the selection, as long as the logits have a place to go
    if (T >= ROUTE_SPREAD_TOKENS && (logits_out || (logits_scratch && (uint64_t)T * n_experts <= ROUTE_SCRATCH_FLOATS))) {
        float* lg = logits_out ? logits_out : logits_scratch;
        hipLaunchKernelGGL(route_logits_tiled_kernel<8>, dim3((n_experts + 3u) / 4u, (T + 7u) / 8u), dim3(256), 0, s, X,
                           router_w, T, hidden, n_experts, lg);
        return launch_topk_softmax(lg, T, n_experts, k, normalize, idx, wt, s);
    }
    hipLaunchKernelGGL(route_kernel, dim3(T), dim3(256), 0, s, X, router_w, hidden, n_experts, k, normalize,
                       logits_out, idx, wt);
    return hipGetLastError();
}

}  // namespace kq
