// kq_fuse.hip — the stand-alone forms of what the lanes-along-K decode kernels fold into their activation
// prologue and their stores: RMSNorm of a row, act(gate) * up, and the residual add.  They serve the
// shapes those kernels decline (more than two tokens, rows longer than their registers hold), so that
// the fused entry point computes the same function for every shape.
//
// Reference forms: norm/rms_norm.wgsl:15-20 and quant_kq/q4k_matmul_norm.wgsl:50-91 (y = x * rstd * w,
// rstd = 1/sqrt(mean(x^2) + eps)); fused/silu_mul_fused.wgsl:39-49; fused/gelu_mul_fused.wgsl:22-32; the
// add_inplace dispatch after down (runtime/model_runner.cpp:3775-3793).
#include <hip/hip_runtime.h>

#include "kq_kernels.h"
#include "kq_wave.h"

namespace kq {

// An output element as fp32, or as bf16 (round to nearest even: the activation rows of the prefill GEMM).
__device__ __forceinline__ void put_out(float* out, size_t at, float v) { out[at] = v; }
__device__ __forceinline__ void put_out(uint16_t* out, size_t at, float v)
{
    out[at] = __builtin_bit_cast(uint16_t, (__bf16)v);
}

// One workgroup of 256 lanes per row.
template <typename OUT>
__global__ __launch_bounds__(256) void rms_norm_rows_kernel(const float* X, const float* w, float eps, uint32_t K,
                                                            OUT* out)
{
    __shared__ float part[4];
    const float* x = X + (size_t)blockIdx.x * K;
    float ss = 0.0f;
    for (uint32_t k = threadIdx.x; k < K; k += 256u) ss = __builtin_fmaf(x[k], x[k], ss);
    ss = wave_total(ss);
    if ((threadIdx.x & 63u) == 0) part[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float rstd = 1.0f / sqrtf(((part[0] + part[1]) + (part[2] + part[3])) / (float)K + eps);
    const size_t o = (size_t)blockIdx.x * K;
    for (uint32_t k = threadIdx.x; k < K; k += 256u) put_out(out, o + k, x[k] * rstd * w[k]);
}

// out[m, k] = X[m, k] converted (blockIdx.y = row)
__global__ __launch_bounds__(256) void cast_rows_bf16_kernel(const float* X, uint32_t K, uint16_t* out)
{
    const uint32_t k = blockIdx.x * 256u + threadIdx.x;
    if (k >= K) return;
    const size_t at = (size_t)blockIdx.y * K + k;
    put_out(out, at, X[at]);
}

// GU rows are gate | up (2K floats); out rows are K floats.
template <bool GELU, typename OUT>
__global__ __launch_bounds__(256) void act_mul_rows_kernel(const float* GU, uint32_t K, OUT* out)
{
    const float* g = GU + (size_t)blockIdx.y * 2u * K;
    const uint32_t k = blockIdx.x * 256u + threadIdx.x;
    if (k >= K) return;
    const float gv = g[k], uv = g[K + k];
    float a;
    if (GELU) {
        const float inner = 0.7978845608f * (gv + 0.044715f * gv * gv * gv);
        a = 0.5f * gv * (1.0f + tanhf(inner));
    } else {
        a = gv / (expf(-gv) + 1.0f);
    }
    put_out(out, (size_t)blockIdx.y * K + k, a * uv);
}

// Y[m, y_offset + n] = T[m, n] + R[m, y_offset + n]   (R may be Y)
__global__ __launch_bounds__(256) void add_residual_kernel(const float* T, const float* R, float* Y, uint32_t N,
                                                           uint32_t ldy, uint32_t y_offset)
{
    const uint32_t n = blockIdx.x * 256u + threadIdx.x;
    if (n >= N) return;
    const size_t at = (size_t)blockIdx.y * ldy + y_offset + n;
    Y[at] = T[(size_t)blockIdx.y * N + n] + R[at];
}

template <typename OUT>
static hipError_t launch_prologue_rows_as(int pro, const float* X, const float* norm_w, float eps, uint32_t M, uint32_t K,
                                          OUT* out, hipStream_t s)
{
    if (pro == 1) hipLaunchKernelGGL(rms_norm_rows_kernel<OUT>, dim3(M), dim3(256), 0, s, X, norm_w, eps, K, out);
    else if (pro == 2) hipLaunchKernelGGL((act_mul_rows_kernel<false, OUT>), dim3((K + 255u) / 256u, M), dim3(256), 0, s, X, K, out);
    else hipLaunchKernelGGL((act_mul_rows_kernel<true, OUT>), dim3((K + 255u) / 256u, M), dim3(256), 0, s, X, K, out);
    return hipGetLastError();
}

hipError_t launch_prologue_rows(int pro, const float* X, const float* norm_w, float eps, uint32_t M, uint32_t K,
                                float* out, hipStream_t s)
{
    return launch_prologue_rows_as(pro, X, norm_w, eps, M, K, out, s);
}

// pro 0: the rows as they are
hipError_t launch_prologue_rows_bf16(int pro, const float* X, const float* norm_w, float eps, uint32_t M, uint32_t K,
                                     uint16_t* out, hipStream_t s)
{
    if (pro != 0) return launch_prologue_rows_as(pro, X, norm_w, eps, M, K, out, s);
    hipLaunchKernelGGL(cast_rows_bf16_kernel, dim3((K + 255u) / 256u, M), dim3(256), 0, s, X, K, out);
    return hipGetLastError();
}

hipError_t launch_add_residual(const float* T, const float* R, float* Y, uint32_t M, uint32_t N, uint32_t ldy,
                               uint32_t y_offset, hipStream_t s)
{
    hipLaunchKernelGGL(add_residual_kernel, dim3((N + 255u) / 256u, M), dim3(256), 0, s, T, R, Y, N, ldy, y_offset);
    return hipGetLastError();
}

}  // namespace kq
