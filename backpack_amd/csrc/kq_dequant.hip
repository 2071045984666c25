// kq_dequant.hip — dequantise selected rows of a packed Q4_K / Q5_K / Q6_K matrix to
// fp32, bit-identical to the CPU formula.  One thread per output element; the
// 256 threads of a workgroup cover one superblock of one output row, so the
// block's bytes are read once from HBM and served from cache to the rest.
#include "kq_format.h"
#include "kq_kernels.h"

namespace kq {

template <int TYPE>
__global__ __launch_bounds__(256) void dequant_rows_kernel(const uint8_t* __restrict__ W,
                                                           uint32_t row_stride_bytes,
                                                           const int32_t* __restrict__ rows,
                                                           uint32_t K, float* __restrict__ out)
{
    const uint32_t m = blockIdx.y;
    const uint32_t b = blockIdx.x;
    const int32_t rid = rows ? rows[m] : (int32_t)m;
    const uint32_t row = rid > 0 ? (uint32_t)rid : 0u;
    constexpr uint32_t BB = TYPE == KQ_TYPE_Q4_K ? KQ_Q4K_BYTES : TYPE == KQ_TYPE_Q5_K ? KQ_Q5K_BYTES : KQ_Q6K_BYTES;
    const uint8_t* blk = W + (size_t)row * row_stride_bytes + (size_t)b * BB;
    const uint32_t e = threadIdx.x;
    const float v = kq_element<TYPE>(blk, e);
    out[(size_t)m * K + (size_t)b * KQ_QK + e] = v;
}

hipError_t launch_dequant_rows(int type, const uint8_t* W, uint32_t row_stride_bytes,
                               const int32_t* rows, uint32_t M, uint32_t K, float* out,
                               hipStream_t s)
{
    if (M == 0 || K == 0) return hipSuccess;
    // grid.y is limited to 65535: walk M in slabs
    for (uint32_t m0 = 0; m0 < M; m0 += 65535u) {
        const uint32_t mc = M - m0 < 65535u ? M - m0 : 65535u;
        dim3 grid(K / KQ_QK, mc);
        const int32_t* r = rows ? rows + m0 : nullptr;
        // with rows == nullptr the kernel uses blockIdx.y, so shift W instead
        const uint8_t* w = rows ? W : W + (size_t)m0 * row_stride_bytes;
        float* o = out + (size_t)m0 * K;
        if (type == KQ_TYPE_Q4_K)
            hipLaunchKernelGGL(dequant_rows_kernel<KQ_TYPE_Q4_K>, grid, dim3(256), 0, s, w,
                               row_stride_bytes, r, K, o);
        else if (type == KQ_TYPE_Q5_K)
            hipLaunchKernelGGL(dequant_rows_kernel<KQ_TYPE_Q5_K>, grid, dim3(256), 0, s, w,
                               row_stride_bytes, r, K, o);
        else
            hipLaunchKernelGGL(dequant_rows_kernel<KQ_TYPE_Q6_K>, grid, dim3(256), 0, s, w,
                               row_stride_bytes, r, K, o);
    }
    return hipGetLastError();
}

}  // namespace kq
