// kq_stream.hip — decode GEMV (M = 1) with the lanes of a wave laid along K.
//
// A wave owns whole weight rows (rows w, w + waves, w + 2*waves, ...).  For Q4_K, lane (b, j) = (lane / 8, lane % 8)
// takes the j-th 16-byte piece of the quants of superblock b of the row, so one
// load instruction per lane pulls eight consecutive superblocks (1152 bytes of
// a row, contiguous in memory) and a row of K = 4096 is two such passes.  Piece
// j holds the low nibbles of 16 elements of sub-block 2*(j/2) and the high
// nibbles of 16 elements of sub-block 2*(j/2)+1.  The lane's 32 activations per
// pass are the same for every row, so they are loaded once into registers and
// stay there; a row then costs each lane two 16-byte loads per pass (its piece
// and the block header, which the eight lanes of a block share), the unpack, 32
// v_fma_mix_f32 and the scale arithmetic.  Nothing passes through LDS, nothing
// is shared between waves, and no K split is needed: the reduction over K is a
// DPP butterfly across the wave, once per row.
//
// Nibbles are never converted: w & 0x000F000F leaves two fp16 subnormals
// q * 2^-24, w & 0x00F000F0 two subnormals q * 2^-20; v_fma_mix_f32 multiplies
// them exactly with the fp32 activation and the power of two moves into the
// scale.  The per-sub-block minimum is applied against the lane's own sum of
// its 16 activations, a per-lane constant.
#include "kq_format.h"
#include "kq_kernels.h"

namespace kq {

typedef _Float16 s_half2 __attribute__((ext_vector_type(2)));
typedef uint32_t s_u32x4 __attribute__((ext_vector_type(4)));

struct StreamParams {
    const float* X;
    const uint8_t* W;
    const float* bias;
    float* Y;
    uint32_t N, K, n_blocks, row_stride_bytes, y_offset;
};

__device__ __forceinline__ float s_fma_h(_Float16 h, float x, float acc) { return __builtin_fmaf((float)h, x, acc); }

template <int CTRL>
__device__ __forceinline__ float s_dpp(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}

// Sum over the 64 lanes; the result is wave-uniform.
__device__ __forceinline__ float wave_sum(float v)
{
    v += s_dpp<0xB1>(v);    // quad: lanes ^ 1
    v += s_dpp<0x4E>(v);    // quad: lanes ^ 2
    v += s_dpp<0x141>(v);   // mirror within 8
    v += s_dpp<0x140>(v);   // mirror within 16
    const float a = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
    const float b = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
    const float c = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
    const float d = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
    return (a + b) + (c + d);
}

// One lane's share of one pass of a Q4_K row.
//   hdr: the block's first 16 bytes; q: 16 quant bytes (piece j of the block)
//   xlo/xhi: activations of the piece's 16 elements in the even / odd sub-block
//   sel_hi: lane constant, j/2 >= 2;  sh: lane constant, 16 * ((j/2) & 1)
__device__ __forceinline__ float q4k_piece_dot(const s_u32x4 hdr, const s_u32x4 q, const float (&xlo)[16],
                                               const float (&xhi)[16], float xs_lo, float xs_hi, bool sel_hi,
                                               uint32_t sh)
{
    float alo = 0.0f, ahi = 0.0f;
#pragma unroll
    for (int m = 0; m < 4; ++m) {
        const uint32_t w = q[m];
        const uint32_t w8 = w >> 8;
        const s_half2 a = __builtin_bit_cast(s_half2, w & 0x000F000Fu);     // low nibbles of bytes 0, 2
        const s_half2 b = __builtin_bit_cast(s_half2, w & 0x00F000F0u);     // high nibbles of bytes 0, 2 (x16)
        const s_half2 c = __builtin_bit_cast(s_half2, w8 & 0x000F000Fu);    // low nibbles of bytes 1, 3
        const s_half2 d = __builtin_bit_cast(s_half2, w8 & 0x00F000F0u);    // high nibbles of bytes 1, 3 (x16)
        alo = s_fma_h(a.x, xlo[4 * m + 0], alo);
        ahi = s_fma_h(b.x, xhi[4 * m + 0], ahi);
        alo = s_fma_h(c.x, xlo[4 * m + 1], alo);
        ahi = s_fma_h(d.x, xhi[4 * m + 1], ahi);
        alo = s_fma_h(a.y, xlo[4 * m + 2], alo);
        ahi = s_fma_h(b.y, xhi[4 * m + 2], ahi);
        alo = s_fma_h(c.y, xlo[4 * m + 3], alo);
        ahi = s_fma_h(d.y, xhi[4 * m + 3], ahi);
    }
    // 6-bit scale and min of sub-blocks 2g and 2g+1: two adjacent bytes of each
    // scale word, at bit sh
    const uint32_t y2 = hdr.y >> sh, z2 = hdr.z >> sh, w2 = hdr.w >> sh;
    const uint32_t sc_a = y2 & 0x3F3Fu, mn_a = z2 & 0x3F3Fu;
    const uint32_t sc_b = (w2 & 0x0F0Fu) | ((y2 >> 2) & 0x3030u);
    const uint32_t mn_b = ((w2 >> 4) & 0x0F0Fu) | ((z2 >> 2) & 0x3030u);
    const uint32_t sc = sel_hi ? sc_b : sc_a;
    const uint32_t mn = sel_hi ? mn_b : mn_a;
    const float sc0 = (float)(sc & 0xFFu), sc1 = (float)(sc >> 8);
    const float mn0 = (float)(mn & 0xFFu), mn1 = (float)(mn >> 8);
    const float d = half_bits_to_float(hdr.x & 0xFFFFu);
    const float dmin = half_bits_to_float(hdr.x >> 16);
    // alo carries 2^-24, ahi 2^-20
    const float t = __builtin_fmaf(sc1 * 0.0625f, ahi, sc0 * alo);
    const float u = __builtin_fmaf(mn1, xs_hi, mn0 * xs_lo);
    return __builtin_fmaf(d * 16777216.0f, t, -(dmin * u));
}

// P passes of 8 superblocks cover a row (n_blocks <= 8 * P); D rows in flight.
template <int P, int NW, int D>
__global__ __launch_bounds__(64 * NW) void q4k_stream_kernel(StreamParams p)
{
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t gw = blockIdx.x * NW + wave;
    // rows gw, gw + stride, ...: at any moment the waves of the grid read
    // consecutive rows, one contiguous stream across the memory channels
    const uint32_t stride = gridDim.x * NW;
    if (gw >= p.N) return;
    const uint32_t n_rows = (p.N - gw + stride - 1u) / stride;
    const uint32_t bl = lane >> 3, j = lane & 7u, g = j >> 1, h = j & 1u;
    const bool sel_hi = g >= 2u;
    const uint32_t sh = 16u * (g & 1u);

    float xlo[P][16], xhi[P][16], xs_lo[P], xs_hi[P];
    uint32_t hoff[P];
#pragma unroll
    for (int pass = 0; pass < P; ++pass) {
        uint32_t b = pass * 8u + bl;
        const bool valid = b < p.n_blocks;
        b = valid ? b : p.n_blocks - 1u;
        hoff[pass] = b * KQ_Q4K_BYTES;
        const float4* xp = (const float4*)(p.X + (size_t)b * KQ_QK + 64u * g + 16u * h);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float4 lo = xp[i], hi = xp[8 + i];
            if (!valid) { lo = float4{0, 0, 0, 0}; hi = lo; }
            xlo[pass][4 * i + 0] = lo.x; xlo[pass][4 * i + 1] = lo.y; xlo[pass][4 * i + 2] = lo.z; xlo[pass][4 * i + 3] = lo.w;
            xhi[pass][4 * i + 0] = hi.x; xhi[pass][4 * i + 1] = hi.y; xhi[pass][4 * i + 2] = hi.z; xhi[pass][4 * i + 3] = hi.w;
        }
        float sl = 0.0f, sh_ = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; ++i) { sl += xlo[pass][i]; sh_ += xhi[pass][i]; }
        xs_lo[pass] = sl;
        xs_hi[pass] = sh_;
    }

    s_u32x4 hdr[D][P], q[D][P];
#pragma unroll
    for (int d = 0; d < D; ++d) {
        const uint32_t r = gw + min((uint32_t)d, n_rows - 1u) * stride;
        const uint8_t* rp = p.W + (size_t)r * p.row_stride_bytes;
#pragma unroll
        for (int pass = 0; pass < P; ++pass) {
            hdr[d][pass] = *(const s_u32x4*)(rp + hoff[pass]);
            q[d][pass] = *(const s_u32x4*)(rp + hoff[pass] + 16u + 16u * j);
        }
    }
    for (uint32_t i0 = 0; i0 < n_rows; i0 += D) {
#pragma unroll
        for (int d = 0; d < D; ++d) {
            const uint32_t i = i0 + d;
            if (i < n_rows) {
                const uint32_t r = gw + i * stride;
                float acc = 0.0f;
#pragma unroll
                for (int pass = 0; pass < P; ++pass)
                    acc += q4k_piece_dot(hdr[d][pass], q[d][pass], xlo[pass], xhi[pass], xs_lo[pass], xs_hi[pass],
                                         sel_hi, sh);
                if (i + D < n_rows) {
                    const uint8_t* rp = p.W + (size_t)(r + D * stride) * p.row_stride_bytes;
#pragma unroll
                    for (int pass = 0; pass < P; ++pass) {
                        hdr[d][pass] = *(const s_u32x4*)(rp + hoff[pass]);
                        q[d][pass] = *(const s_u32x4*)(rp + hoff[pass] + 16u + 16u * j);
                    }
                }
                const float tot = wave_sum(acc);
                if (lane == 0) p.Y[p.y_offset + r] = tot + (p.bias ? p.bias[r] : 0.0f);
            }
        }
    }
}

bool gemv_stream_supported(const MatmulArgs& a)
{
    if (a.expert_idx) return false;
    if (a.M != 1) return false;
    if (a.type != KQ_TYPE_Q4_K) return false;
    if (a.n_blocks < 1 || a.n_blocks > 16) return false;
    if (((uintptr_t)a.W & 15u) || (a.row_stride_bytes & 15u)) return false;
    if (((uintptr_t)a.X & 15u)) return false;
    return true;
}

hipError_t launch_gemv_stream(const MatmulArgs& a, const GemvTuning& t, hipStream_t s)
{
    StreamParams p;
    p.X = (const float*)a.X;
    p.W = a.W;
    p.bias = a.bias;
    p.Y = a.Y;
    p.N = a.N; p.K = a.K;
    p.n_blocks = a.n_blocks;
    p.row_stride_bytes = a.row_stride_bytes;
    p.y_offset = a.y_offset;
    // about 4096 waves (16 per CU), at least two rows each so that the
    // activations are not loaded for a single row
    uint32_t rpw = t.splits > 0 ? (uint32_t)t.splits : (a.N + 4095u) / 4096u;
    if (t.splits <= 0 && rpw < 2u) rpw = 2u;
    constexpr int NW = 4;
    const uint32_t waves = (a.N + rpw - 1u) / rpw;
    const uint32_t wgs = (waves + NW - 1u) / NW;
    const int depth = t.depth > 0 ? t.depth : 2;
#define KQ_STREAM_LAUNCH(P, D) hipLaunchKernelGGL((q4k_stream_kernel<P, NW, D>), dim3(wgs), dim3(64 * NW), 0, s, p)
    if (a.n_blocks <= 8u) {
        if (depth <= 1) KQ_STREAM_LAUNCH(1, 1);
        else if (depth <= 2) KQ_STREAM_LAUNCH(1, 2);
        else KQ_STREAM_LAUNCH(1, 4);
    } else {
        if (depth <= 1) KQ_STREAM_LAUNCH(2, 1);
        else if (depth <= 2) KQ_STREAM_LAUNCH(2, 2);
        else KQ_STREAM_LAUNCH(2, 4);
    }
#undef KQ_STREAM_LAUNCH
    return hipGetLastError();
}

}  // namespace kq
