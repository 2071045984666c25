// kq_format.h — GGUF Q4_K / Q6_K superblock layout and element decode (device).
//
// Q4_K, 144 B / 256 elements (runtime/gguf_loader.cpp:460-496 in the reference):
//   [0,2) d fp16 | [2,4) dmin fp16 | [4,16) 12 scale bytes | [16,144) 128 quant bytes
//   element sb*32+i: byte 16+(sb/2)*32+i, low nibble for even sb, high for odd;
//   w = (d*sc[sb])*q - (dmin*mn[sb])
// Q6_K, 210 B / 256 elements (runtime/gguf_loader.cpp:537-571):
//   [0,128) ql | [128,192) qh | [192,208) int8 scales | [208,210) d fp16
//   element 128h+32t+l: low nibble (t even) / high nibble (t>=2) of
//   ql[64h + 32(t&1) + l], bits 2t..2t+1 of qh[32h+l];
//   w = d * scale[8h + 2t + l/16] * (q - 32)
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define KQ_TYPE_Q4_K 12
#define KQ_TYPE_Q5_K 13
#define KQ_TYPE_Q6_K 14
#define KQ_QK 256
#define KQ_Q4K_BYTES 144
#define KQ_Q5K_BYTES 176
#define KQ_Q6K_BYTES 210

namespace kq {

__host__ __device__ inline uint32_t block_bytes(int type)
{
    return type == KQ_TYPE_Q4_K ? KQ_Q4K_BYTES : type == KQ_TYPE_Q5_K ? KQ_Q5K_BYTES : type == KQ_TYPE_Q6_K ? KQ_Q6K_BYTES : 0u;
}

// Exact IEEE half -> float including subnormals, infinities and NaN payloads:
// the hardware conversion, which is exact for every input.
__device__ __forceinline__ float half_bits_to_float(uint32_t h16)
{
    union { uint16_t u; _Float16 h; } v;
    v.u = (uint16_t)h16;
    return (float)v.h;
}

// 6-bit scale and min of sub-block sb from the three scale words
// (bytes 4..15 of the block read as little-endian u32).
__device__ __forceinline__ void q4k_scale_min(uint32_t u0, uint32_t u1, uint32_t u2, int sb,
                                              uint32_t& sc, uint32_t& mn)
{
    // (both layouts are computed and one is selected: a branch here cuts the caller's loop body into basic blocks)
    const int j = sb & 3;
    const uint32_t a = (u0 >> (8 * j)) & 255u;
    const uint32_t b = (u1 >> (8 * j)) & 255u;
    const uint32_t c = (u2 >> (8 * j)) & 255u;
    const bool low = sb < 4;
    sc = low ? (a & 63u) : ((c & 15u) | ((a >> 6) << 4));
    mn = low ? (b & 63u) : ((c >> 4) | ((b >> 6) << 4));
}

// Byte-granular read through the word array (any alignment of the block).
__device__ __forceinline__ uint32_t byte_at(const uint8_t* p, uint32_t off) { return p[off]; }

__device__ __forceinline__ uint32_t u16_at(const uint8_t* p, uint32_t off)
{
    return (uint32_t)p[off] | ((uint32_t)p[off + 1] << 8);
}

// One Q4_K element, bit-identical to the CPU formula: products rounded
// separately, no contraction (the products are exact in fp32 anyway).
__device__ __forceinline__ float q4k_element(const uint8_t* blk, uint32_t e)
{
    const float d = half_bits_to_float(u16_at(blk, 0));
    const float dmin = half_bits_to_float(u16_at(blk, 2));
    const uint32_t sb = e >> 5, i = e & 31u;
    uint32_t u0 = 0, u1 = 0, u2 = 0;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        u0 |= byte_at(blk, 4 + t) << (8 * t);
        u1 |= byte_at(blk, 8 + t) << (8 * t);
        u2 |= byte_at(blk, 12 + t) << (8 * t);
    }
    uint32_t sc, mn;
    q4k_scale_min(u0, u1, u2, (int)sb, sc, mn);
    const uint32_t qb = byte_at(blk, 16 + (sb >> 1) * 32 + i);
    const uint32_t q = (sb & 1u) ? (qb >> 4) : (qb & 15u);
    const float a = __fmul_rn(__fmul_rn(d, (float)sc), (float)q);
    const float b = __fmul_rn(dmin, (float)mn);
    return __fsub_rn(a, b);
}

// One Q5_K element (176-byte block: d, dmin, the Q4_K scale bytes, 32 bytes of fifth bits at 16, the
// nibbles at 48): (d*sc)*(nibble | bit<<4) - dmin*mn, rounded as the CPU formula rounds it.
__device__ __forceinline__ float q5k_element(const uint8_t* blk, uint32_t e)
{
    const float d = half_bits_to_float(u16_at(blk, 0));
    const float dmin = half_bits_to_float(u16_at(blk, 2));
    const uint32_t sb = e >> 5, i = e & 31u;
    uint32_t u0 = 0, u1 = 0, u2 = 0;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        u0 |= byte_at(blk, 4 + t) << (8 * t);
        u1 |= byte_at(blk, 8 + t) << (8 * t);
        u2 |= byte_at(blk, 12 + t) << (8 * t);
    }
    uint32_t sc, mn;
    q4k_scale_min(u0, u1, u2, (int)sb, sc, mn);
    const uint32_t qb = byte_at(blk, 48 + (sb >> 1) * 32 + i);
    const uint32_t lo = (sb & 1u) ? (qb >> 4) : (qb & 15u);
    const uint32_t q = lo | (((byte_at(blk, 16 + i) >> sb) & 1u) << 4);
    const float a = __fmul_rn(__fmul_rn(d, (float)sc), (float)q);
    const float b = __fmul_rn(dmin, (float)mn);
    return __fsub_rn(a, b);
}

// Element e of a block of any of the three types.
template <int TYPE>
__device__ __forceinline__ float kq_element(const uint8_t* blk, uint32_t e);

__device__ __forceinline__ float q6k_element(const uint8_t* blk, uint32_t e)
{
    const float d = half_bits_to_float(u16_at(blk, 208));
    const uint32_t h = e >> 7, r = e & 127u, t = r >> 5, l = r & 31u;
    const uint32_t qlb = byte_at(blk, 64 * h + 32 * (t & 1u) + l);
    const uint32_t qhb = byte_at(blk, 128 + 32 * h + l);
    const uint32_t lo = (t & 2u) ? (qlb >> 4) : (qlb & 15u);
    const int q = (int)(lo | (((qhb >> (2 * t)) & 3u) << 4)) - 32;
    const int sc = (int)(int8_t)byte_at(blk, 192 + 8 * h + 2 * t + (l >> 4));
    return __fmul_rn(__fmul_rn(d, (float)sc), (float)q);
}

template <> __device__ __forceinline__ float kq_element<KQ_TYPE_Q4_K>(const uint8_t* blk, uint32_t e) { return q4k_element(blk, e); }
template <> __device__ __forceinline__ float kq_element<KQ_TYPE_Q5_K>(const uint8_t* blk, uint32_t e) { return q5k_element(blk, e); }
template <> __device__ __forceinline__ float kq_element<KQ_TYPE_Q6_K>(const uint8_t* blk, uint32_t e) { return q6k_element(blk, e); }

}  // namespace kq
