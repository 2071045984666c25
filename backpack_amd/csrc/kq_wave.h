// kq_wave.h — wave-wide "largest value, lowest index" for the selection kernels (router top-k, greedy pick).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace kq {

// The better of two (value, index) candidates: larger value, then lower index.
__device__ __forceinline__ void best_of(float& v, uint32_t& i, float ov, uint32_t oi)
{
    const bool take = ov > v || (ov == v && oi < i);
    v = take ? ov : v;
    i = take ? oi : i;
}

// Exchanges inside a row of 16 lanes as data-parallel-primitive moves (one VALU instruction each; the
// LDS-routed shuffles cost a hundred cycles apiece, and a selection chains dozens of them).
template <int CTRL>
__device__ __forceinline__ void best_dpp_step(float& v, uint32_t& i)
{
    const float ov = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
    const uint32_t oi = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)i, CTRL, 0xF, 0xF, false);
    best_of(v, i, ov, oi);
}

// The best (value, index) of the wave, in every lane.
__device__ __forceinline__ void wave_best(float& v, uint32_t& i)
{
    best_dpp_step<0xB1>(v, i);    // quad: lanes ^ 1
    best_dpp_step<0x4E>(v, i);    // quad: lanes ^ 2
    best_dpp_step<0x141>(v, i);   // mirror within 8
    best_dpp_step<0x140>(v, i);   // mirror within 16
    float bv = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
    uint32_t bi = (uint32_t)__builtin_amdgcn_readlane((int)i, 0);
#pragma unroll
    for (int r = 16; r < 64; r += 16)
        best_of(bv, bi, __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), r)),
                (uint32_t)__builtin_amdgcn_readlane((int)i, r));
    v = bv;
    i = bi;
}

}  // namespace kq
