// kq_wave.h — wave-wide "largest value, lowest index" for the selection kernels (router top-k, greedy pick).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace kq {

// One step of an all-reduce over an aligned group of 2, 4, 8 or 16 lanes, taken in the order OFF = 1, 2,
// 4, 8: the partner's value as a DPP move.  Steps 1 and 2 are lane ^ 1 and lane ^ 2; steps 4 and 8 are the
// mirrors within 8 and 16 lanes, which pair every lane with one from the other half — the same thing for
// an all-reduce, since after the earlier steps all lanes of a half hold the same value.
template <int OFF>
__device__ __forceinline__ int group_partner(int x)
{
    static_assert(OFF == 1 || OFF == 2 || OFF == 4 || OFF == 8, "steps of an all-reduce over up to 16 lanes");
    constexpr int CTRL = OFF == 1 ? 0xB1 : OFF == 2 ? 0x4E : OFF == 4 ? 0x141 : 0x140;
    return __builtin_amdgcn_update_dpp(0, x, CTRL, 0xF, 0xF, false);
}
template <int OFF>
__device__ __forceinline__ float group_partner(float x)
{
    return __builtin_bit_cast(float, group_partner<OFF>(__builtin_bit_cast(int, x)));
}

// The sum over the wave, in every lane: four DPP steps inside the rows of 16, then the four rows' values.
__device__ __forceinline__ float wave_total(float v)
{
    v += group_partner<1>(v);
    v += group_partner<2>(v);
    v += group_partner<4>(v);
    v += group_partner<8>(v);
    const float a = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
    const float b = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
    const float c = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
    const float d = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
    return (a + b) + (c + d);
}

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
