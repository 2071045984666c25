// kq_mgemv.hip — decode matvec (one token) for Q4_K matrices of many rows, contraction on the matrix cores.
//
// The lanes-along-K kernel (kq_stream.hip) spends three vector instructions per weight — one multiply-add, the
// nibble masks and the scale arithmetic — and on a 28672 x 4096 matrix that arithmetic, not HBM, sets its
// pace (counters: vector ALUs busy three quarters of the launch).  Here the multiply-adds move to
// v_mfma_f32_16x16x32_f16 and the scale arithmetic is paid once per superblock instead of once per sub-block:
//
//  - B = weights: lane (n = l%16, g = l/16) holds eight consecutive quant bytes of row n; their low nibbles are
//    eight elements of sub-block 2c, their high nibbles eight of 2c+1, left in the mantissa of fp16 subnormals
//    (q * 2^-24, q * 2^-20), ten bit-ops per sixteen weights.
//  - A = the token: one token needs two of the sixteen rows of A (x = hi + lo, two fp16 of 11 bits each after a
//    power-of-two scale per superblock), so the sixteen rows carry the EIGHT sub-blocks of a superblock: row sb
//    holds hi(x) of sub-block sb for the instruction that multiplies sub-block sb and zeros for the other seven,
//    row sb + 8 the same for lo(x).  Eight instructions accumulate into ONE 16 x 16 tile whose row sb is the sum
//    over sub-block sb; a lane then holds four sub-block sums of its weight row and applies four scales at once.
//    The A operands depend on x only: a wave builds them once and reuses them for every tile of rows it walks.
//  - the minima: sum_sb mn[sb] * sum(x over sb), four multiply-adds per lane and superblock.
//
// A workgroup of eight waves owns tiles of 16 rows; wave w owns superblocks 2w and 2w+1 of every row (K <= 4096),
// its partial sums meet the other waves' in LDS once per eight tiles.  Weights travel HBM -> registers -> a
// window of LDS private to the wave in 16-byte units that are consecutive along a row (every cache line is
// fetched once and whole), and the lanes read their 8-byte pieces from there.
//
// Three tiles of weights are in flight per wave; their loads are issued from inline asm and waited for by hand
// (the compiler's own placement drains the whole queue at every refill inside a loop), under the rules written
// out in kq_stream_core.h: KQ_REQUIRES_NO_SPILL, every register a load fills passes through the wait that
// names it, the number of loads in flight is the same at every wait (past its last tile a wave issues its
// requests with no lane active).  The ring lives in straight-line code here (KQ_RING_STRAIGHT_LINE), so the
// build also reads the listing top to bottom and refuses any instruction that mentions a register between its
// load and its wait.
//
// Results differ from the lanes-along-K kernel's by the hi + lo split of x: 22 bits relative to the largest
// |x| of a superblock.
#include "kq_format.h"
#include "kq_kernels.h"
#include "kq_stream_core.h"
#include "kq_wave.h"

namespace kq {

typedef _Float16 g_half8 __attribute__((ext_vector_type(8)));
typedef float g_f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t g_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t g_u32x2 __attribute__((ext_vector_type(2)));

// S superblocks per wave, WAVES waves per workgroup: S * WAVES = 16 superblocks = K 4096 at most.
template <int S, int WAVES>
struct MgGeo {
    static constexpr int SPAN = S * KQ_Q4K_BYTES;            // bytes of a row a wave covers
    static constexpr int UPR = SPAN / 16;                    // 16-byte units per row
    static constexpr int NU = (16 * UPR + 63) / 64;          // units per lane
    static constexpr int PITCH = S == 1 ? 160 : 304;         // window row pitch: the 16 rows start in different banks
    static constexpr int WIN = 16 * PITCH;
};
constexpr int MG_DEPTH = 2;                          // tiles in flight per wave (three measured slower: 14.6 against 13.7 us)
constexpr int MG_GROUP = 8;                          // tiles between two meetings of the waves

__device__ __forceinline__ void mg_window_fence()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// A 16-byte load at base (uniform) + off (per lane), waited for by hand (ring_load16 of kq_stream_core.h with a
// scalar base: no 64-bit address arithmetic on the vector units).
__device__ __forceinline__ void mg_load16(g_u32x4& v, uint32_t off, const uint8_t* base)
{
#ifdef KQ_TRACKED_LOADS
    v = *(const g_u32x4*)(base + off);
#else
    asm volatile("global_load_dwordx4 %0, %1, %2 ; ringld" : "+v"(v) : "v"(off), "s"(base));
#endif
}

// The loads of one tile as one statement, issued with no lane active when `on` is zero: such a load moves nothing
// but keeps its place in the memory counter, so the number of loads in flight is the same at every wait and a
// wave past its last tile requests nothing real.  (One statement: the compiler must not place an instruction of
// its own between the change of EXEC and its restoration.)
__device__ __forceinline__ void mg_request(g_u32x4 (&d)[5], const uint32_t (&o)[5], const uint8_t* base, uint32_t on)
{
#ifdef KQ_TRACKED_LOADS
    if (on)
        for (int k = 0; k < 5; ++k) d[k] = *(const g_u32x4*)(base + o[k]);
#else
    uint64_t saved;
    asm volatile("s_mov_b64 %[sv], exec\n\t"
                 "s_and_b32 exec_lo, exec_lo, %[on]\n\t"
                 "s_and_b32 exec_hi, exec_hi, %[on]\n\t"
                 "global_load_dwordx4 %0, %6, %[b] ; ringld\n\t"
                 "global_load_dwordx4 %1, %7, %[b] ; ringld\n\t"
                 "global_load_dwordx4 %2, %8, %[b] ; ringld\n\t"
                 "global_load_dwordx4 %3, %9, %[b] ; ringld\n\t"
                 "global_load_dwordx4 %4, %10, %[b] ; ringld\n\t"
                 "s_mov_b64 exec, %[sv]"
                 : "+v"(d[0]), "+v"(d[1]), "+v"(d[2]), "+v"(d[3]), "+v"(d[4]), [sv] "=&s"(saved)
                 : "v"(o[0]), "v"(o[1]), "v"(o[2]), "v"(o[3]), "v"(o[4]), [b] "s"(base), [on] "s"(on));
#endif
}
__device__ __forceinline__ void mg_request(g_u32x4 (&d)[3], const uint32_t (&o)[3], const uint8_t* base, uint32_t on)
{
#ifdef KQ_TRACKED_LOADS
    if (on)
        for (int k = 0; k < 3; ++k) d[k] = *(const g_u32x4*)(base + o[k]);
#else
    uint64_t saved;
    asm volatile("s_mov_b64 %[sv], exec\n\t"
                 "s_and_b32 exec_lo, exec_lo, %[on]\n\t"
                 "s_and_b32 exec_hi, exec_hi, %[on]\n\t"
                 "global_load_dwordx4 %0, %4, %[b] ; ringld\n\t"
                 "global_load_dwordx4 %1, %5, %[b] ; ringld\n\t"
                 "global_load_dwordx4 %2, %6, %[b] ; ringld\n\t"
                 "s_mov_b64 exec, %[sv]"
                 : "+v"(d[0]), "+v"(d[1]), "+v"(d[2]), [sv] "=&s"(saved)
                 : "v"(o[0]), "v"(o[1]), "v"(o[2]), [b] "s"(base), [on] "s"(on));
#endif
}

// Every register of a buffer passes through the wait that leaves N younger loads in flight.
template <int N>
__device__ __forceinline__ void mg_wait(g_u32x4 (&b)[5])
{
#ifndef KQ_TRACKED_LOADS
    asm volatile("s_waitcnt vmcnt(%5) ; ringwait %0 %1 %2 %3 %4" : "+v"(b[0]), "+v"(b[1]), "+v"(b[2]), "+v"(b[3]), "+v"(b[4]) : "n"(N));
#endif
}
template <int N>
__device__ __forceinline__ void mg_wait(g_u32x4 (&b)[3])
{
#ifndef KQ_TRACKED_LOADS
    asm volatile("s_waitcnt vmcnt(%3) ; ringwait %0 %1 %2" : "+v"(b[0]), "+v"(b[1]), "+v"(b[2]) : "n"(N));
#endif
}
template <int N>
__device__ __forceinline__ void mg_wait_x(g_u32x4 (&x)[2][2])
{
#ifndef KQ_TRACKED_LOADS
    asm volatile("s_waitcnt vmcnt(%4) ; ringwait %0 %1 %2 %3" : "+v"(x[0][0]), "+v"(x[0][1]), "+v"(x[1][0]), "+v"(x[1][1]) : "n"(N));
#endif
}
template <int N>
__device__ __forceinline__ void mg_wait_x(g_u32x4 (&x)[1][2])
{
#ifndef KQ_TRACKED_LOADS
    asm volatile("s_waitcnt vmcnt(%2) ; ringwait %0 %1" : "+v"(x[0][0]), "+v"(x[0][1]) : "n"(N));
#endif
}

// The sum over the four lanes l%16, l%16 + 16, + 32, + 48, in all of them: two register swaps between rows of
// 16 and halves of 32 lanes (vector instructions; a shuffle through LDS costs a hundred cycles).
__device__ __forceinline__ float mg_sum_over_g(float v)
{
    const unsigned u = __builtin_bit_cast(unsigned, v);
    const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    const unsigned r0 = r[0], r1 = r[1];   // (components through plain scalars, see the note on __builtin_bit_cast below)
    const float s = __builtin_bit_cast(float, r0) + __builtin_bit_cast(float, r1);
    const unsigned us = __builtin_bit_cast(unsigned, s);
    const auto q = __builtin_amdgcn_permlane32_swap(us, us, false, false);
    const unsigned q0 = q[0], q1 = q[1];
    return __builtin_bit_cast(float, q0) + __builtin_bit_cast(float, q1);
}

// KQ_KERNARG_PRELOAD: scalar arguments, the first of them arrive in scalar registers with the wave.
template <int S, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void q4k_mgemv_kernel(const uint8_t* __restrict__ W, const float* __restrict__ X,
                                                               float* __restrict__ Y, const float* __restrict__ bias,
                                                               uint32_t N, uint32_t n_blocks, uint32_t row_stride,
                                                               uint32_t n_tiles, uint32_t G)
{
    using Geo = MgGeo<S, WAVES>;
    constexpr int NU = Geo::NU, UPR = Geo::UPR, PITCH = Geo::PITCH;
    __shared__ __align__(16) uint8_t win_all[WAVES * Geo::WIN];
    __shared__ float red[2][MG_GROUP][WAVES][16];
    __shared__ __align__(16) float xpart[WAVES][S][8][4];

    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t n = lane & 15u, g = lane >> 4;
    uint8_t* win = win_all + wave * Geo::WIN;
    const uint32_t b0 = wave * S;
    const uint32_t row_bytes = n_blocks * KQ_Q4K_BYTES;
    const uint32_t wg = blockIdx.x;
    const uint32_t n_i = (n_tiles - wg + G - 1u) / G;   // tiles this workgroup walks (the grid has at most n_tiles workgroups)

    // ---- requests: the token's elements first, then the first tiles (weights never depend on x) --------------
    // as a holder of A, lane (m = l%16, g) owns eight k of sub-block m%8: hi part for m < 8, lo part for m >= 8
    const uint32_t sbA = n & 7u, part = n >> 3;
    g_u32x4 xr[S][2] = {};
    bool live[S];
#pragma unroll
    for (int s = 0; s < S; ++s) {
        live[s] = b0 + s < n_blocks;
        const uint32_t b = min(b0 + (uint32_t)s, n_blocks - 1u);
        const uint32_t at = (b * KQ_QK + sbA * 32u + g * 8u) * 4u;
        mg_load16(xr[s][0], at, (const uint8_t*)X);
        mg_load16(xr[s][1], at + 16u, (const uint8_t*)X);
    }
    // staging units of this lane: unit u = (row u / UPR, 16-byte column u % UPR) of the wave's span
    uint32_t u_src[NU], u_dst[NU];
#pragma unroll
    for (int i = 0; i < NU; ++i) {
        const uint32_t u = min((uint32_t)i * 64u + lane, 16u * UPR - 1u);   // spare lanes repeat the last unit
        const uint32_t r = u / UPR, c = u - r * UPR;
        const uint32_t o = b0 * KQ_Q4K_BYTES + c * 16u;
        u_src[i] = r * row_stride + (o < row_bytes ? o : row_bytes - 16u);   // units of superblocks that do not exist: never multiplied
        u_dst[i] = r * PITCH + c * 16u;
    }
    // tile i of this workgroup covers rows row0 .. row0 + 15; the matrix's last tile is moved up so that it ends
    // at row N - 1 (its first rows then repeat the tile before it and are not stored)
    auto tile_row0 = [&](uint32_t i) { return min(min(wg + i * G, n_tiles - 1u) * 16u, N - 16u); };
    g_u32x4 raw[MG_DEPTH][NU] = {};
    auto request = [&](uint32_t i, g_u32x4 (&dst)[NU]) {
        const uint8_t* base = W + (size_t)tile_row0(i) * row_stride;
        // past the last tile: a request of no lanes
        mg_request(dst, u_src, base, (uint32_t)__builtin_amdgcn_readfirstlane(i < n_i ? -1 : 0));
    };
#pragma unroll
    for (int d = 0; d < MG_DEPTH; ++d) request((uint32_t)d, raw[d]);
    mg_wait_x<MG_DEPTH * NU>(xr);

    // ---- the token's operands for this wave's superblocks ------------------------------------------------
    g_half8 Aop[S][8];
    float SX[S][4], c24[S];
#pragma unroll
    for (int s = 0; s < S; ++s) {
        // (through a plain uint32_t: __builtin_bit_cast applied to a vector's component reads component 0)
        float xv[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t bits = xr[s][i >> 2][i & 3];
            xv[i] = __builtin_bit_cast(float, bits);
        }
        uint32_t amax = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) amax = max(amax, __builtin_bit_cast(uint32_t, xv[i]) & 0x7FFFFFFFu);
        amax = max(amax, (uint32_t)group_partner<1>((int)amax));
        amax = max(amax, (uint32_t)group_partner<2>((int)amax));
        amax = max(amax, (uint32_t)group_partner<4>((int)amax));
        amax = max(amax, (uint32_t)group_partner<8>((int)amax));
        amax = max(max((uint32_t)__builtin_amdgcn_readlane((int)amax, 0), (uint32_t)__builtin_amdgcn_readlane((int)amax, 16)),
                   max((uint32_t)__builtin_amdgcn_readlane((int)amax, 32), (uint32_t)__builtin_amdgcn_readlane((int)amax, 48)));
        uint32_t e = amax >> 23;                  // biased exponent of the superblock's largest |x|
        e = e < 15u ? 15u : (e > 253u ? 253u : e);
        const float sc = __builtin_bit_cast(float, (268u - e) << 23);       // amax * sc in [2^14, 2^15)
        c24[s] = __builtin_bit_cast(float, (e - 14u) << 23) * 16777216.0f;  // 1 / sc, and the nibbles' 2^24
        _Float16 h[8];
        float psum = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float a = xv[i] * sc;
            const _Float16 hi = (_Float16)a;
            h[i] = part ? (_Float16)(a - (float)hi) : hi;
            psum += xv[i];
        }
        const g_half8 mine = {h[0], h[2], h[1], h[3], h[4], h[6], h[5], h[7]};
        const g_half8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < 8; ++j) Aop[s][j] = (sbA == (uint32_t)j && live[s]) ? mine : zero;
        if (part == 0u) xpart[wave][s][sbA][g] = psum;
    }
    mg_window_fence();
#pragma unroll
    for (int s = 0; s < S; ++s) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float4 p = *(const float4*)&xpart[wave][s][4u * (g & 1u) + r][0];
            SX[s][r] = g < 2u ? (p.x + p.y) + (p.z + p.w) : 0.0f;   // the minima are counted once: by the hi lanes
        }
    }
    // ---- tiles -------------------------------------------------------------------------------------------
    auto tile = [&](uint32_t i, g_u32x4 (&buf)[NU]) {
        mg_wait<(MG_DEPTH - 1) * NU>(buf);   // the other buffers' loads stay in flight
#pragma unroll
        for (int k = 0; k < NU; ++k) *(g_u32x4*)(win + u_dst[k]) = buf[k];
        request(i + MG_DEPTH, buf);
        mg_window_fence();
        float tot = 0.0f;
        const uint8_t* rowp = win + n * PITCH;
        g_u32x4 hdr[S];
        g_u32x2 w[S][4];
#pragma unroll
        for (int s = 0; s < S; ++s) {
            hdr[s] = *(const g_u32x4*)(rowp + s * KQ_Q4K_BYTES);
#pragma unroll
            for (int c = 0; c < 4; ++c) w[s][c] = *(const g_u32x2*)(rowp + s * KQ_Q4K_BYTES + 16 + 32 * c + 8u * g);
        }
        g_f32x4 D[S];
#pragma unroll
        for (int s = 0; s < S; ++s) D[s] = g_f32x4{0, 0, 0, 0};
        // the superblocks' chains of eight dependent instructions take turns
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            g_u32x4 blo[S], bhi[S];
#pragma unroll
            for (int s = 0; s < S; ++s) {
                const uint32_t d0 = w[s][c].x, d1 = w[s][c].y;
                const uint32_t e0 = d0 >> 8, e1 = d1 >> 8;
                blo[s] = g_u32x4{d0 & 0x000F000Fu, e0 & 0x000F000Fu, d1 & 0x000F000Fu, e1 & 0x000F000Fu};
                bhi[s] = g_u32x4{d0 & 0x00F000F0u, e0 & 0x00F000F0u, d1 & 0x00F000F0u, e1 & 0x00F000F0u};
            }
#pragma unroll
            for (int s = 0; s < S; ++s)
                D[s] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Aop[s][2 * c], __builtin_bit_cast(g_half8, blo[s]), D[s], 0, 0, 0);
#pragma unroll
            for (int s = 0; s < S; ++s)
                D[s] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Aop[s][2 * c + 1], __builtin_bit_cast(g_half8, bhi[s]), D[s], 0, 0, 0);
        }
        // lane (n, g): D[r] is the sum over sub-block 4*(g&1) + r of row n (hi part for g < 2, lo part beyond)
#pragma unroll
        for (int s = 0; s < S; ++s) {
            if (!live[s]) continue;   // wave-uniform
            const g_u32x4 hd = hdr[s];
            const float d = half_bits_to_float(hd.x & 0xFFFFu);
            const float dmin = half_bits_to_float(hd.x >> 16);
            const uint32_t scA = hd.y & 0x3F3F3F3Fu, mnA = hd.z & 0x3F3F3F3Fu;
            const uint32_t scB = (hd.w & 0x0F0F0F0Fu) | ((hd.y >> 2) & 0x30303030u);
            const uint32_t mnB = ((hd.w >> 4) & 0x0F0F0F0Fu) | ((hd.z >> 2) & 0x30303030u);
            const uint32_t scw = (g & 1u) ? scB : scA, mnw = (g & 1u) ? mnB : mnA;
            const float s0 = (float)(scw & 255u), s1 = (float)((scw >> 8) & 255u);
            const float s2 = (float)((scw >> 16) & 255u), s3 = (float)(scw >> 24);
            const float m0 = (float)(mnw & 255u), m1 = (float)((mnw >> 8) & 255u);
            const float m2 = (float)((mnw >> 16) & 255u), m3 = (float)(mnw >> 24);
            // the high nibbles (odd sub-blocks) sit four bits up
            const float U = fmaf(fmaf(s1, D[s][1], s3 * D[s][3]), 0.0625f, fmaf(s0, D[s][0], s2 * D[s][2]));
            const float V = fmaf(m0, SX[s][0], m1 * SX[s][1]) + fmaf(m2, SX[s][2], m3 * SX[s][3]);
            tot += fmaf(d * c24[s], U, -(dmin * V));
        }
        tot = mg_sum_over_g(tot);
        if (g == 0u) red[(i / MG_GROUP) & 1u][i % MG_GROUP][wave][n] = tot;
    };
    auto meet = [&](uint32_t i_last) {
        // tiles [first, i_last] of this round: the first of them are folded by a wave each, 64 / WAVES rows per pass
        __syncthreads();
        const uint32_t first = i_last - i_last % MG_GROUP, cnt = i_last - first + 1u;
        const uint32_t rb = (first / MG_GROUP) & 1u;
        // lane (row nn, part q) of wave j: tile first + j (+ WAVES for a second pass when WAVES < MG_GROUP)
        constexpr int LPR = 64 / 16;   // lanes per row
        const uint32_t nn = lane >> 2, q = lane & 3u;
        for (uint32_t j = wave; j < cnt; j += WAVES) {
            float sum = 0.0f;
#pragma unroll
            for (int k = 0; k < WAVES / LPR; ++k) sum += red[rb][j][q * (WAVES / LPR) + k][nn];
            sum += group_partner<1>(sum);
            sum += group_partner<2>(sum);
            const uint32_t t = wg + (first + j) * G;
            const uint32_t row = tile_row0(first + j) + nn;
            if (q == 0u && row >= t * 16u) Y[row] = sum + (bias ? bias[row] : 0.0f);
        }
    };
    for (uint32_t i0 = 0; i0 < n_i; i0 += MG_DEPTH) {
#pragma unroll
        for (int d = 0; d < MG_DEPTH; ++d) {
            const uint32_t i = i0 + d;
            if (i < n_i) {
                tile(i, raw[d]);
                if ((i % MG_GROUP) == MG_GROUP - 1u || i == n_i - 1u) meet(i);
            }
        }
    }
#ifndef KQ_TRACKED_LOADS
    asm volatile("s_waitcnt vmcnt(0)");   // nothing is in flight when the wave ends
#endif
}

bool mgemv_supported(const MatmulArgs& a)
{
    if (a.type != KQ_TYPE_Q4_K || a.M != 1u || a.expert_idx || a.pro || a.epi || a.residual) return false;
    if (a.n_blocks == 0u || a.n_blocks > 16u || a.N < 16u) return false;
    if ((uint64_t)16u * a.row_stride_bytes > 0x7FFFFFFFull || (uint64_t)a.K * 4u > 0x7FFFFFFFull) return false;   // 32-bit offsets
    if (((uintptr_t)a.W & 15u) || (a.row_stride_bytes & 15u) || ((uintptr_t)a.X & 15u)) return false;
    return true;
}

hipError_t launch_mgemv(const MatmulArgs& a, uint32_t cus, int form, hipStream_t s)
{
    const uint32_t n_tiles = (a.N + 15u) / 16u;
    const uint32_t G = n_tiles < cus ? n_tiles : cus;
    if (form == 1)
        hipLaunchKernelGGL((q4k_mgemv_kernel<1, 16>), dim3(G), dim3(1024), 0, s, a.W, (const float*)a.X, a.Y + a.y_offset, a.bias,
                           a.N, a.n_blocks, a.row_stride_bytes, n_tiles, G);
    else
        hipLaunchKernelGGL((q4k_mgemv_kernel<2, 8>), dim3(G), dim3(512), 0, s, a.W, (const float*)a.X, a.Y + a.y_offset, a.bias,
                           a.N, a.n_blocks, a.row_stride_bytes, n_tiles, G);
    return hipGetLastError();
}

}  // namespace kq
