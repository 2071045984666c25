// kq_gemm.hip — prefill dequant-GEMM: Y[M,N] = X[M,K] (bf16) * dequant(W)[N,K]^T.
//
// A workgroup owns a BM x BN tile of Y and walks K in steps of 64.  Per step the
// X tile is copied to LDS as is, and the W tile is dequantised from its Q4_K /
// Q6_K bytes to bf16 (fp32 arithmetic, one RNE rounding) straight into LDS, so
// weights cross HBM as 4.5 / 6.56 bits per element and are expanded once per
// BM tokens.  The waves contract their part of the tile with
// v_mfma_f32_32x32x16_bf16, fp32 accumulation in registers.  LDS is
// double-buffered with one barrier per step.
//
// Two kernels:
//  - 256 x 256 tile, 8 waves (2 x 4, 128 x 64 each, two per SIMD), persistent.  Every wave runs the same
//    software-pipelined schedule: a step is four k slices of 16; in a slice the wave issues the LDS operand
//    reads of the next slice, the 8 matrix instructions of this slice and, between them, a quarter of its
//    share of the next tile (X piece copied, 8 weights dequantised, the global loads that refill the
//    registers just freed).  The step's barrier sits before the last slice, whose operands are already in
//    registers, so the matrix cores have work the moment the barrier opens.  The walk over (tile, k step)
//    units is either one tile per workgroup or cut into equal shares per CU ("stream-K"): a tile cut
//    between workgroups is summed into Y with fp32 atomics after a small kernel has cleared it (two
//    addends per element in the common case, so the sum does not depend on their order).
//  - 128 x 128 tile, 4 waves (2 x 2), two workgroups per CU: for shapes whose 256-tiles would leave half
//    the CUs idle and whose K is too short to be worth cutting.
//
// LDS rows are 64 bf16 + 16 bytes of padding (144 B = an odd number of 16-byte
// slots), which makes the 128-bit fragment reads of 32 consecutive rows
// conflict-free.
//
// Operand roles: MFMA A = X (i = token), B = W (j = weight row), so the lane
// index of the accumulator is the weight row and a register's 32 lanes store
// 32 consecutive floats of one Y row.
#include "kq_format.h"
#include "kq_kernels.h"
#include "kq_gemm_plan.h"
#include <type_traits>

namespace kq {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int GEMM_BK = 64;
constexpr int GEMM_LD = GEMM_BK * 2 + 16;   // bytes per LDS row

struct GemmParams {
    const uint16_t* X;   // bf16 [M,K]
    const uint8_t* W;
    const float* bias;
    float* Y;
    uint32_t M, N, K, n_blocks, row_stride_bytes, ldy;
    // walk of the persistent kernel: units = k steps (of 64) of all 256 x 256 tiles, tile after tile
    // (tiles of one token block next to each other), cut into equal shares
    uint32_t tiles_n, units, units_per_wg;
    // runs that cover part of a tile leave their sums here: two slots of 256 x 256 floats per workgroup
    float* partial;
};

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi)
{
    f32x2 v = {lo, hi};
    bf16x2 b = __builtin_convertvector(v, bf16x2);
    return __builtin_bit_cast(uint32_t, b);
}

// 32 consecutive elements of one Q4_K sub-block -> 32 bf16 (64 bytes) in LDS.
// kc = 64-element chunk of the row (sub-block pair), hf = which of the pair.
__device__ __forceinline__ void q4k_load(const uint8_t* row, uint32_t kc, uint32_t (&raw)[12])
{
    const uint8_t* blk = row + (size_t)(kc >> 2) * KQ_Q4K_BYTES;
    const u32x4 h = *(const u32x4*)blk;
    const u32x4* q = (const u32x4*)(blk + 16 + (kc & 3u) * 32u);
    const u32x4 q0 = q[0], q1 = q[1];
    raw[0] = h.x; raw[1] = h.y; raw[2] = h.z; raw[3] = h.w;
    raw[4] = q0.x; raw[5] = q0.y; raw[6] = q0.z; raw[7] = q0.w;
    raw[8] = q1.x; raw[9] = q1.y; raw[10] = q1.z; raw[11] = q1.w;
}

__device__ __forceinline__ void q4k_expand(const uint32_t (&raw)[12], uint32_t kc, uint32_t hf, uint8_t* dst)
{
    const float d = half_bits_to_float(raw[0] & 0xFFFFu);
    const float dmin = half_bits_to_float(raw[0] >> 16);
    uint32_t sc, mn;
    q4k_scale_min(raw[1], raw[2], raw[3], (int)((kc & 3u) * 2u + hf), sc, mn);
    const float a = d * (float)sc;
    const float nb = -(dmin * (float)mn);
    const uint32_t sh = hf * 4u;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        u32x4 out;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint32_t w = (raw[4 + v * 2 + j] >> sh) & 0x0F0F0F0Fu;
            const float f0 = fmaf(a, (float)(w & 255u), nb);
            const float f1 = fmaf(a, (float)((w >> 8) & 255u), nb);
            const float f2 = fmaf(a, (float)((w >> 16) & 255u), nb);
            const float f3 = fmaf(a, (float)(w >> 24), nb);
            out[j * 2] = pack_bf16(f0, f1);
            out[j * 2 + 1] = pack_bf16(f2, f3);
        }
        *(u32x4*)(dst + v * 16) = out;
    }
}

// Q5_K: the Q4_K layout with the quants 32 bytes further on and, before them, the 32 bytes of fifth bits
// (bit sb of byte i belongs to element i of sub-block sb).
__device__ __forceinline__ void q5k_load(const uint8_t* row, uint32_t kc, uint32_t (&raw)[20])
{
    const uint8_t* blk = row + (size_t)(kc >> 2) * KQ_Q5K_BYTES;
    const u32x4 h = *(const u32x4*)blk;
    const u32x4 b0 = *(const u32x4*)(blk + 16), b1 = *(const u32x4*)(blk + 32);
    const u32x4* q = (const u32x4*)(blk + 48 + (kc & 3u) * 32u);
    const u32x4 q0 = q[0], q1 = q[1];
    raw[0] = h.x; raw[1] = h.y; raw[2] = h.z; raw[3] = h.w;
    raw[4] = q0.x; raw[5] = q0.y; raw[6] = q0.z; raw[7] = q0.w;
    raw[8] = q1.x; raw[9] = q1.y; raw[10] = q1.z; raw[11] = q1.w;
    raw[12] = b0.x; raw[13] = b0.y; raw[14] = b0.z; raw[15] = b0.w;
    raw[16] = b1.x; raw[17] = b1.y; raw[18] = b1.z; raw[19] = b1.w;
}

__device__ __forceinline__ void q5k_expand(const uint32_t (&raw)[20], uint32_t kc, uint32_t hf, uint8_t* dst)
{
    const float d = half_bits_to_float(raw[0] & 0xFFFFu);
    const float dmin = half_bits_to_float(raw[0] >> 16);
    const uint32_t sb = (kc & 3u) * 2u + hf;
    uint32_t sc, mn;
    q4k_scale_min(raw[1], raw[2], raw[3], (int)sb, sc, mn);
    const float a = d * (float)sc;
    const float nb = -(dmin * (float)mn);
    const uint32_t sh = hf * 4u;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        u32x4 out;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint32_t w = ((raw[4 + v * 2 + j] >> sh) & 0x0F0F0F0Fu) | (((raw[12 + v * 2 + j] >> sb) & 0x01010101u) << 4);
            const float f0 = fmaf(a, (float)(w & 255u), nb);
            const float f1 = fmaf(a, (float)((w >> 8) & 255u), nb);
            const float f2 = fmaf(a, (float)((w >> 16) & 255u), nb);
            const float f3 = fmaf(a, (float)(w >> 24), nb);
            out[j * 2] = pack_bf16(f0, f1);
            out[j * 2 + 1] = pack_bf16(f2, f3);
        }
        *(u32x4*)(dst + v * 16) = out;
    }
}

// Q6_K: chunk kc of the row covers elements 64*kc .. 64*kc+63 = (half h, t pair);
// hf picks t.  Blocks are only 2-byte aligned, so bytes are fetched as u16.
struct Q6Raw {
    uint32_t ql[8], qh[8];
    uint32_t sc2;   // the two int8 scales of this run of 32 elements
    uint32_t d16;
};

__device__ __forceinline__ void q6k_load(const uint8_t* row, uint32_t kc, uint32_t hf, Q6Raw& r)
{
    const uint32_t c = kc & 3u, h = c >> 1, t = (c & 1u) * 2u + hf;
    const uint8_t* blk = row + (size_t)(kc >> 2) * KQ_Q6K_BYTES;
    // 2-byte aligned 128-bit loads: the hardware takes them as they are
    u32x4 a0, a1, b0, b1;
    __builtin_memcpy(&a0, blk + 64u * h + 32u * (t & 1u), 16);
    __builtin_memcpy(&a1, blk + 64u * h + 32u * (t & 1u) + 16u, 16);
    __builtin_memcpy(&b0, blk + 128u + 32u * h, 16);
    __builtin_memcpy(&b1, blk + 128u + 32u * h + 16u, 16);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        r.ql[i] = a0[i]; r.ql[4 + i] = a1[i];
        r.qh[i] = b0[i]; r.qh[4 + i] = b1[i];
    }
    uint16_t s2, d2;
    __builtin_memcpy(&s2, blk + 192u + 8u * h + 2u * t, 2);
    __builtin_memcpy(&d2, blk + 208u, 2);
    r.sc2 = s2;
    r.d16 = d2;
}

__device__ __forceinline__ void q6k_expand(const Q6Raw& r, uint32_t kc, uint32_t hf, uint8_t* dst)
{
    const uint32_t t = ((kc & 3u) & 1u) * 2u + hf;
    const float d = half_bits_to_float(r.d16);
    const float s0 = d * (float)(int)(int8_t)(r.sc2 & 255u);
    const float s1 = d * (float)(int)(int8_t)(r.sc2 >> 8);
    const uint32_t lsh = (t & 2u) ? 4u : 0u;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        u32x4 out;
        const float s = v < 2 ? s0 : s1;   // elements 0..15 / 16..31 of the run
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint32_t lo = (r.ql[v * 2 + j] >> lsh) & 0x0F0F0F0Fu;
            const uint32_t hi = ((r.qh[v * 2 + j] >> (2u * t)) & 0x03030303u) << 4;
            const uint32_t q = lo | hi;   // four 6-bit stored values
            const float f0 = s * (float)((int)(q & 255u) - 32);
            const float f1 = s * (float)((int)((q >> 8) & 255u) - 32);
            const float f2 = s * (float)((int)((q >> 16) & 255u) - 32);
            const float f3 = s * (float)((int)(q >> 24) - 32);
            out[j * 2] = pack_bf16(f0, f1);
            out[j * 2 + 1] = pack_bf16(f2, f3);
        }
        *(u32x4*)(dst + v * 16) = out;
    }
}

// Epilogue of both kernels.  Accumulator register r of lane l of a 32 x 32 block: token row
// 8*(r/4) + 4*(l/32) + r%4, weight row l%32, so a register's 32 lanes store 128 contiguous bytes of one Y
// row.  A wave whose rows all exist stores without per-row branches: a branch per store would make every
// store wait for the one before it (the bias load keeps the memory counter ambiguous at each join).
template <int TM, int TN, bool ATOMIC = false>
__device__ __forceinline__ void store_acc(const GemmParams& p, const f32x16 (&acc)[TM][TN], uint32_t m_base, uint32_t n_base,
                                          uint32_t lane, bool with_bias = true)
{
    const bool full = m_base + TM * 32u <= p.M;   // wave-uniform
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const uint32_t n = n_base + j * 32u + (lane & 31u);
        if (n >= p.N) continue;
        const float bias = (p.bias && with_bias) ? p.bias[n] : 0.0f;
        float* y = p.Y + (size_t)(m_base + 4u * (lane >> 5)) * p.ldy + n;
        auto put = [&](float* dst, float v) {
            if (ATOMIC) __builtin_amdgcn_global_atomic_fadd_f32(dst, v);   // no return value: fire and forget
            else *dst = v;
        };
        if (full) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    put(y + (size_t)(i * 32 + 8 * (r >> 2) + (r & 3)) * p.ldy, acc[i][j][r] + bias);
        } else {
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const uint32_t dm = i * 32 + 8 * (r >> 2) + (r & 3);
                    if (m_base + 4u * (lane >> 5) + dm < p.M) put(y + (size_t)dm * p.ldy, acc[i][j][r] + bias);
                }
        }
    }
}

template <int TYPE, int BM, int BN, int NWAVES>
__global__ __launch_bounds__(64 * NWAVES) void gemm_bf16_kernel(GemmParams p)
{
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr int NT = 64 * NWAVES;
    constexpr int WAVES_N = NWAVES / 2;                       // waves are laid out 2 (M) x NWAVES/2 (N)
    constexpr int WM = BM / 2, WN = BN / WAVES_N, TM = WM / 32, TN = WN / 32;
    constexpr int A_BYTES = BM * GEMM_LD, B_BYTES = BN * GEMM_LD;
    constexpr int XROWS = NT / 8;         // X rows per pass: 8 threads x 16 bytes per row
    constexpr int XP = BM / XROWS;        // X passes
    constexpr int WI = BN * 2 / NT;       // W items (row, 32-element run) per thread
    uint8_t* As = smem;
    uint8_t* Bs = smem + 2 * A_BYTES;

    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t wm = wave / WAVES_N, wn = wave % WAVES_N;
    const uint32_t m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const uint32_t nk = p.K / GEMM_BK;

    // X: thread -> (row tid/8 of each pass, 16-byte column tid%8)
    const uint8_t* xsrc[XP];
#pragma unroll
    for (int i = 0; i < XP; ++i) {
        const uint32_t m = min(m0 + i * XROWS + (tid >> 3), p.M - 1u);
        xsrc[i] = (const uint8_t*)p.X + (size_t)m * p.K * 2u + (tid & 7u) * 16u;
    }
    // W: item it -> row (tid + NT*it)/2, run (tid + NT*it)%2
    const uint8_t* wsrc[WI];
    uint32_t wrow[WI], whf[WI];
#pragma unroll
    for (int i = 0; i < WI; ++i) {
        const uint32_t item = tid + NT * i;
        wrow[i] = item >> 1;
        whf[i] = item & 1u;
        wsrc[i] = p.W + (size_t)min(n0 + wrow[i], p.N - 1u) * p.row_stride_bytes;
    }

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    u32x4 xr[XP];
    uint32_t w4[TYPE == KQ_TYPE_Q4_K ? WI : 1][12];
    uint32_t w5[TYPE == KQ_TYPE_Q5_K ? WI : 1][20];
    Q6Raw w6[TYPE == KQ_TYPE_Q6_K ? WI : 1];

    auto load_tile = [&](uint32_t kt) {
#pragma unroll
        for (int i = 0; i < XP; ++i) xr[i] = *(const u32x4*)(xsrc[i] + (size_t)kt * (GEMM_BK * 2));
#pragma unroll
        for (int i = 0; i < WI; ++i) {
            if constexpr (TYPE == KQ_TYPE_Q4_K) q4k_load(wsrc[i], kt, w4[i]);
            else if constexpr (TYPE == KQ_TYPE_Q5_K) q5k_load(wsrc[i], kt, w5[i]);
            else q6k_load(wsrc[i], kt, whf[i], w6[i]);
        }
    };
    auto store_tile = [&](uint32_t kt, uint32_t buf) {
        uint8_t* a = As + buf * A_BYTES;
        uint8_t* b = Bs + buf * B_BYTES;
#pragma unroll
        for (int i = 0; i < XP; ++i)
            *(u32x4*)(a + (i * XROWS + (tid >> 3)) * GEMM_LD + (tid & 7u) * 16u) = xr[i];
#pragma unroll
        for (int i = 0; i < WI; ++i) {
            uint8_t* dst = b + wrow[i] * GEMM_LD + whf[i] * 64u;
            if constexpr (TYPE == KQ_TYPE_Q4_K) q4k_expand(w4[i], kt, whf[i], dst);
            else if constexpr (TYPE == KQ_TYPE_Q5_K) q5k_expand(w5[i], kt, whf[i], dst);
            else q6k_expand(w6[i], kt, whf[i], dst);
        }
    };
    auto multiply = [&](uint32_t buf) {
        const uint8_t* a = As + buf * A_BYTES + (wm * WM + (lane & 31u)) * GEMM_LD + (lane >> 5) * 16u;
        const uint8_t* b = Bs + buf * B_BYTES + (wn * WN + (lane & 31u)) * GEMM_LD + (lane >> 5) * 16u;
#pragma unroll
        for (int s = 0; s < GEMM_BK / 16; ++s) {
            bf16x8 af[TM], bfr[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) af[i] = *(const bf16x8*)(a + i * 32 * GEMM_LD + s * 32);
#pragma unroll
            for (int j = 0; j < TN; ++j) bfr[j] = *(const bf16x8*)(b + j * 32 * GEMM_LD + s * 32);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
        }
    };

    load_tile(0);
    store_tile(0, 0);
    __syncthreads();

    for (uint32_t kt = 0; kt < nk; ++kt) {
        const uint32_t buf = kt & 1u;
        if (kt + 1 < nk) load_tile(kt + 1);
        multiply(buf);
        if (kt + 1 < nk) store_tile(kt + 1, buf ^ 1u);
        __syncthreads();
    }

    store_acc<TM, TN>(p, acc, m0 + wm * WM, n0 + wn * WN, lane);
}

// ---------------------------------------------------------------------------------------------------------
// Persistent 256 x 256 x 64 kernel.  A thread owns one (weight row, run of 32 k) item of the W tile and four
// 16-byte pieces of the X tile per step; their raw bytes live in registers one step ahead of their use.
struct RawQ4 { u32x4 h, q0, q1; };
struct RawQ6 { u32x4 a0, a1, b0, b1; uint32_t sc2, d16; };
struct RawQ5 { u32x4 h, q0, q1, b0, b1; };   // header, the run's 32 quant bytes, the block's 32 bytes of fifth bits

__device__ __forceinline__ void il_load_head(const uint8_t* row, uint32_t kc, uint32_t, RawQ4& r, bool new_block = true)
{
    if (new_block) r.h = *(const u32x4*)(row + (size_t)(kc >> 2) * KQ_Q4K_BYTES);
}
__device__ __forceinline__ void il_load_q(const uint8_t* row, uint32_t kc, uint32_t, int half, RawQ4& r, bool = true)
{
    const u32x4* q = (const u32x4*)(row + (size_t)(kc >> 2) * KQ_Q4K_BYTES + 16 + (kc & 3u) * 32u);
    if (half == 0) r.q0 = q[0]; else r.q1 = q[1];
}
// Scale and minimum of sub-block 2 * c + hf of a Q4_K / Q5_K header, c = the k step's place in its superblock.  The
// k loop knows c at compile time (cpos >= 0): the choice between the two 6-bit layouts is then no branch, which
// q4k_scale_min's is (it cut every k step of the loop into three basic blocks).
__device__ __forceinline__ void il_scale_min(uint32_t u0, uint32_t u1, uint32_t u2, uint32_t kc, uint32_t hf, int cpos,
                                             uint32_t& sc, uint32_t& mn)
{
    if (cpos < 0) {
        q4k_scale_min(u0, u1, u2, (int)((kc & 3u) * 2u + hf), sc, mn);
        return;
    }
    const uint32_t sh = 8u * ((2u * (uint32_t)cpos + hf) & 3u);
    const uint32_t a = (u0 >> sh) & 255u, b = (u1 >> sh) & 255u;
    if (cpos < 2) {
        sc = a & 63u;
        mn = b & 63u;
    } else {
        const uint32_t c = (u2 >> sh) & 255u;
        sc = (c & 15u) | ((a >> 6) << 4);
        mn = (c >> 4) | ((b >> 6) << 4);
    }
}
__device__ __forceinline__ void il_scales(const RawQ4& r, uint32_t kc, uint32_t hf, float& s0, float& s1, float& nb, int cpos = -1)
{
    const float d = half_bits_to_float(r.h.x & 0xFFFFu);
    const float dmin = half_bits_to_float(r.h.x >> 16);
    uint32_t sc, mn;
    il_scale_min(r.h.y, r.h.z, r.h.w, kc, hf, cpos, sc, mn);
    // a masked nibble is left where it is and read as an fp16 subnormal, q * 2^-24 (low nibble) or q * 2^-20 (high
    // nibble): the scale carries the matching power of two (an exact scaling, so fma(q_h, s0, nb) rounds the same
    // exact value as fma(d * sc, q, nb) does)
    s0 = d * (float)sc * (hf ? 1048576.0f : 16777216.0f);
    s1 = s0;
    nb = -(dmin * (float)mn);
}
typedef _Float16 gm_half2 __attribute__((ext_vector_type(2)));
// 8 weights (piece v of the thread's run of 32) -> 16 bytes of bf16.  No integer-to-float conversion: the nibbles
// enter v_fma_mix_f32 as fp16 subnormals (two masks and a shift per four weights instead of a mask and four
// conversions).
__device__ __forceinline__ u32x4 il_expand(const RawQ4& r, uint32_t, uint32_t hf, int v, float s0, float, float nb)
{
    const u32x4 src = v < 2 ? r.q0 : r.q1;
    const uint32_t mask = hf ? 0x00F000F0u : 0x000F000Fu;
    u32x4 out;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const uint32_t w = src[(v & 1) * 2 + j];
        const gm_half2 a = __builtin_bit_cast(gm_half2, w & mask);          // bytes 0 and 2
        const gm_half2 b = __builtin_bit_cast(gm_half2, (w >> 8) & mask);   // bytes 1 and 3
        const _Float16 a0 = a.x, a1 = a.y, b0 = b.x, b1 = b.y;
        const float f0 = fmaf((float)a0, s0, nb);
        const float f1 = fmaf((float)b0, s0, nb);
        const float f2 = fmaf((float)a1, s0, nb);
        const float f3 = fmaf((float)b1, s0, nb);
        out[j * 2] = pack_bf16(f0, f1);
        out[j * 2 + 1] = pack_bf16(f2, f3);
    }
    return out;
}

// new_block = false: the step lies in the same superblock as the one before it (d is already there)
// Q5_K: the Q4_K walk with the quants 32 bytes further on; the fifth bits of a run's 32 elements are bit
// 2c + hf of the block's 32 bytes of qh (the same bytes for the four k steps c of a superblock: extra = false
// leaves them in their registers).  Both nibbles come down to bits 0..3 so that the fifth bit joins at bit 4.
__device__ __forceinline__ void il_load_head(const uint8_t* row, uint32_t kc, uint32_t, RawQ5& r, bool new_block = true)
{
    if (new_block) r.h = *(const u32x4*)(row + (size_t)(kc >> 2) * KQ_Q5K_BYTES);
}
__device__ __forceinline__ void il_load_q(const uint8_t* row, uint32_t kc, uint32_t, int half, RawQ5& r, bool extra = true)
{
    const uint8_t* blk = row + (size_t)(kc >> 2) * KQ_Q5K_BYTES;
    const u32x4* q = (const u32x4*)(blk + 48 + (kc & 3u) * 32u);
    const u32x4* b = (const u32x4*)(blk + 16);
    if (half == 0) { r.q0 = q[0]; if (extra) r.b0 = b[0]; }
    else { r.q1 = q[1]; if (extra) r.b1 = b[1]; }
}
__device__ __forceinline__ void il_scales(const RawQ5& r, uint32_t kc, uint32_t hf, float& s0, float& s1, float& nb, int cpos = -1)
{
    const float d = half_bits_to_float(r.h.x & 0xFFFFu);
    const float dmin = half_bits_to_float(r.h.x >> 16);
    uint32_t sc, mn;
    il_scale_min(r.h.y, r.h.z, r.h.w, kc, hf, cpos, sc, mn);
    s0 = d * (float)sc;
    s1 = s0;
    nb = -(dmin * (float)mn);
}
__device__ __forceinline__ u32x4 il_expand(const RawQ5& r, uint32_t kc, uint32_t hf, int v, float s0, float, float nb)
{
    const u32x4 src = v < 2 ? r.q0 : r.q1, bits = v < 2 ? r.b0 : r.b1;
    const uint32_t sh = hf * 4u, sb = (kc & 3u) * 2u + hf;
    u32x4 out;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const uint32_t w = ((src[(v & 1) * 2 + j] >> sh) & 0x0F0F0F0Fu) | (((bits[(v & 1) * 2 + j] >> sb) & 0x01010101u) << 4);
        const float f0 = fmaf(s0, (float)(w & 255u), nb);
        const float f1 = fmaf(s0, (float)((w >> 8) & 255u), nb);
        const float f2 = fmaf(s0, (float)((w >> 16) & 255u), nb);
        const float f3 = fmaf(s0, (float)(w >> 24), nb);
        out[j * 2] = pack_bf16(f0, f1);
        out[j * 2 + 1] = pack_bf16(f2, f3);
    }
    return out;
}

__device__ __forceinline__ void il_load_head(const uint8_t* row, uint32_t kc, uint32_t hf, RawQ6& r, bool new_block = true)
{
    const uint32_t c = kc & 3u, h = c >> 1, t = (c & 1u) * 2u + hf;
    const uint8_t* blk = row + (size_t)(kc >> 2) * KQ_Q6K_BYTES;
    uint16_t s2, d2;
    __builtin_memcpy(&s2, blk + 192u + 8u * h + 2u * t, 2);
    r.sc2 = s2;
    if (new_block) {
        __builtin_memcpy(&d2, blk + 208u, 2);
        r.d16 = d2;
    }
}
__device__ __forceinline__ void il_load_q(const uint8_t* row, uint32_t kc, uint32_t hf, int half, RawQ6& r, bool = true)
{
    const uint32_t c = kc & 3u, h = c >> 1, t = (c & 1u) * 2u + hf;
    const uint8_t* blk = row + (size_t)(kc >> 2) * KQ_Q6K_BYTES;
    // blocks are 2-byte aligned; the hardware takes unaligned 128-bit loads as they are
    if (half == 0) {
        __builtin_memcpy(&r.a0, blk + 64u * h + 32u * (t & 1u), 16);
        __builtin_memcpy(&r.b0, blk + 128u + 32u * h, 16);
    } else {
        __builtin_memcpy(&r.a1, blk + 64u * h + 32u * (t & 1u) + 16u, 16);
        __builtin_memcpy(&r.b1, blk + 128u + 32u * h + 16u, 16);
    }
}
__device__ __forceinline__ void il_scales(const RawQ6& r, uint32_t, uint32_t, float& s0, float& s1, float& nb, int = -1)
{
    const float d = half_bits_to_float(r.d16);
    s0 = d * (float)(int)(int8_t)(r.sc2 & 255u);
    s1 = d * (float)(int)(int8_t)(r.sc2 >> 8);
    nb = 0.0f;
}
__device__ __forceinline__ u32x4 il_expand(const RawQ6& r, uint32_t kc, uint32_t hf, int v, float s0, float s1, float)
{
    const uint32_t t = ((kc & 3u) & 1u) * 2u + hf;
    const uint32_t lsh = (t & 2u) ? 4u : 0u;
    const float s = v < 2 ? s0 : s1;
    const float off = -32.0f * s;
    const u32x4 ql = v < 2 ? r.a0 : r.a1, qh = v < 2 ? r.b0 : r.b1;
    u32x4 out;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const uint32_t lo = (ql[(v & 1) * 2 + j] >> lsh) & 0x0F0F0F0Fu;
        const uint32_t hi = ((qh[(v & 1) * 2 + j] >> (2u * t)) & 0x03030303u) << 4;
        const uint32_t q = lo | hi;   // four 6-bit stored values
        const float f0 = fmaf(s, (float)(q & 255u), off);
        const float f1 = fmaf(s, (float)((q >> 8) & 255u), off);
        const float f2 = fmaf(s, (float)((q >> 16) & 255u), off);
        const float f3 = fmaf(s, (float)(q >> 24), off);
        out[j * 2] = pack_bf16(f0, f1);
        out[j * 2 + 1] = pack_bf16(f2, f3);
    }
    return out;
}

template <int TYPE>
__global__ __launch_bounds__(512) void gemm_bf16_sk_kernel(GemmParams p)
{
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr int BM = 256, BN = 256, WAVES_N = 4, WM = 128, WN = 64, TM = 4, TN = 2;
    constexpr int A_BYTES = BM * GEMM_LD, B_BYTES = BN * GEMM_LD;
    constexpr int XROWS = 64;   // X rows per piece: 8 threads x 16 bytes per row, 4 pieces
    using Raw = typename std::conditional<TYPE == KQ_TYPE_Q4_K, RawQ4,
                                          typename std::conditional<TYPE == KQ_TYPE_Q5_K, RawQ5, RawQ6>::type>::type;
    uint8_t* As = smem;
    uint8_t* Bs = smem + 2 * A_BYTES;

    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t wm = wave / WAVES_N, wn = wave % WAVES_N;
    const uint32_t nk_all = p.K / GEMM_BK;
    const uint32_t x_dst = (tid >> 3) * GEMM_LD + (tid & 7u) * 16u;
    const uint32_t wrow = tid >> 1, whf = tid & 1u;
    const uint32_t w_dst = wrow * GEMM_LD + whf * 64u;
    const uint32_t a_src = (wm * WM + (lane & 31u)) * GEMM_LD + (lane >> 5) * 16u;
    const uint32_t b_src = (wn * WN + (lane & 31u)) * GEMM_LD + (lane >> 5) * 16u;

    // this workgroup's share of the walk: units [u, u_end), a unit = one k step of one tile
    uint32_t u = blockIdx.x * p.units_per_wg;
    const uint32_t u_end = min(u + p.units_per_wg, p.units);
    while (u < u_end) {
    const uint32_t tile = u / nk_all, k_first = u - tile * nk_all;
    const uint32_t nk = min(nk_all - k_first, u_end - u);   // k steps of this segment
    u += nk;
        const uint32_t m0 = (tile / p.tiles_n) * BM, n0 = (tile % p.tiles_n) * BN;

    const uint8_t* xsrc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t m = min(m0 + i * XROWS + (tid >> 3), p.M - 1u);
        xsrc[i] = (const uint8_t*)p.X + (size_t)m * p.K * 2u + (tid & 7u) * 16u;
    }
    const uint8_t* wsrc = p.W + (size_t)min(n0 + wrow, p.N - 1u) * p.row_stride_bytes;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    // Raw registers: piece v of xr / w holds tile T(v) of the k walk.  Piece 0 runs one tile ahead of
    // pieces 1..3 (it is converted in the slice after the barrier, the others in the three slices before).
    u32x4 xr[4];
    Raw w;
    float s0, s1, nb;   // scales of the tile being converted
    auto tile_at = [&](uint32_t t) { return k_first + min(t, nk - 1u); };   // k step t of the segment, clamped
    auto load_x = [&](uint32_t t, int i) { xr[i] = *(const u32x4*)(xsrc[i] + (size_t)tile_at(t) * (GEMM_BK * 2)); };
    auto read_ops = [&](uint32_t buf, int s, bf16x8 (&af)[TM], bf16x8 (&bfr)[TN]) {
        const uint8_t* a = As + buf * A_BYTES + a_src + s * 32;
        const uint8_t* b = Bs + buf * B_BYTES + b_src + s * 32;
#pragma unroll
        for (int i = 0; i < TM; ++i) af[i] = *(const bf16x8*)(a + i * 32 * GEMM_LD);
#pragma unroll
        for (int j = 0; j < TN; ++j) bfr[j] = *(const bf16x8*)(b + j * 32 * GEMM_LD);
    };
    auto mfma_ops = [&](const bf16x8 (&af)[TM], const bf16x8 (&bfr)[TN]) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
    };
    // piece v of tile t: X copy and 8 dequantised weights into LDS buffer t&1, then the registers of the
    // piece are refilled from tile t+1 (a full step before they are converted)
    // refill = false: tile t+1 is made of the same quant bytes as tile t (see the k loop), nothing to fetch;
    // extra = false: tile t+1 lies in the superblock of tile t (Q5_K keeps its fifth bits)
    auto convert_piece = [&](uint32_t t, int v, bool refill = true, bool extra = true) {
        const uint32_t buf = t & 1u;
        *(u32x4*)(As + buf * A_BYTES + x_dst + v * XROWS * GEMM_LD) = xr[v];
        *(u32x4*)(Bs + buf * B_BYTES + w_dst + v * 16) = il_expand(w, tile_at(t), whf, v, s0, s1, nb);
        load_x(t + 1u, v);
        if (v == 1 && refill) il_load_q(wsrc, tile_at(t + 1u), whf, 0, w, extra);
        if (v == 3 && refill) il_load_q(wsrc, tile_at(t + 1u), whf, 1, w, extra);
    };
    // the matrix instructions of a slice take turns with the conversion arithmetic; LDS reads go first
    auto slice_schedule = [&]() {
        __builtin_amdgcn_sched_group_barrier(0x100, TM + TN, 0);
#pragma unroll
        for (int g = 0; g < TM * TN; ++g) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 5, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
    };

    // prologue: tile 0 whole and piece 0 of tile 1 into LDS; registers end up holding pieces 1..3 of tile 1,
    // piece 0 of tile 2 and the scales of tile 1
#pragma unroll
    for (int i = 0; i < 4; ++i) load_x(0, i);
    il_load_head(wsrc, tile_at(0), whf, w);
    il_load_q(wsrc, tile_at(0), whf, 0, w);
    il_load_q(wsrc, tile_at(0), whf, 1, w);
    il_scales(w, tile_at(0), whf, s0, s1, nb, 0);
    il_load_head(wsrc, tile_at(1), whf, w);
#pragma unroll
    for (int v = 0; v < 4; ++v) convert_piece(0, v);
    il_scales(w, tile_at(1), whf, s0, s1, nb, 1);
    il_load_head(wsrc, tile_at(2), whf, w);
    convert_piece(1, 0);
    __syncthreads();

    bf16x8 af[2][TM], bfr[2][TN];
    read_ops(0, 0, af[0], bfr[0]);
    // one k step; refill = whether the quant registers freed by tile kt+1 are loaded with tile kt+2,
    // new_block = whether tile kt+3 opens a superblock (else its header is the one already in registers)
    // (opens = whether tile kt+2 opens a superblock; pos2 = the place of tile kt+2 in its superblock: runs start on
    // a superblock, and the tiles past a run's end, clamped to its last, are never multiplied)
    auto k_step = [&](uint32_t kt, bool refill, bool new_block, bool opens, int pos2) {
        const uint32_t buf = kt & 1u;
        // slices 0..2 of tile kt; pieces 1..3 of tile kt+1 go to the other buffer
#pragma unroll
        for (int s = 0; s < 3; ++s) {
            read_ops(buf, s + 1, af[(s + 1) & 1], bfr[(s + 1) & 1]);
            mfma_ops(af[s & 1], bfr[s & 1]);
            convert_piece(kt + 1u, s + 1, refill, opens);
            slice_schedule();
        }
        // every wave has now read all of tile kt and written its part of tile kt+1
        __syncthreads();
        // slice 3 of tile kt needs no LDS: its operands are in registers.  Behind it the first operands of
        // tile kt+1 are fetched and piece 0 of tile kt+2 replaces tile kt in LDS.
        read_ops(buf ^ 1u, 0, af[0], bfr[0]);
        mfma_ops(af[1], bfr[1]);
        il_scales(w, tile_at(kt + 2u), whf, s0, s1, nb, pos2);
        il_load_head(wsrc, tile_at(kt + 3u), whf, w, new_block);
        convert_piece(kt + 2u, 0);
        slice_schedule();
    };
    // Runs start on a superblock (k step 4j) and cover whole superblocks (the launcher sees to it), so the four
    // steps of a superblock are told apart at compile time.  The header of tile kt+3 has to be fetched when
    // kt+3 is a multiple of 4 (the tile beyond the run is the clamped last one: same superblock, no fetch is
    // lost).  Q6_K: k steps 2j and 2j+1 of a row take the low and the high nibbles of the same 32 bytes of ql
    // and different bit pairs of the same 32 bytes of qh, so the registers loaded for an even tile serve the
    // odd tile after it.
    constexpr bool Q6 = TYPE == KQ_TYPE_Q6_K;
    for (uint32_t kt = 0; kt < nk; kt += 4u) {
        k_step(kt, true, false, false, 2);
        k_step(kt + 1u, !Q6, true, false, 3);
        k_step(kt + 2u, true, false, true, 0);
        k_step(kt + 3u, !Q6, false, false, 1);
    }

    // A tile walked in one piece is stored.  A run over part of a tile leaves its sums in the workspace, in
    // register order (a wave writes 1 KB per instruction): slot 2b of workgroup b if the run starts the
    // workgroup's share, slot 2b+1 if it ends it.  gemm_sum_cut_tiles_kernel adds the runs of each cut tile
    // in the order of the walk afterwards, so the result does not depend on timing.
    if (nk == nk_all) {
        store_acc<TM, TN>(p, acc, m0 + wm * WM, n0 + wn * WN, lane);
    } else {
        const uint32_t slot = 2u * blockIdx.x + (blockIdx.x * p.units_per_wg < tile * nk_all ? 1u : 0u);
        f32x4* dst = (f32x4*)(p.partial + (size_t)slot * 65536u) + wave * 2048u + lane;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    dst[((i * TN + j) * 4 + r) * 64] =
                        f32x4{acc[i][j][4 * r], acc[i][j][4 * r + 1], acc[i][j][4 * r + 2], acc[i][j][4 * r + 3]};
    }
    __syncthreads();   // the next segment's prologue overwrites LDS
    }
}

// The thread's 16 quant bytes of a k step when four threads share a weight row (quarter = 2 * hf + wq: the
// sub-block pair's half hf, the first or second 16 of its 32 bytes): they go where the loaders above put the
// FIRST 16 bytes, so that il_expand serves pieces 0 and 1 of them.
__device__ __forceinline__ void il1_load_q(const uint8_t* row, uint32_t kc, uint32_t, uint32_t wq, RawQ4& r, bool = true)
{
    const u32x4* q = (const u32x4*)(row + (size_t)(kc >> 2) * KQ_Q4K_BYTES + 16 + (kc & 3u) * 32u);
    r.q0 = q[wq];
}
__device__ __forceinline__ void il1_load_q(const uint8_t* row, uint32_t kc, uint32_t, uint32_t wq, RawQ5& r, bool extra = true)
{
    const uint8_t* blk = row + (size_t)(kc >> 2) * KQ_Q5K_BYTES;
    r.q0 = ((const u32x4*)(blk + 48 + (kc & 3u) * 32u))[wq];
    if (extra) r.b0 = ((const u32x4*)(blk + 16))[wq];
}
__device__ __forceinline__ void il1_load_q(const uint8_t* row, uint32_t kc, uint32_t hf, uint32_t wq, RawQ6& r, bool = true)
{
    const uint32_t c = kc & 3u, h = c >> 1, t = (c & 1u) * 2u + hf;
    const uint8_t* blk = row + (size_t)(kc >> 2) * KQ_Q6K_BYTES;
    __builtin_memcpy(&r.a0, blk + 64u * h + 32u * (t & 1u) + 16u * wq, 16);
    __builtin_memcpy(&r.b0, blk + 128u + 32u * h + 16u * wq, 16);
}

// 256 tokens x 128 weight rows per workgroup, whole tiles, one per workgroup: for matrices of few rows at many
// tokens (N = 4096 at M = 2048 is 256 such tiles, one per CU over the full K, where 256 x 256 tiles fill half the
// CUs or need their K cut in two and a second kernel to add the halves).  Eight waves as 4 x 2, 64 x 64 each; four
// threads share a weight row of a k step (16 weights each), the X tile and the schedule are those of the kernel
// above.
template <int TYPE>
__global__ __launch_bounds__(512) void gemm_bf16_n128_kernel(GemmParams p)
{
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr int BM = 256, BN = 128, WAVES_N = 2, WM = 64, WN = 64, TM = 2, TN = 2;
    constexpr int A_BYTES = BM * GEMM_LD, B_BYTES = BN * GEMM_LD;
    constexpr int XROWS = 64;
    using Raw = typename std::conditional<TYPE == KQ_TYPE_Q4_K, RawQ4,
                                          typename std::conditional<TYPE == KQ_TYPE_Q5_K, RawQ5, RawQ6>::type>::type;
    constexpr bool Q6 = TYPE == KQ_TYPE_Q6_K;
    uint8_t* As = smem;
    uint8_t* Bs = smem + 2 * A_BYTES;

    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t wm = wave / WAVES_N, wn = wave % WAVES_N;
    const uint32_t nk = p.K / GEMM_BK;
    const uint32_t x_dst = (tid >> 3) * GEMM_LD + (tid & 7u) * 16u;
    const uint32_t wrow = tid >> 2, whf = (tid >> 1) & 1u, wq = tid & 1u;
    const uint32_t w_dst = wrow * GEMM_LD + (tid & 3u) * 32u;
    const uint32_t a_src = (wm * WM + (lane & 31u)) * GEMM_LD + (lane >> 5) * 16u;
    const uint32_t b_src = (wn * WN + (lane & 31u)) * GEMM_LD + (lane >> 5) * 16u;
    const uint32_t tile = blockIdx.x;
    const uint32_t m0 = (tile / p.tiles_n) * BM, n0 = (tile % p.tiles_n) * BN;

    const uint8_t* xsrc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t m = min(m0 + i * XROWS + (tid >> 3), p.M - 1u);
        xsrc[i] = (const uint8_t*)p.X + (size_t)m * p.K * 2u + (tid & 7u) * 16u;
    }
    const uint8_t* wsrc = p.W + (size_t)min(n0 + wrow, p.N - 1u) * p.row_stride_bytes;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    u32x4 xr[4];
    Raw w;
    float s0, s1, nb;
    auto tile_at = [&](uint32_t t) { return min(t, nk - 1u); };
    auto load_x = [&](uint32_t t, int i) { xr[i] = *(const u32x4*)(xsrc[i] + (size_t)tile_at(t) * (GEMM_BK * 2)); };
    auto scales = [&](uint32_t t, int pos) {
        il_scales(w, tile_at(t), whf, s0, s1, nb, pos);
        if (Q6 && wq) s0 = s1;   // Q6_K: the second 16 of a run of 32 have a scale of their own
    };
    auto read_ops = [&](uint32_t buf, int s, bf16x8 (&af)[TM], bf16x8 (&bfr)[TN]) {
        const uint8_t* a = As + buf * A_BYTES + a_src + s * 32;
        const uint8_t* b = Bs + buf * B_BYTES + b_src + s * 32;
#pragma unroll
        for (int i = 0; i < TM; ++i) af[i] = *(const bf16x8*)(a + i * 32 * GEMM_LD);
#pragma unroll
        for (int j = 0; j < TN; ++j) bfr[j] = *(const bf16x8*)(b + j * 32 * GEMM_LD);
    };
    auto mfma_ops = [&](const bf16x8 (&af)[TM], const bf16x8 (&bfr)[TN]) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
    };
    // piece v of tile t: the X copy, and for v < 2 eight of the thread's sixteen weights, into LDS buffer t&1; the
    // piece's registers are then refilled from tile t+1
    auto convert_piece = [&](uint32_t t, int v, bool refill = true, bool extra = true) {
        const uint32_t buf = t & 1u;
        *(u32x4*)(As + buf * A_BYTES + x_dst + v * XROWS * GEMM_LD) = xr[v];
        if (v < 2) *(u32x4*)(Bs + buf * B_BYTES + w_dst + v * 16) = il_expand(w, tile_at(t), whf, v, s0, s1, nb);
        load_x(t + 1u, v);
        if (v == 1 && refill) il1_load_q(wsrc, tile_at(t + 1u), whf, wq, w, extra);
    };
    auto slice_schedule = [&]() {
        __builtin_amdgcn_sched_group_barrier(0x100, TM + TN, 0);
#pragma unroll
        for (int g = 0; g < TM * TN; ++g) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
    };

#pragma unroll
    for (int i = 0; i < 4; ++i) load_x(0, i);
    il_load_head(wsrc, tile_at(0), whf, w);
    il1_load_q(wsrc, tile_at(0), whf, wq, w);
    scales(0, 0);
    il_load_head(wsrc, tile_at(1), whf, w);
#pragma unroll
    for (int v = 0; v < 4; ++v) convert_piece(0, v);
    scales(1, 1);
    il_load_head(wsrc, tile_at(2), whf, w);
    convert_piece(1, 0);
    __syncthreads();

    bf16x8 af[2][TM], bfr[2][TN];
    read_ops(0, 0, af[0], bfr[0]);
    auto k_step = [&](uint32_t kt, bool refill, bool new_block, bool opens, int pos2) {
        const uint32_t buf = kt & 1u;
#pragma unroll
        for (int s = 0; s < 3; ++s) {
            read_ops(buf, s + 1, af[(s + 1) & 1], bfr[(s + 1) & 1]);
            mfma_ops(af[s & 1], bfr[s & 1]);
            convert_piece(kt + 1u, s + 1, refill, opens);
            slice_schedule();
        }
        __syncthreads();
        read_ops(buf ^ 1u, 0, af[0], bfr[0]);
        mfma_ops(af[1], bfr[1]);
        scales(kt + 2u, pos2);
        il_load_head(wsrc, tile_at(kt + 3u), whf, w, new_block);
        convert_piece(kt + 2u, 0);
        slice_schedule();
    };
    for (uint32_t kt = 0; kt < nk; kt += 4u) {
        k_step(kt, true, false, false, 2);
        k_step(kt + 1u, !Q6, true, false, 3);
        k_step(kt + 2u, true, false, true, 0);
        k_step(kt + 3u, !Q6, false, false, 1);
    }
    store_acc<TM, TN>(p, acc, m0 + wm * WM, n0 + wn * WN, lane);
}

// 256 tokens x 192 weight rows per workgroup, whole tiles: N = 6144 at M = 2048 is 256 such tiles, one per CU, where
// 256 x 256 tiles leave a quarter of the CUs without one.  The kernel above with waves of 64 x 96 and two items
// per thread: a quarter row of rows 0..127 (as above) and one of rows 128..191 — those 64 rows are taken twice,
// by threads t and t + 256, which store the same bytes: no wave has a path of its own, so the k loop stays one
// basic block.  Item A's two pieces are expanded in the slice behind the barrier and the first slice of the next
// step, item B's in the two slices after that: the places of pieces 0..3 in the 256-tile kernel.
template <int TYPE>
__global__ __launch_bounds__(512) void gemm_bf16_n192_kernel(GemmParams p)
{
    extern __shared__ __align__(16) uint8_t smem[];
    constexpr int BM = 256, BN = 192, WAVES_N = 2, WM = 64, WN = 96, TM = 2, TN = 3;
    constexpr int A_BYTES = BM * GEMM_LD, B_BYTES = BN * GEMM_LD;
    constexpr int XROWS = 64;
    using Raw = typename std::conditional<TYPE == KQ_TYPE_Q4_K, RawQ4,
                                          typename std::conditional<TYPE == KQ_TYPE_Q5_K, RawQ5, RawQ6>::type>::type;
    constexpr bool Q6 = TYPE == KQ_TYPE_Q6_K;
    uint8_t* As = smem;
    uint8_t* Bs = smem + 2 * A_BYTES;

    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t wm = wave / WAVES_N, wn = wave % WAVES_N;
    const uint32_t nk = p.K / GEMM_BK;
    const uint32_t x_dst = (tid >> 3) * GEMM_LD + (tid & 7u) * 16u;
    const uint32_t wrow = tid >> 2, whf = (tid >> 1) & 1u, wq = tid & 1u;
    const uint32_t wrow_b = 128u + ((tid >> 2) & 63u);
    const uint32_t w_dst = wrow * GEMM_LD + (tid & 3u) * 32u;
    const uint32_t w_dst_b = wrow_b * GEMM_LD + (tid & 3u) * 32u;
    const uint32_t a_src = (wm * WM + (lane & 31u)) * GEMM_LD + (lane >> 5) * 16u;
    const uint32_t b_src = (wn * WN + (lane & 31u)) * GEMM_LD + (lane >> 5) * 16u;
    const uint32_t tile = blockIdx.x;
    const uint32_t m0 = (tile / p.tiles_n) * BM, n0 = (tile % p.tiles_n) * BN;

    const uint8_t* xsrc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t m = min(m0 + i * XROWS + (tid >> 3), p.M - 1u);
        xsrc[i] = (const uint8_t*)p.X + (size_t)m * p.K * 2u + (tid & 7u) * 16u;
    }
    const uint8_t* wsrc = p.W + (size_t)min(n0 + wrow, p.N - 1u) * p.row_stride_bytes;
    const uint8_t* wsrc_b = p.W + (size_t)min(n0 + wrow_b, p.N - 1u) * p.row_stride_bytes;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    u32x4 xr[4];
    Raw w, wb;
    float s0, s1, nb, s0b, s1b, nbb;
    auto tile_at = [&](uint32_t t) { return min(t, nk - 1u); };
    auto load_x = [&](uint32_t t, int i) { xr[i] = *(const u32x4*)(xsrc[i] + (size_t)tile_at(t) * (GEMM_BK * 2)); };
    auto scales_a = [&](uint32_t t, int pos) {
        il_scales(w, tile_at(t), whf, s0, s1, nb, pos);
        if (Q6 && wq) s0 = s1;   // Q6_K: the second 16 of a run of 32 have a scale of their own
    };
    auto scales_b = [&](uint32_t t, int pos) {
        il_scales(wb, tile_at(t), whf, s0b, s1b, nbb, pos);
        if (Q6 && wq) s0b = s1b;
    };
    auto read_ops = [&](uint32_t buf, int s, bf16x8 (&af)[TM], bf16x8 (&bfr)[TN]) {
        const uint8_t* a = As + buf * A_BYTES + a_src + s * 32;
        const uint8_t* b = Bs + buf * B_BYTES + b_src + s * 32;
#pragma unroll
        for (int i = 0; i < TM; ++i) af[i] = *(const bf16x8*)(a + i * 32 * GEMM_LD);
#pragma unroll
        for (int j = 0; j < TN; ++j) bfr[j] = *(const bf16x8*)(b + j * 32 * GEMM_LD);
    };
    auto mfma_ops = [&](const bf16x8 (&af)[TM], const bf16x8 (&bfr)[TN]) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
    };
    // piece v of tile t: the X copy and eight weights (v < 2 of item A, else of item B) into LDS buffer t&1; an
    // item's registers are refilled from tile t+1 behind its second piece
    auto convert_piece = [&](uint32_t t, int v, bool refill = true, bool extra = true) {
        const uint32_t buf = t & 1u;
        *(u32x4*)(As + buf * A_BYTES + x_dst + v * XROWS * GEMM_LD) = xr[v];
        if (v < 2) *(u32x4*)(Bs + buf * B_BYTES + w_dst + v * 16) = il_expand(w, tile_at(t), whf, v, s0, s1, nb);
        else *(u32x4*)(Bs + buf * B_BYTES + w_dst_b + (v - 2) * 16) = il_expand(wb, tile_at(t), whf, v - 2, s0b, s1b, nbb);
        load_x(t + 1u, v);
        if (v == 1 && refill) il1_load_q(wsrc, tile_at(t + 1u), whf, wq, w, extra);
        if (v == 3 && refill) il1_load_q(wsrc_b, tile_at(t + 1u), whf, wq, wb, extra);
    };
    auto slice_schedule = [&]() {
        __builtin_amdgcn_sched_group_barrier(0x100, TM + TN, 0);
#pragma unroll
        for (int g = 0; g < TM * TN; ++g) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 5, 0);   // (4 .. 8 per group measured level)
        }
        __builtin_amdgcn_sched_barrier(0);
    };

#pragma unroll
    for (int i = 0; i < 4; ++i) load_x(0, i);
    il_load_head(wsrc, tile_at(0), whf, w);
    il_load_head(wsrc_b, tile_at(0), whf, wb);
    il1_load_q(wsrc, tile_at(0), whf, wq, w);
    il1_load_q(wsrc_b, tile_at(0), whf, wq, wb);
    scales_a(0, 0);
    scales_b(0, 0);
    il_load_head(wsrc, tile_at(1), whf, w);
    il_load_head(wsrc_b, tile_at(1), whf, wb);
#pragma unroll
    for (int v = 0; v < 4; ++v) convert_piece(0, v);
    scales_a(1, 1);
    il_load_head(wsrc, tile_at(2), whf, w);
    convert_piece(1, 0);
    __syncthreads();

    bf16x8 af[2][TM], bfr[2][TN];
    read_ops(0, 0, af[0], bfr[0]);
    auto k_step = [&](uint32_t kt, bool refill, bool new_block, bool opens, int pos2) {
        const uint32_t buf = kt & 1u;
#pragma unroll
        for (int s = 0; s < 3; ++s) {
            read_ops(buf, s + 1, af[(s + 1) & 1], bfr[(s + 1) & 1]);
            mfma_ops(af[s & 1], bfr[s & 1]);
            if (s == 0) {   // item B runs a slice behind item A: its scales of tile kt+1, then the header of kt+2
                scales_b(kt + 1u, (pos2 + 3) & 3);
                il_load_head(wsrc_b, tile_at(kt + 2u), whf, wb, opens);
            }
            convert_piece(kt + 1u, s + 1, refill, opens);
            slice_schedule();
        }
        __syncthreads();
        read_ops(buf ^ 1u, 0, af[0], bfr[0]);
        mfma_ops(af[1], bfr[1]);
        scales_a(kt + 2u, pos2);
        il_load_head(wsrc, tile_at(kt + 3u), whf, w, new_block);
        convert_piece(kt + 2u, 0);
        slice_schedule();
    };
    for (uint32_t kt = 0; kt < nk; kt += 4u) {
        k_step(kt, true, false, false, 2);
        k_step(kt + 1u, !Q6, true, false, 3);
        k_step(kt + 2u, true, false, true, 0);
        k_step(kt + 3u, !Q6, false, false, 1);
    }
    store_acc<TM, TN>(p, acc, m0 + wm * WM, n0 + wn * WN, lane);
}

// Sums the runs of the tiles that the persistent kernel's cut points split, adds the bias and stores Y.
// blockIdx.x = cut point (between workgroups b and b+1 of the walk), blockIdx.y = which of the 8
// accumulator blocks of every wave's 128 x 64 share; thread = (wave, lane) of the persistent kernel.  The
// first cut point inside a tile serves the tile.
__global__ __launch_bounds__(512) void gemm_sum_cut_tiles_kernel(GemmParams p)
{
    const uint32_t nk_all = p.K / GEMM_BK, share = p.units_per_wg;
    const uint32_t cut = (blockIdx.x + 1u) * share;
    if (cut >= p.units || cut % nk_all == 0u) return;
    const uint32_t tile = cut / nk_all, tile_u = tile * nk_all;
    if (blockIdx.x * share > tile_u) return;   // an earlier cut point lies inside the same tile
    const uint32_t b_first = blockIdx.x, b_last = min((tile_u + nk_all - 1u) / share, (p.units - 1u) / share);
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63u, g = blockIdx.y;
    f32x4 sum[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) sum[r] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    for (uint32_t b = b_first; b <= b_last; ++b) {
        const uint32_t slot = 2u * b + (b * share < tile_u ? 1u : 0u);
        const f32x4* src = (const f32x4*)(p.partial + (size_t)slot * 65536u) + wave * 2048u + g * 256u + lane;
#pragma unroll
        for (int r = 0; r < 4; ++r) sum[r] += src[r * 64];
    }
    // register 4r+e of block (i, j) of wave (wm, wn): token row 8r + 4*(lane/32) + e, weight row lane%32
    const uint32_t m0 = (tile / p.tiles_n) * 256u + (wave >> 2) * 128u + (g >> 1) * 32u + 4u * (lane >> 5);
    const uint32_t n = (tile % p.tiles_n) * 256u + (wave & 3u) * 64u + (g & 1u) * 32u + (lane & 31u);
    if (n >= p.N) return;
    const float bias = p.bias ? p.bias[n] : 0.0f;
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const uint32_t m = m0 + 8u * r + e;
            if (m < p.M) p.Y[(size_t)m * p.ldy + n] = sum[r][e] + bias;
        }
}

bool gemm_bf16_supported(const MatmulArgs& a)
{
    if (a.expert_idx) return false;
    if (a.type != KQ_TYPE_Q4_K && a.type != KQ_TYPE_Q5_K && a.type != KQ_TYPE_Q6_K) return false;
    if ((uintptr_t)a.X & 15u) return false;            // 128-bit loads of bf16 rows (K % 256 == 0 already)
    if (a.type != KQ_TYPE_Q6_K && (((uintptr_t)a.W & 15u) || (a.row_stride_bytes & 15u))) return false;
    if (a.type == KQ_TYPE_Q6_K && ((uintptr_t)a.W & 1u)) return false;
    return true;
}

template <int TYPE, int BM, int BN, int NWAVES>
static hipError_t launch_gemm(const GemmParams& p, hipStream_t s)
{
    constexpr size_t shmem = 2 * (size_t)(BM + BN) * GEMM_LD;
    auto kern = gemm_bf16_kernel<TYPE, BM, BN, NWAVES>;
    if (shmem > 64u * 1024u) {
        static bool raised = false;   // per instantiation
        if (!raised) {
            hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
            if (e != hipSuccess) return e;
            raised = true;
        }
    }
    dim3 grid((p.N + BN - 1) / BN, (p.M + BM - 1) / BM);
    hipLaunchKernelGGL(kern, grid, dim3(64 * NWAVES), shmem, s, p);
    return hipGetLastError();
}

// 256-tile kernel.  share = k steps per workgroup: nk for one tile per workgroup, otherwise the walk over all
// (tile, k step) units is cut into runs of that length.
template <int TYPE>
static hipError_t launch_gemm_persistent(GemmParams p, uint32_t share, const SplitScratch& sc, hipStream_t s)
{
    constexpr size_t shmem = 2 * (size_t)(256 + 256) * GEMM_LD;
    auto kern = gemm_bf16_sk_kernel<TYPE>;
    static bool raised = false;   // per instantiation
    if (!raised) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
        if (e != hipSuccess) return e;
        raised = true;
    }
    const uint32_t nk = p.K / GEMM_BK;
    p.tiles_n = (p.N + 255u) / 256u;
    const uint32_t tiles = ((p.M + 255u) / 256u) * p.tiles_n;
    p.units = tiles * nk;
    // cut tiles need two workspace slots per workgroup: without them, whole tiles
    if ((size_t)2u * ((p.units + share - 1u) / share) * 65536u > sc.capacity_floats) share = nk;
    share = (share + 3u) & ~3u;   // the k loop takes whole superblocks (nk is a multiple of 4)
    p.units_per_wg = share;
    p.partial = sc.partial;
    const uint32_t wgs = (p.units + p.units_per_wg - 1u) / p.units_per_wg;
    hipLaunchKernelGGL(kern, dim3(wgs), dim3(512), shmem, s, p);
    if (wgs > 1u && p.units_per_wg % nk != 0u)
        hipLaunchKernelGGL(gemm_sum_cut_tiles_kernel, dim3(wgs - 1u, 8), dim3(512), 0, s, p);
    return hipGetLastError();
}

template <int TYPE>
static hipError_t launch_gemm_n128(GemmParams p, hipStream_t s)
{
    constexpr size_t shmem = 2 * (size_t)(256 + 128) * GEMM_LD;
    auto kern = gemm_bf16_n128_kernel<TYPE>;
    static bool raised = false;   // per instantiation
    if (!raised) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
        if (e != hipSuccess) return e;
        raised = true;
    }
    p.tiles_n = (p.N + 127u) / 128u;
    const uint32_t tiles = ((p.M + 255u) / 256u) * p.tiles_n;
    hipLaunchKernelGGL(kern, dim3(tiles), dim3(512), shmem, s, p);
    return hipGetLastError();
}

template <int TYPE>
static hipError_t launch_gemm_n192(GemmParams p, hipStream_t s)
{
    constexpr size_t shmem = 2 * (size_t)(256 + 192) * GEMM_LD;
    auto kern = gemm_bf16_n192_kernel<TYPE>;
    static bool raised = false;   // per instantiation
    if (!raised) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
        if (e != hipSuccess) return e;
        raised = true;
    }
    p.tiles_n = (p.N + 191u) / 192u;
    const uint32_t tiles = ((p.M + 255u) / 256u) * p.tiles_n;
    hipLaunchKernelGGL(kern, dim3(tiles), dim3(512), shmem, s, p);
    return hipGetLastError();
}

hipError_t launch_gemm_bf16(const MatmulArgs& a, int tile, int split, const SplitScratch& sc, hipStream_t s)
{
    GemmParams p{};
    p.X = (const uint16_t*)a.X;
    p.W = a.W;
    p.bias = a.bias;
    p.Y = a.Y;
    p.M = a.M; p.N = a.N; p.K = a.K;
    p.n_blocks = a.n_blocks;
    p.row_stride_bytes = a.row_stride_bytes;
    p.ldy = a.ldy;
    const bool q4 = a.type == KQ_TYPE_Q4_K, q5 = a.type == KQ_TYPE_Q5_K;
    const GemmPlan plan = plan_gemm_bf16(a.type, a.M, a.N, a.K, device_cu_count(), tile, split);
    switch (plan.form) {
    case GEMM_FORM_HALF:
        return q4 ? launch_gemm_n128<KQ_TYPE_Q4_K>(p, s) : q5 ? launch_gemm_n128<KQ_TYPE_Q5_K>(p, s) : launch_gemm_n128<KQ_TYPE_Q6_K>(p, s);
    case GEMM_FORM_192:
        return q4 ? launch_gemm_n192<KQ_TYPE_Q4_K>(p, s) : q5 ? launch_gemm_n192<KQ_TYPE_Q5_K>(p, s) : launch_gemm_n192<KQ_TYPE_Q6_K>(p, s);
    case GEMM_FORM_ROUNDS_THEN_HALF: {
        GemmParams p1 = p, p2 = p;
        p1.N = plan.rows_first;
        p2.N = a.N - plan.rows_first;
        p2.W = p.W + (size_t)plan.rows_first * p.row_stride_bytes;
        p2.Y = p.Y + plan.rows_first;
        p2.bias = p.bias ? p.bias + plan.rows_first : nullptr;
        hipError_t e = q4 ? launch_gemm_persistent<KQ_TYPE_Q4_K>(p1, plan.share, sc, s)
                          : q5 ? launch_gemm_persistent<KQ_TYPE_Q5_K>(p1, plan.share, sc, s)
                               : launch_gemm_persistent<KQ_TYPE_Q6_K>(p1, plan.share, sc, s);
        if (e != hipSuccess) return e;
        return q4 ? launch_gemm_n128<KQ_TYPE_Q4_K>(p2, s) : q5 ? launch_gemm_n128<KQ_TYPE_Q5_K>(p2, s) : launch_gemm_n128<KQ_TYPE_Q6_K>(p2, s);
    }
    case GEMM_FORM_WHOLE:
    case GEMM_FORM_SHARES:
        return q4 ? launch_gemm_persistent<KQ_TYPE_Q4_K>(p, plan.share, sc, s)
                  : q5 ? launch_gemm_persistent<KQ_TYPE_Q5_K>(p, plan.share, sc, s) : launch_gemm_persistent<KQ_TYPE_Q6_K>(p, plan.share, sc, s);
    default:
        return q4 ? launch_gemm<KQ_TYPE_Q4_K, 128, 128, 4>(p, s)
                  : q5 ? launch_gemm<KQ_TYPE_Q5_K, 128, 128, 4>(p, s) : launch_gemm<KQ_TYPE_Q6_K, 128, 128, 4>(p, s);
    }
}

}  // namespace kq
