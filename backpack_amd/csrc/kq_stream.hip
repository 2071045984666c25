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
#include "kq_wave.h"
#include "kq_stream_core.h"   // hand-waited loads: KQ_REQUIRES_NO_SPILL (the build refuses this file if a kernel spills)
#include <type_traits>


namespace kq {


// Kernel arguments come in three sizes, and a kernel is compiled for each: the wave's first
// instructions fetch them, and every further 64 bytes of them cost a launch a measurable fraction of a
// microsecond, so the dense decode matvec gets the smallest set that describes it.
struct StreamDense {          // 64 bytes = the 16 dwords that kernel-argument preloading holds
    const float* X;
    const uint8_t* W;
    const float* bias;
    float* Y;
    uint32_t N, K, n_blocks, row_stride_bytes, y_offset, ldy;
    uint32_t M;   // tokens; read only by the four-token kernels (three tokens run as four, the last one masked)
    uint32_t grid_x;   // workgroups of the launch along x (as an argument: the hidden one would be a fetch of its own)
    static constexpr bool kGrouped = false, kFused = false, kCombine = false;
};

// Dense matvec with a prologue on the activations (STREAM_PRO_*; for the act forms the X rows are
// gate | up, 2K floats) and a term added to every output (indexed like Y; may be Y itself).
struct StreamFused {
    const float* X;
    const uint8_t* W;
    const float* bias;
    float* Y;
    uint32_t N, K, n_blocks, row_stride_bytes, y_offset, ldy;
    uint32_t M;
    int pro;
    float eps;
    const float* norm_w;
    const float* residual;
    // 0, or STREAM_PRO_SILU / STREAM_PRO_GELU: W is gate | up stacked (N rows in all, N/2 outputs) and
    // Y[n] = act(gate_n . x) * (up_n . x): a wave takes both rows of a pair, one after the other
    int epi;
    uint32_t grid_x;   // workgroups of the launch along x
    static constexpr bool kGrouped = false, kFused = true, kCombine = false;
};

// Expert indirection: blockIdx.y is a (token, slot) pair that uses weight rows expert_idx[pair]*N ..
// +N-1, X row pair / k_slots (or pair, x_per_slot) and Y row pair.  MoE FFN fusions: a twin matrix of
// the same shape served by blockIdx.z == 1 (gate and up read the same x), and an activation input:
// x = silu(X) * X2 (down reads gate and up).
struct StreamGrouped {
    const float* X;
    const uint8_t* W;
    const float* bias;
    float* Y;
    uint32_t N, K, n_blocks, row_stride_bytes, y_offset, ldy;
    uint32_t M;
    const uint32_t* expert_idx;
    uint32_t k_slots;
    int x_per_slot;
    const uint8_t* W2;
    float* Y2;
    const float* X2;
    static constexpr bool kGrouped = true, kFused = false, kCombine = false;
};

// The last matvec of an expert FFN with the weighted sum over a token's slots folded in (Q6_K kernel): blockIdx.y
// is a token, wave w of the workgroup serves the token's slot w (pair token * k_slots + w) over the same rows as
// the other waves, and where the K slices of a long row would meet, the slots' results meet instead:
// Y[token, r] = sum over slots, in slot order, of wt[pair] * (W[expert_idx[pair]] x[pair])[r].
struct StreamCombine : StreamGrouped {
    const float* wt;
    static constexpr bool kCombine = true;
};


// Redirects the pointers of a grouped launch to the pair this workgroup serves.
__device__ __forceinline__ void stream_select_pair(StreamGrouped& p)
{
    if (blockIdx.z) { p.W = p.W2; p.Y = p.Y2; }
    const uint32_t pair = blockIdx.y;
    p.W += (size_t)p.expert_idx[pair] * p.N * p.row_stride_bytes;
    const size_t xrow = (size_t)(p.x_per_slot ? pair : pair / p.k_slots) * p.K;
    p.X += xrow;
    if (p.X2) p.X2 += xrow;
    p.Y += (size_t)pair * p.ldy;
}
// The pair of wave `wave` in a slot-combining launch; returns the pair's weight.  Waves beyond the token's
// slots repeat the last slot and are left out of the sum.
__device__ __forceinline__ float stream_select_slot(StreamCombine& p, uint32_t wave)
{
    const uint32_t tok = blockIdx.y;
    const uint32_t pair = tok * p.k_slots + min(wave, p.k_slots - 1u);
    p.W += (size_t)p.expert_idx[pair] * p.N * p.row_stride_bytes;
    const size_t xrow = (size_t)(p.x_per_slot ? pair : tok) * p.K;
    p.X += xrow;
    if (p.X2) p.X2 += xrow;
    p.Y += (size_t)tok * p.ldy;
    return p.wt[pair];
}
template <typename PT> __device__ __forceinline__ float stream_select_slot(PT&, uint32_t) { return 1.0f; }
__device__ __forceinline__ void stream_select_pair(StreamDense&) {}
__device__ __forceinline__ void stream_touch_late_args(const StreamFused& p)
{
    asm volatile("" ::"s"(p.Y), "s"(p.bias), "s"(p.residual), "s"(p.ldy), "s"(p.y_offset));
}
template <typename PT> __device__ __forceinline__ void stream_touch_late_args(const PT&) {}
__device__ __forceinline__ uint32_t stream_grid_x(const StreamDense& p) { return p.grid_x; }
__device__ __forceinline__ uint32_t stream_grid_x(const StreamFused& p) { return p.grid_x; }
template <typename PT> __device__ __forceinline__ uint32_t stream_grid_x(const PT&) { return gridDim.x; }
__device__ __forceinline__ void stream_select_pair(StreamFused&) {}

// Which prologue a launch runs, where the second activation input lies relative to the first (in
// floats), and the distance between the X rows of two tokens.
__device__ __forceinline__ int stream_pro(const StreamDense&) { return STREAM_PRO_NONE; }
__device__ __forceinline__ int stream_pro(const StreamFused& p) { return p.pro; }
__device__ __forceinline__ int stream_pro(const StreamGrouped& p) { return p.X2 ? STREAM_PRO_SILU : STREAM_PRO_NONE; }
__device__ __forceinline__ ptrdiff_t stream_x2_off(const StreamDense&) { return 0; }
__device__ __forceinline__ ptrdiff_t stream_x2_off(const StreamFused& p) { return (ptrdiff_t)p.K; }
__device__ __forceinline__ ptrdiff_t stream_x2_off(const StreamGrouped& p) { return p.X2 - p.X; }
__device__ __forceinline__ const float* stream_norm_w(const StreamFused& p) { return p.norm_w; }
__device__ __forceinline__ float stream_eps(const StreamFused& p) { return p.eps; }
template <typename PT> __device__ __forceinline__ const float* stream_norm_w(const PT&) { return nullptr; }
template <typename PT> __device__ __forceinline__ float stream_eps(const PT&) { return 0.0f; }
__device__ __forceinline__ const float* stream_residual(const StreamFused& p) { return p.residual; }
__device__ __forceinline__ int stream_epi(const StreamFused& p) { return p.epi; }
template <typename PT> __device__ __forceinline__ int stream_epi(const PT&) { return 0; }
template <typename PT> __device__ __forceinline__ const float* stream_residual(const PT&) { return nullptr; }
__device__ __forceinline__ uint32_t stream_ldx(const StreamDense& p) { return p.K; }
__device__ __forceinline__ uint32_t stream_ldx(const StreamFused& p) { return p.pro >= STREAM_PRO_SILU ? 2u * p.K : p.K; }
__device__ __forceinline__ uint32_t stream_ldx(const StreamGrouped& p) { return p.K; }


// v where mask is all ones, +0 where it is zero (bitwise: no branch, no NaN from a product with zero)
__device__ __forceinline__ float4 stream_keep(float4 v, uint32_t mask)
{
    return float4{__builtin_bit_cast(float, __builtin_bit_cast(uint32_t, v.x) & mask),
                  __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, v.y) & mask),
                  __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, v.z) & mask),
                  __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, v.w) & mask)};
}

// Four activations: X as it is (also for the norm, which scales afterwards), or act(X) * X2.
template <int PRO, bool FAST>
__device__ __forceinline__ float4 stream_x4(const float4* xp, ptrdiff_t x2_off)
{
    float4 v = *xp;
    if constexpr (PRO == STREAM_PRO_SILU || PRO == STREAM_PRO_GELU) {
        const float4 u = *(const float4*)((const float*)xp + x2_off);
        v.x = stream_act<PRO, FAST>(v.x, u.x);
        v.y = stream_act<PRO, FAST>(v.y, u.y);
        v.z = stream_act<PRO, FAST>(v.z, u.z);
        v.w = stream_act<PRO, FAST>(v.w, u.w);
    }
    return v;
}

// A workgroup barrier that waits for the wave's LDS traffic only (__syncthreads also drains the vector memory
// counter, i.e. the ring of weight rows in flight).
__device__ __forceinline__ void lds_barrier()
{
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// One branch around a whole x prologue, so that every form issues its loads back to back.  A kernel
// carries only the forms its argument set can ask for.
template <typename PT, typename F>
__device__ __forceinline__ void stream_dispatch_pro(const PT& p, F&& f)
{
    if constexpr (PT::kFused) {
        const int pro = stream_pro(p);
        if (pro == STREAM_PRO_NONE) f(std::integral_constant<int, STREAM_PRO_NONE>{});
        else if (pro == STREAM_PRO_SILU) f(std::integral_constant<int, STREAM_PRO_SILU>{});
        else if (pro == STREAM_PRO_NORM) f(std::integral_constant<int, STREAM_PRO_NORM>{});
        else f(std::integral_constant<int, STREAM_PRO_GELU>{});
    } else if constexpr (PT::kGrouped) {
        if (stream_pro(p) == STREAM_PRO_SILU) f(std::integral_constant<int, STREAM_PRO_SILU>{});
        else f(std::integral_constant<int, STREAM_PRO_NONE>{});
    } else {
        f(std::integral_constant<int, STREAM_PRO_NONE>{});
    }
}


// P passes of 8 superblocks cover a row (n_blocks <= 8 * P) or, with KW > 1, a wave's K slice of it
// (n_blocks <= 8 * P * KW); D rows in flight; MT tokens.  KW == 1: a workgroup is NW independent waves,
// each with rows of its own.  KW > 1: the KW waves of a workgroup walk the same rows, one K slice each,
// and their sums meet in LDS once per 64 rows (the form of the Q6_K kernel below).
template <int P, int NW, int D, int MT, typename PT, bool Q5 = false, int KW = 1>
__device__ __forceinline__ void q4k_stream_body(PT p)
{
    stream_select_pair(p);
    __shared__ float part[KW > 1 ? KW * NW : 1][MT][64];
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // NW > 1 and KW > 1 together: the workgroup is KW K slices x NW walkers; the walkers of a slice share its
    // activations, the slices of a walker fold their sums (wave = slice * NW + walker)
    const uint32_t slice = KW > 1 ? (NW > 1 ? wave / NW : wave) : 0u;
    const uint32_t walker = NW > 1 ? (KW > 1 ? wave % NW : wave) : 0u;
    const uint32_t gw0 = blockIdx.x * NW + walker;
    // rows gw, gw + stride, ...: at any moment the waves of the grid read
    // consecutive rows, one contiguous stream across the memory channels
    const uint32_t stride = stream_grid_x(p) * NW;
    // pair mode (fused kernels only): the wave walks pairs gw, gw + stride, ... of the N/2 outputs and its
    // ring alternates between a pair's gate row and its up row, N/2 rows further on
    const bool pairs = PT::kFused && stream_epi(p) != 0;
    const uint32_t n_walk_all = pairs ? p.N / 2u : p.N;
    // STAGE (whole-row waves, several to a workgroup): the workgroup fetches the activations once and its waves
    // take their operands from LDS; every wave loading the row for itself costs a CU's vector cache eight times
    // the bytes (16 KB per wave and token, twice that with norm weights: 1 to 3 us of a launch).
    constexpr bool STAGE = NW > 1;
    extern __shared__ float4 xstage_all[];   // STAGE: [slice][token][8 * P slots][64 lanes], sized by the launch
    float4* xstage = xstage_all + slice * (MT * P * 8 * 64);
    __shared__ float ssq_part[STAGE ? NW * KW : 1][MT];
    const bool idle = gw0 >= n_walk_all;   // NW == 1: the whole workgroup
    if (!STAGE && idle) return;
    const uint32_t gw = idle ? 0u : gw0;   // (a staged workgroup's idle waves help fetch the activations, then leave)
    const uint32_t n_walk = (n_walk_all - gw + stride - 1u) / stride;
    const uint32_t n_rows = pairs ? 2u * n_walk : n_walk;
    auto row_of = [&](uint32_t i) -> size_t {
        i = min(i, n_rows - 1u);
        if (PT::kFused && pairs) return (size_t)(gw + (i >> 1) * stride) + (size_t)(i & 1u) * n_walk_all;
        return (size_t)(gw + i * stride);
    };
    const uint32_t bl = lane >> 3, j = lane & 7u, g = j >> 1, h = j & 1u;
    const bool sel_hi = g >= 2u;
    const uint32_t sh = 16u * (g & 1u);
    constexpr uint32_t BLOCK = Q5 ? KQ_Q5K_BYTES : KQ_Q4K_BYTES;

    float xlo[P][MT][16], xhi[P][MT][16], xs_lo[P][MT], xs_hi[P][MT];
    uint32_t hoff[P];
    const uint32_t ldx = stream_ldx(p);
    const ptrdiff_t x2_off = stream_x2_off(p);
    // RMSNorm prologue: the activations are held as x * norm_w (both loaded back to back: one round trip
    // to memory, not two) and the row's 1/rms, which needs the whole row, scales the finished outputs.
    float rstd0 = 1.0f, rstd1 = 1.0f;   // (the fused forms take one or two tokens; two scalars: an array went to scratch memory)
    auto load_x = [&](auto pro) {
        constexpr int PRO = decltype(pro)::value;
        constexpr bool NORM = PRO == STREAM_PRO_NORM && PT::kFused;
        float ssq[MT];
#pragma unroll
        for (int t = 0; t < MT; ++t) ssq[t] = 0.0f;
#pragma unroll
        for (int pass = 0; pass < P; ++pass) {
            uint32_t b = (slice * P + pass) * 8u + bl;
            const bool valid = b < p.n_blocks;
            const uint32_t keep = valid ? 0xFFFFFFFFu : 0u;   // activations of superblocks beyond K read as zero
            b = valid ? b : p.n_blocks - 1u;
            hoff[pass] = b * BLOCK;
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                const uint32_t xt = MT > 2 ? min((uint32_t)t, p.M - 1u) : (uint32_t)t;   // a masked token re-reads the last one
                const float4* xp = (const float4*)(p.X + (size_t)xt * ldx + (size_t)b * KQ_QK + 64u * g + 16u * h);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float4 lo = stream_x4<PRO, PT::kFused>(xp + i, x2_off), hi = stream_x4<PRO, PT::kFused>(xp + 8 + i, x2_off);
                    lo = stream_keep(lo, keep);   // (no branch here: one around a load makes every load wait for the one before)
                    hi = stream_keep(hi, keep);
                    if constexpr (NORM) {
                        const float4* wp = (const float4*)(stream_norm_w(p) + (size_t)b * KQ_QK + 64u * g + 16u * h);
                        const float4 wl = wp[i], wh = wp[8 + i];
                        float s = ssq[t];
                        s = __builtin_fmaf(lo.x, lo.x, s); s = __builtin_fmaf(lo.y, lo.y, s);
                        s = __builtin_fmaf(lo.z, lo.z, s); s = __builtin_fmaf(lo.w, lo.w, s);
                        s = __builtin_fmaf(hi.x, hi.x, s); s = __builtin_fmaf(hi.y, hi.y, s);
                        s = __builtin_fmaf(hi.z, hi.z, s); s = __builtin_fmaf(hi.w, hi.w, s);
                        ssq[t] = s;
                        lo.x *= wl.x; lo.y *= wl.y; lo.z *= wl.z; lo.w *= wl.w;
                        hi.x *= wh.x; hi.y *= wh.y; hi.z *= wh.z; hi.w *= wh.w;
                    }
                    xlo[pass][t][4 * i + 0] = lo.x; xlo[pass][t][4 * i + 1] = lo.y; xlo[pass][t][4 * i + 2] = lo.z; xlo[pass][t][4 * i + 3] = lo.w;
                    xhi[pass][t][4 * i + 0] = hi.x; xhi[pass][t][4 * i + 1] = hi.y; xhi[pass][t][4 * i + 2] = hi.z; xhi[pass][t][4 * i + 3] = hi.w;
                }
                float sl = 0.0f, sh_ = 0.0f;
#pragma unroll
                for (int i = 0; i < 16; ++i) { sl += xlo[pass][t][i]; sh_ += xhi[pass][t][i]; }
                xs_lo[pass][t] = sl;
                xs_hi[pass][t] = sh_;
            }
        }
        if constexpr (NORM) {
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                float ss = wave_sum(ssq[t]);   // the wave holds the whole row, or a K slice of it
                if (KW > 1) {                  // the slices' sums of squares meet in LDS
                    if (lane == 0) part[slice][t][0] = ss;
                    __syncthreads();
                    ss = part[0][t][0];
#pragma unroll
                    for (int w = 1; w < KW; ++w) ss += part[w][t][0];
                }
                const float r = 1.0f / sqrtf(ss / (float)p.K + stream_eps(p));
                if (t == 0) rstd0 = r; else rstd1 = r;
            }
            if (KW > 1) __syncthreads();   // part is reused by the row loop
        }
    };
    // Ring of D rows in flight.  Slot d is refilled as soon as its row has been
    // consumed; the wait before a slot's arithmetic leaves the (D-1) younger
    // slots' loads outstanding.  Past the end of the wave's rows the last row is
    // fetched and summed again (cache hits, result dropped), so the row loop has
    // no branch and the number of loads in flight is the same at every wait.
    constexpr int SLOT_LOADS = (Q5 ? 3 : 2) * P;
    Q4Slot<P, Q5> ring[D] = {};
    if constexpr (STAGE) {
        // Slot sl = 8 * pass + q of the staging area holds, for lane L, the q-th 16 bytes of that lane's
        // operands of the pass (q < 4: low nibbles' elements, else high nibbles'): wave w fetches slots
        // w, w + NW, ... exactly as the lane would have, and a wave's reads are 1 KB runs.
        // Order: the wave's few activation loads, then the ring's first rows (weights never depend on x), then
        // a wait that leaves exactly the ring outstanding: the whole x path — prologue arithmetic, LDS, the
        // barrier (which waits for LDS only), the sums — runs under the first weights' flight.
        constexpr int XL = P * 8 / NW;
        constexpr bool EXTRA = PT::kFused || PT::kGrouped;   // a second operand: norm weights, or the act's other input
        s_u32x4 xr[MT][XL] = {}, er[EXTRA ? MT : 1][EXTRA ? XL : 1] = {};
        uint32_t keep[XL];
        const int pro_rt = stream_pro(p);
#pragma unroll
        for (int k = 0; k < XL; ++k) {
            const uint32_t sl = walker + (uint32_t)k * NW, q = sl & 7u;
            uint32_t b = (slice * P + (sl >> 3)) * 8u + bl;
            const bool valid = b < p.n_blocks;
            keep[k] = valid ? 0xFFFFFFFFu : 0u;   // activations of superblocks beyond K read as zero
            b = valid ? b : p.n_blocks - 1u;
            const size_t at = (size_t)b * KQ_QK + 64u * g + 16u * h + 32u * (q >> 2) + 4u * (q & 3u);
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                const uint32_t xt = MT > 2 ? min((uint32_t)t, p.M - 1u) : (uint32_t)t;   // a masked token re-reads the last one
                const float* xp = p.X + (size_t)xt * ldx + at;
                ring_load16(xr[t][k], (const uint8_t*)xp);
                if constexpr (EXTRA) {
                    const float* ep = pro_rt == STREAM_PRO_NORM ? stream_norm_w(p) + at
                                    : pro_rt == STREAM_PRO_NONE ? xp : xp + x2_off;
                    ring_load16(er[t][k], (const uint8_t*)ep);
                }
            }
        }
#pragma unroll
        for (int pass = 0; pass < P; ++pass) hoff[pass] = min((slice * P + (uint32_t)pass) * 8u + bl, p.n_blocks - 1u) * BLOCK;
#pragma unroll
        for (int d = 0; d < D; ++d)
            ring[d].fill(p.W + row_of((uint32_t)d) * p.row_stride_bytes, hoff, j);
        // (arguments beyond the preloaded ones are fetched now, under the first weights' flight, not at the stores)
        stream_touch_late_args(p);
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(D * SLOT_LOADS));
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int k = 0; k < XL; ++k) {
                asm volatile("; ringwait %0" : "+v"(xr[t][k]));
                if constexpr (EXTRA) asm volatile("; ringwait %0" : "+v"(er[t][k]));
            }
        auto stage_x = [&](auto pro) {
            constexpr int PRO = decltype(pro)::value;
            constexpr bool NORM = PRO == STREAM_PRO_NORM && PT::kFused;
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                float ssq = 0.0f;
#pragma unroll
                for (int k = 0; k < XL; ++k) {
                    const uint32_t sl = walker + (uint32_t)k * NW;
                    float4 v = __builtin_bit_cast(float4, xr[t][k]);
                    if constexpr (PRO == STREAM_PRO_SILU || PRO == STREAM_PRO_GELU) {
                        const float4 u = __builtin_bit_cast(float4, er[EXTRA ? t : 0][EXTRA ? k : 0]);
                        v.x = stream_act<PRO, PT::kFused>(v.x, u.x);
                        v.y = stream_act<PRO, PT::kFused>(v.y, u.y);
                        v.z = stream_act<PRO, PT::kFused>(v.z, u.z);
                        v.w = stream_act<PRO, PT::kFused>(v.w, u.w);
                    }
                    v = stream_keep(v, keep[k]);
                    if constexpr (NORM) {
                        const float4 w = __builtin_bit_cast(float4, er[EXTRA ? t : 0][EXTRA ? k : 0]);
                        ssq = __builtin_fmaf(v.x, v.x, __builtin_fmaf(v.y, v.y, __builtin_fmaf(v.z, v.z, __builtin_fmaf(v.w, v.w, ssq))));
                        v.x *= w.x; v.y *= w.y; v.z *= w.z; v.w *= w.w;
                    }
                    xstage[((uint32_t)t * P * 8u + sl) * 64u + lane] = v;
                }
                if constexpr (NORM) {
                    const float ss = wave_sum(ssq);
                    if (lane == 0) ssq_part[wave][t] = ss;   // (every element of x is fetched by exactly one wave)
                }
            }
        };
        stream_dispatch_pro(p, stage_x);
        // (the workgroup's LDS writes are all the barrier has to wait for: a full fence would drain the ring)
        lds_barrier();
        if (idle) {
            asm volatile("s_waitcnt vmcnt(0)");
            return;
        }
#pragma unroll
        for (int pass = 0; pass < P; ++pass) {
#pragma unroll
            for (int t = 0; t < MT; ++t) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float4 lo = xstage[((uint32_t)t * P * 8u + pass * 8u + i) * 64u + lane];
                    const float4 hi = xstage[((uint32_t)t * P * 8u + pass * 8u + 4u + i) * 64u + lane];
                    xlo[pass][t][4 * i + 0] = lo.x; xlo[pass][t][4 * i + 1] = lo.y; xlo[pass][t][4 * i + 2] = lo.z; xlo[pass][t][4 * i + 3] = lo.w;
                    xhi[pass][t][4 * i + 0] = hi.x; xhi[pass][t][4 * i + 1] = hi.y; xhi[pass][t][4 * i + 2] = hi.z; xhi[pass][t][4 * i + 3] = hi.w;
                }
                float sl = 0.0f, sh_ = 0.0f;
#pragma unroll
                for (int i = 0; i < 16; ++i) { sl += xlo[pass][t][i]; sh_ += xhi[pass][t][i]; }
                xs_lo[pass][t] = sl;
                xs_hi[pass][t] = sh_;
            }
        }
        if (PT::kFused && pro_rt == STREAM_PRO_NORM) {
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                float ss = ssq_part[0][t];
#pragma unroll
                for (int w = 1; w < NW * KW; ++w) ss += ssq_part[w][t];
                const float r = 1.0f / sqrtf(ss / (float)p.K + stream_eps(p));
                if (t == 0) rstd0 = r; else rstd1 = r;
            }
        }
    } else {
        stream_dispatch_pro(p, load_x);
        // (the activation sums are finished before the first weight is requested)
#pragma unroll
        for (int pass = 0; pass < P; ++pass)
#pragma unroll
            for (int t = 0; t < MT; ++t) asm volatile("" ::"v"(xs_lo[pass][t]), "v"(xs_hi[pass][t]));
        // (Here the ring is filled after the prologue even where that is long: the sliced forms' prologue has
        // a full barrier in it.)
#pragma unroll
        for (int d = 0; d < D; ++d)
            ring[d].fill(p.W + row_of((uint32_t)d) * p.row_stride_bytes, hoff, j);
        // (arguments beyond the preloaded ones are fetched now, under the first weights' flight, not at the stores)
        stream_touch_late_args(p);
    }
    // Rows are taken 64 at a time: lane i keeps the sums of the chunk's row i, and the
    // chunk is stored (bias added) after its last row.
    for (uint32_t c0 = 0; c0 < n_rows; c0 += 64u) {
        const uint32_t cnt = min(64u, n_rows - c0);
        float res[MT];
#pragma unroll
        for (int t = 0; t < MT; ++t) res[t] = 0.0f;
        for (uint32_t i0 = 0; i0 < cnt; i0 += D) {
#pragma unroll
            for (int d = 0; d < D; ++d) {
                const uint32_t i = i0 + d;
                ring[d].template wait<(D - 1) * SLOT_LOADS>();
                float acc[MT];
#pragma unroll
                for (int t = 0; t < MT; ++t) acc[t] = 0.0f;
#pragma unroll
                for (int pass = 0; pass < P; ++pass)
                    q4k_piece_dot<MT, Q5>(ring[d].hdr[pass], ring[d].q[pass], xlo[pass], xhi[pass], xs_lo[pass],
                                          xs_hi[pass], sel_hi, sh, acc, ring[d].qh[Q5 ? pass : 0], 2u * g);
                ring[d].fill(p.W + row_of(c0 + i + D) * p.row_stride_bytes, hoff, j);
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    const float tot = wave_sum(acc[t]);
                    res[t] = (lane == i && i < cnt) ? tot : res[t];
                }
            }
        }
        // (the slices' barriers wait for LDS only: a full fence would drain the ring.  Walkers of a workgroup may
        // differ by a chunk; a wave that has ended no longer counts at a barrier.)
        if (KW > 1) {
#pragma unroll
            for (int t = 0; t < MT; ++t) part[slice * NW + walker][t][lane] = res[t];
            lds_barrier();
        }
        // (the lane guard stays outside: with it inside, the gate|up launch measured 3 us slower.  In pair
        // mode cnt is even, so a lane inside the guard finds its partner there too.)
        if ((KW == 1 || slice == 0) && lane < cnt) {
            const uint32_t r = (uint32_t)row_of(c0 + lane);
            const float bias = p.bias ? p.bias[r] : 0.0f;
#pragma unroll
            for (int t = 0; t < MT; ++t) {
                float y = res[t];
                if (KW > 1) {
                    y = part[walker][t][lane];
#pragma unroll
                    for (int w = 1; w < KW; ++w) y += part[w * NW + walker][t][lane];
                }
                if constexpr (PT::kFused) y *= t == 0 ? rstd0 : rstd1;
                y += bias;
                if (PT::kFused && pairs) {
                    // lanes 2j and 2j + 1 hold a pair's gate and up products: the even lane stores the output
                    const float up = group_partner<1>(y);
                    y = stream_epi(p) == STREAM_PRO_SILU ? stream_act<STREAM_PRO_SILU, true>(y, up)
                                                         : stream_act<STREAM_PRO_GELU, true>(y, up);
                    if (!(lane & 1u)) p.Y[(size_t)t * p.ldy + p.y_offset + r] = y;
                    continue;
                }
                if (MT > 2 && (uint32_t)t >= p.M) continue;
                const size_t at = (size_t)t * p.ldy + p.y_offset + r;
                if constexpr (PT::kFused) y += stream_residual(p) ? stream_residual(p)[at] : 0.0f;
                p.Y[at] = y;
            }
        }
        if (KW > 1) lds_barrier();
    }
    asm volatile("s_waitcnt vmcnt(0)");   // the ring's last refills land before the wave ends
}

// ---------------------------------------------------------------------------
// Q6_K.  Lane (b, t) = (lane / 8, lane % 8) of a pass takes, in superblock b of
// the pass's eight, half n = t / 4 and the eight positions l = 8*(t%4) .. +7:
// 8 bytes of ql[64n + l], 8 of ql[64n + 32 + l], 8 of qh[32n + l] — the 32
// elements 128n + 32k + l, k = 0..3 — plus the half's 8 scale bytes and d.
// Blocks are 210 bytes, so these loads are only 2-byte aligned; the hardware
// takes them as they are.  A row longer than 8*P blocks is cut into KW slices,
// one wave each; the slices' sums meet in LDS once per 64 rows.
// ---------------------------------------------------------------------------


// Workgroup = KW waves, one K slice of 8*P superblocks each; the workgroup walks
// rows blockIdx.x, + gridDim.x, ...; D rows in flight per wave.
// RW = 2 (combining and grouped launches, rows of at most four superblocks): the two halves of a wave take two rows at a
// time, four superblocks of eight lanes each, so that a row of three superblocks keeps 48 of the 64 lanes busy
// instead of 24; a step's two sums are those of the halves.
template <int P, int KW, int D, int MT, typename PT, int RW = 1>
__device__ __forceinline__ void q6k_stream_body(PT p)
{
    constexpr bool COMBINE = PT::kCombine;   // the waves are a token's slots, not K slices
    static_assert(RW == 1 || (RW == 2 && (COMBINE || (PT::kGrouped && KW == 1)) && P == 1 && MT == 1),
                  "two rows per step: the combining launch, or a grouped one whose rows one wave walks");
    __shared__ float part[KW > 1 ? KW : 1][MT][64];
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t slots = COMBINE ? min(p.M, (uint32_t)KW) : (uint32_t)KW;   // (a combining launch passes its slots per token in M)
    float slot_wt = 1.0f;
    if constexpr (COMBINE) slot_wt = stream_select_slot(p, wave);
    else stream_select_pair(p);
    const uint32_t kslice = COMBINE ? 0u : wave;
    const uint32_t g = blockIdx.x, stride = stream_grid_x(p);
    const uint32_t n_rows = g < p.N ? (p.N - g + stride - 1u) / stride : 0u;
    const uint32_t bl = RW == 2 ? (lane >> 3) & 3u : lane >> 3, t = lane & 7u, n = t >> 2, lg = t & 3u;
    const uint32_t rsel = RW == 2 ? lane >> 5 : 0u;   // which of a step's rows this half of the wave takes
    const uint32_t sc_shift = 8u * (lg >> 1);
    // row of this workgroup's walk that the lane takes in step j (clamped to the last: fetched, never stored)
    auto row_ptr = [&](uint32_t j) {
        const uint32_t ri = min(RW == 2 ? 2u * j + rsel : j, n_rows - 1u);
        return p.W + (size_t)(g + ri * stride) * p.row_stride_bytes;
    };

    float x[P][MT][4][8], m32xs[P][MT][4];
    uint32_t boff[P];
    const uint32_t ldx = stream_ldx(p);
    const ptrdiff_t x2_off = stream_x2_off(p);
    // (RMSNorm prologue as in the Q4_K kernel: x * norm_w in one round trip, 1/rms on the outputs)
    float rstd0 = 1.0f, rstd1 = 1.0f;   // (the fused forms take one or two tokens; two scalars: an array went to scratch memory)
    auto load_x = [&](auto pro) {
        constexpr int PRO = decltype(pro)::value;
        constexpr bool NORM = PRO == STREAM_PRO_NORM && PT::kFused;
        float ssq[MT];
#pragma unroll
        for (int tk = 0; tk < MT; ++tk) ssq[tk] = 0.0f;
#pragma unroll
        for (int pass = 0; pass < P; ++pass) {
            uint32_t b = (kslice * P + pass) * 8u + bl;
            const bool valid = b < p.n_blocks;
            const uint32_t keep = valid ? 0xFFFFFFFFu : 0u;   // activations of superblocks beyond K read as zero
            b = valid ? b : p.n_blocks - 1u;
            boff[pass] = b * KQ_Q6K_BYTES;
#pragma unroll
            for (int tk = 0; tk < MT; ++tk) {
                const uint32_t xt = MT > 2 ? min((uint32_t)tk, p.M - 1u) : (uint32_t)tk;
                const float4* xp = (const float4*)(p.X + (size_t)xt * ldx + (size_t)b * KQ_QK + 128u * n + 8u * lg);
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    float4 lo = stream_x4<PRO, PT::kFused>(xp + 8 * k, x2_off), hi = stream_x4<PRO, PT::kFused>(xp + 8 * k + 1, x2_off);
                    lo = stream_keep(lo, keep);
                    hi = stream_keep(hi, keep);
                    if constexpr (NORM) {
                        const float4* wp = (const float4*)(stream_norm_w(p) + (size_t)b * KQ_QK + 128u * n + 8u * lg);
                        const float4 wl = wp[8 * k], wh = wp[8 * k + 1];
                        float s = ssq[tk];
                        s = __builtin_fmaf(lo.x, lo.x, s); s = __builtin_fmaf(lo.y, lo.y, s);
                        s = __builtin_fmaf(lo.z, lo.z, s); s = __builtin_fmaf(lo.w, lo.w, s);
                        s = __builtin_fmaf(hi.x, hi.x, s); s = __builtin_fmaf(hi.y, hi.y, s);
                        s = __builtin_fmaf(hi.z, hi.z, s); s = __builtin_fmaf(hi.w, hi.w, s);
                        ssq[tk] = s;
                        lo.x *= wl.x; lo.y *= wl.y; lo.z *= wl.z; lo.w *= wl.w;
                        hi.x *= wh.x; hi.y *= wh.y; hi.z *= wh.z; hi.w *= wh.w;
                    }
                    x[pass][tk][k][0] = lo.x; x[pass][tk][k][1] = lo.y; x[pass][tk][k][2] = lo.z; x[pass][tk][k][3] = lo.w;
                    x[pass][tk][k][4] = hi.x; x[pass][tk][k][5] = hi.y; x[pass][tk][k][6] = hi.z; x[pass][tk][k][7] = hi.w;
                    float sum = 0.0f;
#pragma unroll
                    for (int i = 0; i < 8; ++i) sum += x[pass][tk][k][i];
                    m32xs[pass][tk][k] = -32.0f * sum;
                }
            }
        }
        if constexpr (NORM) {
#pragma unroll
            for (int tk = 0; tk < MT; ++tk) {
                float ss = wave_sum(ssq[tk]);   // each wave holds a K slice: the slices' sums of squares meet in LDS
                if (KW > 1) {
                    if (lane == 0) part[wave][tk][0] = ss;
                    __syncthreads();
                    ss = part[0][tk][0];
#pragma unroll
                    for (int w = 1; w < KW; ++w) ss += part[w][tk][0];
                }
                const float r = 1.0f / sqrtf(ss / (float)p.K + stream_eps(p));
                if (tk == 0) rstd0 = r; else rstd1 = r;
            }
            if (KW > 1) __syncthreads();   // part is reused by the row loop
        }
    };
    if (n_rows == 0) return;   // whole workgroup
    constexpr int SLOT_LOADS = 5 * P;
    Q6Slot<P> ring[D] = {};
    stream_dispatch_pro(p, load_x);
    // The activations' sums are complete before the first weight request goes out: here, arithmetic on
    // them that sank below the ring's fill waited for the weights as well and cost half a microsecond
    // per launch (volatile statements keep their order, and this one makes the sums its operands).
    // (The staged Q4_K order — activation loads, ring, a wait that leaves the ring outstanding — measured
    // slower here: down 12.2 -> 12.6 us, with the act * up prologue's sixteen loads +1 us.)
#pragma unroll
    for (int pass = 0; pass < P; ++pass)
#pragma unroll
        for (int tk = 0; tk < MT; ++tk)
            asm volatile("" : "+v"(m32xs[pass][tk][0]), "+v"(m32xs[pass][tk][1]), "+v"(m32xs[pass][tk][2]), "+v"(m32xs[pass][tk][3]));
#pragma unroll
    for (int d = 0; d < D; ++d) ring[d].fill(row_ptr((uint32_t)d), boff, n, lg);
    stream_touch_late_args(p);
    // Rows are taken 64 at a time: lane i keeps the sums of the chunk's row i; the K
    // slices are folded and the chunk stored after its last row.  The row loop is
    // the one of the Q4_K kernel.
    for (uint32_t c0 = 0; c0 < n_rows; c0 += 64u) {
        const uint32_t cnt = min(64u, n_rows - c0);
        float res[MT];
#pragma unroll
        for (int tk = 0; tk < MT; ++tk) res[tk] = 0.0f;
        for (uint32_t i0 = 0; RW * i0 < cnt; i0 += D) {
#pragma unroll
            for (int d = 0; d < D; ++d) {
                const uint32_t i = i0 + d;   // step of the chunk: row i, or (RW = 2) rows 2i and 2i + 1
                ring[d].template wait<(D - 1) * SLOT_LOADS>();
                float acc[MT];
#pragma unroll
                for (int tk = 0; tk < MT; ++tk) acc[tk] = 0.0f;
#pragma unroll
                for (int pass = 0; pass < P; ++pass)
                    q6k_piece_dot<MT>(ring[d].v[pass], x[pass], m32xs[pass], sc_shift, acc);
                ring[d].fill(row_ptr(c0 / RW + i + D), boff, n, lg);
                if constexpr (RW == 2) {
                    float v = acc[0];
                    v += group_partner<1>(v); v += group_partner<2>(v); v += group_partner<4>(v); v += group_partner<8>(v);
                    const float q0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
                    const float q1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 16));
                    const float q2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
                    const float q3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 48));
                    res[0] = lane == 2u * i ? q0 + q1 : lane == 2u * i + 1u ? q2 + q3 : res[0];   // (rows past cnt are not stored)
                } else {
#pragma unroll
                    for (int tk = 0; tk < MT; ++tk) {
                        const float tot = wave_sum(acc[tk]);
                        res[tk] = (lane == i && i < cnt) ? tot : res[tk];
                    }
                }
            }
        }
        if (KW > 1) {
#pragma unroll
            for (int tk = 0; tk < MT; ++tk) part[wave][tk][lane] = COMBINE ? slot_wt * res[tk] : res[tk];
            __syncthreads();
        }
        if (wave == 0 && lane < cnt) {
            const uint32_t r = g + (c0 + lane) * stride;
            const float bias = p.bias ? p.bias[r] : 0.0f;
#pragma unroll
            for (int tk = 0; tk < MT; ++tk) {
                float y = res[tk];
                if (KW > 1) {
                    y = part[0][tk][lane];
#pragma unroll
                    for (int w = 1; w < KW; ++w)
                        if (!COMBINE || (uint32_t)w < slots) y += part[w][tk][lane];
                }
                if (!COMBINE && MT > 2 && (uint32_t)tk >= p.M) continue;
                const size_t at = (size_t)tk * p.ldy + p.y_offset + r;
                if constexpr (PT::kFused) y *= tk == 0 ? rstd0 : rstd1;
                y += bias;
                if constexpr (PT::kFused) y += stream_residual(p) ? stream_residual(p)[at] : 0.0f;
                p.Y[at] = y;
            }
        }
        if (KW > 1) __syncthreads();
    }
    asm volatile("s_waitcnt vmcnt(0)");   // the ring's last refills land before the wave ends
}

static uint32_t cu_count() { return device_cu_count(); }

// Kernel entries.  The dense decode matvec takes its arguments as scalars (16 dwords): built with kernel-argument
// preloading (KQ_KERNARG_PRELOAD: the build adds the compiler option for this file) they arrive in scalar registers with the wave, and the kernel starts without the two dependent
// fetches of an argument struct; the fused and grouped forms keep their structs.
// (14 dwords are preloaded: everything one token needs — a pointer fetched at the stores would cost every wave a
// round trip at its end; Y arrives with the output offset added; M, read by the four-token kernels only, is the 15th)
#define KQ_DENSE_PARAMS                                                                                                   \
    const uint8_t *W, const float *X, float *Y, const float *bias, uint32_t N, uint32_t K, uint32_t n_blocks,             \
        uint32_t row_stride_bytes, uint32_t grid_x, uint32_t ldy, uint32_t M
#define KQ_DENSE_STRUCT StreamDense{X, W, bias, Y, N, K, n_blocks, row_stride_bytes, 0u, ldy, M, grid_x}
#define KQ_DENSE_ARGS(p, gx) (p).W, (p).X, (p).Y + (p).y_offset, (p).bias, (p).N, (p).K, (p).n_blocks, (p).row_stride_bytes, (gx), (p).ldy, (p).M

// The fused forms likewise: the 14 preloaded dwords are what the prologue and the first loads need.
#define KQ_FUSED_PARAMS                                                                                                   \
    const uint8_t *W, const float *X, uint32_t N, uint32_t K, uint32_t n_blocks, uint32_t row_stride_bytes,               \
        uint32_t grid_x, const float *norm_w, int pro, int epi, float eps, float *Y, uint32_t M, uint32_t y_offset,       \
        uint32_t ldy, const float *bias, const float *residual
#define KQ_FUSED_STRUCT StreamFused{X, W, bias, Y, N, K, n_blocks, row_stride_bytes, y_offset, ldy, M, pro, eps, norm_w, residual, epi, grid_x}
#define KQ_FUSED_ARGS(p, gx)                                                                                              \
    (p).W, (p).X, (p).N, (p).K, (p).n_blocks, (p).row_stride_bytes, (gx), (p).norm_w, (p).pro, (p).epi, (p).eps, (p).Y,    \
        (p).M, (p).y_offset, (p).ldy, (p).bias, (p).residual

template <int P, int NW, int D, int MT, typename PT, bool Q5 = false, int KW = 1>
__global__ __launch_bounds__(64 * NW * KW) void q4k_stream_kernel(PT p)
{
    q4k_stream_body<P, NW, D, MT, PT, Q5, KW>(p);
}
template <int P, int NW, int D, int MT, bool Q5 = false, int KW = 1>
__global__ __launch_bounds__(64 * NW * KW) void q4k_stream_fused_kernel(KQ_FUSED_PARAMS)
{
    q4k_stream_body<P, NW, D, MT, StreamFused, Q5, KW>(KQ_FUSED_STRUCT);
}
template <int P, int KW, int D, int MT>
__global__ __launch_bounds__(64 * KW) void q6k_stream_fused_kernel(KQ_FUSED_PARAMS)
{
    q6k_stream_body<P, KW, D, MT, StreamFused>(KQ_FUSED_STRUCT);
}
template <int P, int NW, int D, int MT, bool Q5 = false, int KW = 1>
__global__ __launch_bounds__(64 * NW * KW) void q4k_stream_dense_kernel(KQ_DENSE_PARAMS)
{
    q4k_stream_body<P, NW, D, MT, StreamDense, Q5, KW>(KQ_DENSE_STRUCT);
}
template <int P, int KW, int D, int MT, typename PT, int RW = 1>
__global__ __launch_bounds__(64 * KW) void q6k_stream_kernel(PT p)
{
    q6k_stream_body<P, KW, D, MT, PT, RW>(p);
}
template <int P, int KW, int D, int MT>
__global__ __launch_bounds__(64 * KW) void q6k_stream_dense_kernel(KQ_DENSE_PARAMS)
{
    q6k_stream_body<P, KW, D, MT, StreamDense>(KQ_DENSE_STRUCT);
}

// One launch of an instantiation: the scalar-argument entry for dense calls, the struct entry otherwise.
template <int P, int NW, int D, int MT, bool Q5, int KW, typename PT>
static void launch_q4k_entry(dim3 grid, dim3 block, hipStream_t s, const PT& p)
{
    // the staging area of the activations (workgroups of several walkers): 16 bytes per lane and slot
    constexpr size_t shmem = NW > 1 ? (size_t)KW * MT * P * 8 * 64 * 16 : 0;
    auto raise = [](const void* kern) {
        if (shmem > 32768) (void)hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
    };
    static bool raised = false;   // per instantiation
    if constexpr (std::is_same<PT, StreamDense>::value) {
        if (!raised) { raise((const void*)q4k_stream_dense_kernel<P, NW, D, MT, Q5, KW>); raised = true; }
        hipLaunchKernelGGL((q4k_stream_dense_kernel<P, NW, D, MT, Q5, KW>), grid, block, shmem, s, KQ_DENSE_ARGS(p, grid.x));
    } else if constexpr (std::is_same<PT, StreamFused>::value) {
        if (!raised) { raise((const void*)q4k_stream_fused_kernel<P, NW, D, MT, Q5, KW>); raised = true; }
        hipLaunchKernelGGL((q4k_stream_fused_kernel<P, NW, D, MT, Q5, KW>), grid, block, shmem, s, KQ_FUSED_ARGS(p, grid.x));
    } else {
        if (!raised) { raise((const void*)q4k_stream_kernel<P, NW, D, MT, PT, Q5, KW>); raised = true; }
        hipLaunchKernelGGL((q4k_stream_kernel<P, NW, D, MT, PT, Q5, KW>), grid, block, shmem, s, p);
    }
}
template <int P, int KW, int D, int MT, typename PT, int RW = 1>
static void launch_q6k_entry(dim3 grid, dim3 block, hipStream_t s, const PT& p)
{
    if constexpr (RW != 1)
        hipLaunchKernelGGL((q6k_stream_kernel<P, KW, D, MT, PT, RW>), grid, block, 0, s, p);
    else if constexpr (std::is_same<PT, StreamDense>::value)
        hipLaunchKernelGGL((q6k_stream_dense_kernel<P, KW, D, MT>), grid, block, 0, s, KQ_DENSE_ARGS(p, grid.x));
    else if constexpr (std::is_same<PT, StreamFused>::value)
        hipLaunchKernelGGL((q6k_stream_fused_kernel<P, KW, D, MT>), grid, block, 0, s, KQ_FUSED_ARGS(p, grid.x));
    else
        hipLaunchKernelGGL((q6k_stream_kernel<P, KW, D, MT, PT>), grid, block, 0, s, p);
}

// Workgroups for a kernel whose workgroups walk rows g, g + wgs, ...: a whole
// multiple of the CU count, so that every CU gets the same number of workgroups,
// at least two rows each so that the activations are not loaded for a single row.
static uint32_t stream_workgroups(uint32_t N, uint32_t per_cu, int rows_override)
{
    if (rows_override > 0) return (N + (uint32_t)rows_override - 1u) / (uint32_t)rows_override;
    const uint32_t want = cu_count() * per_cu;
    const uint32_t most = (N + 1u) / 2u;
    return most < want ? (most ? most : 1u) : want;
}

bool gemv_stream_supported(const MatmulArgs& a)
{
    // grouped calls: M counts (token, slot) pairs, each a matvec of its own
    if (!a.expert_idx && (a.M < 1 || a.M > 4)) return false;
    // three and four tokens: plain calls, rows of at most 56 superblocks
    if (!a.expert_idx && a.M > 2 && (a.n_blocks > 56 || a.pro != 0 || a.residual || a.epi)) return false;
    if (a.expert_idx && (a.M < 1 || a.M > 65535u || a.bias)) return false;
    if (((uintptr_t)a.X & 15u)) return false;
    if (a.n_blocks < 1) return false;
    if (a.type == KQ_TYPE_Q4_K || a.type == KQ_TYPE_Q5_K) {
        // longer rows are cut into K slices: dense and fused calls only, and the two-token kernel for
        // the longest rows has no registers for Q5_K's third load or the fused forms
        if (a.n_blocks > 16 && a.expert_idx) return false;
        if (a.n_blocks > 112) return false;
        if (a.n_blocks > 56 && a.M == 2 && (a.type == KQ_TYPE_Q5_K || a.pro != 0 || a.residual || a.epi)) return false;
        if (((uintptr_t)a.W & 15u) || (a.row_stride_bytes & 15u)) return false;
        return true;
    }
    if (a.epi && (a.type == KQ_TYPE_Q6_K || a.expert_idx || a.M > 2 || (a.N & 1u))) return false;   // pair mode: Q4_K / Q5_K
    if (a.type == KQ_TYPE_Q6_K) {
        if (a.n_blocks > 112) return false;
        // the two-token kernel for the longest rows has no registers to spare for the fused forms
        if (a.n_blocks > 56 && a.M == 2 && !a.expert_idx && (a.pro != 0 || a.residual)) return false;
        if (((uintptr_t)a.W & 1u) || (a.row_stride_bytes & 1u)) return false;
        return true;
    }
    return false;
}

// Launches of one instantiation.  Not every combination exists: grouped launches are one token per
// pair, the fused forms run two rows in flight per wave (the Q4_K kernel also four, for one token), and the
// two-token Q6_K kernel for the longest rows has no registers to spare for the fused forms
// (gemv_stream_supported declines those calls).
template <int P, int KW, int D, int MT, typename PT>
static void launch_q6k_one(dim3 grid, hipStream_t s, const PT& p)
{
    constexpr bool absent = (PT::kGrouped && MT == 2) || (PT::kFused && (D != 2 || (P == 2 && KW == 7 && MT == 2)));
    if constexpr (!absent) launch_q6k_entry<P, KW, D, MT>(grid, dim3(64 * KW), s, p);
}

// (Q5_K: at most two rows in flight, the third load per pass leaves no registers for four.)
template <int P, int NW, int D, int MT, typename PT, bool Q5>
static void launch_q4k_one(dim3 grid, hipStream_t s, const PT& p)
{
    constexpr bool absent = (PT::kGrouped && MT == 2) || (PT::kFused && (D == 1 || (D == 4 && MT == 2))) || (Q5 && D > 2);
    if constexpr (!absent) launch_q4k_entry<P, NW, D, MT, Q5, 1>(grid, dim3(64 * NW), s, p);
}

// Rows longer than 16 superblocks: K slices over KW waves, two rows in flight, dense and fused calls.
template <int P, int KW, int MT, typename PT, bool Q5>
static void launch_q4k_sliced(dim3 grid, hipStream_t s, const PT& p)
{
    constexpr bool absent = PT::kGrouped || (P == 2 && KW == 7 && MT == 2 && (PT::kFused || Q5));
    if constexpr (!absent) launch_q4k_entry<P, 1, 2, MT, Q5, KW>(grid, dim3(64 * KW), s, p);
}

// Three or four tokens (dense calls): every wave holds a K slice of eight superblocks for four tokens (128
// activations per lane), so rows of any length up to 56 superblocks are cut over 1, 2, 4 or 7 waves; two
// rows in flight.  Three tokens run as four with the last one masked.
template <typename PT>
static hipError_t launch_stream_four(const MatmulArgs& a, hipStream_t s, const PT& p)
{
    const uint32_t nb = a.n_blocks;
    const int kw = nb <= 8u ? 1 : nb <= 16u ? 2 : nb <= 32u ? 4 : 7;
    if (a.type != KQ_TYPE_Q6_K && kw <= 2) {
        // rows of up to 16 superblocks: four walkers per K slice share the slice's activations through LDS
        // (32 KB per slice; every wave loading its 128 activations per lane for itself moved 64 MB through
        // the vector caches for the 9.4 MB of a 4096 x 4096 matrix)
        const uint32_t wgs4 = stream_workgroups((a.N + 3u) / 4u, 1u, 0);
        const dim3 grid4(wgs4, 1, 1);
        const bool q5 = a.type == KQ_TYPE_Q5_K;
        if (kw == 1) {
            if (q5) launch_q4k_entry<1, 4, 2, 4, true, 1>(grid4, dim3(256), s, p);
            else launch_q4k_entry<1, 4, 2, 4, false, 1>(grid4, dim3(256), s, p);
        } else {
            if (q5) launch_q4k_entry<1, 4, 2, 4, true, 2>(grid4, dim3(512), s, p);
            else launch_q4k_entry<1, 4, 2, 4, false, 2>(grid4, dim3(512), s, p);
        }
        return hipGetLastError();
    }
    const uint32_t wgs = stream_workgroups(a.N, kw >= 7 ? 1u : 8u / (uint32_t)kw, 0);
    const dim3 grid(wgs, 1, 1);
    if (a.type == KQ_TYPE_Q6_K) {
        if (kw == 1) launch_q6k_entry<1, 1, 2, 4>(grid, dim3(64), s, p);
        else if (kw == 2) launch_q6k_entry<1, 2, 2, 4>(grid, dim3(128), s, p);
        else if (kw == 4) launch_q6k_entry<1, 4, 2, 4>(grid, dim3(256), s, p);
        else launch_q6k_entry<1, 7, 2, 4>(grid, dim3(448), s, p);
    } else if (a.type == KQ_TYPE_Q5_K) {
        if (kw == 4) launch_q4k_entry<1, 1, 2, 4, true, 4>(grid, dim3(256), s, p);
        else launch_q4k_entry<1, 1, 2, 4, true, 7>(grid, dim3(448), s, p);
    } else {
        if (kw == 4) launch_q4k_entry<1, 1, 2, 4, false, 4>(grid, dim3(256), s, p);
        else launch_q4k_entry<1, 1, 2, 4, false, 7>(grid, dim3(448), s, p);
    }
    return hipGetLastError();
}

template <typename PT>
static hipError_t launch_stream_with(const MatmulArgs& a, const GemvTuning& t, hipStream_t s, const PT& p,
                                     uint32_t pairs, uint32_t twins)
{
    const bool two = !PT::kGrouped && a.M == 2;       // two tokens share every weight load
    if constexpr (!PT::kGrouped && !PT::kFused) {
        if (a.M > 2) return launch_stream_four(a, s, p);
    }
    // Measured on MI355X: these kernels run best with about 40 KB of weight loads
    // in flight per CU: 4 to 8 waves, two to four rows in flight each.  More waves
    // or deeper rings are slower.
    if (a.type == KQ_TYPE_Q6_K) {
        // K slices of 8 or 16 superblocks, one wave each
        const uint32_t nb = a.n_blocks;
        const int kw = nb <= 16u ? 1 : nb <= 32u ? 4 : 7;
        const int pp = nb <= 8u ? 1 : nb <= 16u ? 2 : nb <= 56u ? 1 : 2;
        uint32_t wgs = stream_workgroups(a.N, kw >= 7 ? 1u : 8u / (uint32_t)kw, t.splits);
        wgs = (wgs + pairs * twins - 1u) / (pairs * twins);   // the pairs of a grouped launch share the machine
        if (PT::kGrouped) wgs *= 2u;                          // ... twice over: measured 13 % faster on a decode MoE layer
        const int depth = PT::kFused ? 2 : t.depth > 0 ? t.depth : 2;
        const dim3 grid(wgs, pairs, twins);
#define KQ_STREAM6_MT(P, KW, MT) \
    do { \
        if (depth <= 1) launch_q6k_one<P, KW, 1, MT>(grid, s, p); \
        else if (depth <= 2) launch_q6k_one<P, KW, 2, MT>(grid, s, p); \
        else launch_q6k_one<P, KW, 4, MT>(grid, s, p); \
    } while (0)
#define KQ_STREAM6(P, KW) \
    do { \
        if (two) KQ_STREAM6_MT(P, KW, 2); \
        else KQ_STREAM6_MT(P, KW, 1); \
    } while (0)
        if constexpr (PT::kGrouped) {
            if (nb <= 4u) {   // short rows (an expert's down projection): two rows per step, see q6k_stream_body
                launch_q6k_entry<1, 1, 2, 1, PT, 2>(grid, dim3(64), s, p);
                return hipGetLastError();
            }
        }
        if (kw == 1 && pp == 1) KQ_STREAM6(1, 1);
        else if (kw == 1) KQ_STREAM6(2, 1);
        else if (kw == 4) KQ_STREAM6(1, 4);
        else if (pp == 1) KQ_STREAM6(1, 7);
        else KQ_STREAM6(2, 7);
#undef KQ_STREAM6
#undef KQ_STREAM6_MT
        return hipGetLastError();
    }
    const bool q5 = a.type == KQ_TYPE_Q5_K;
    if (a.n_blocks > 16u) {
        // the Q6_K kernel's K slices: 4 waves of 8 superblocks up to 32, else 7 waves of 8 or 16
        const uint32_t nb = a.n_blocks;
        const int kw = nb <= 32u ? 4 : 7;
        const int pp = nb <= 56u ? 1 : 2;
        uint32_t wgs = stream_workgroups(a.N, kw >= 7 ? 1u : 2u, t.splits);
        const dim3 grid(wgs, 1, 1);
#define KQ_STREAM4S(P, KW) \
    do { \
        if (q5 && two) launch_q4k_sliced<P, KW, 2, PT, true>(grid, s, p); \
        else if (q5) launch_q4k_sliced<P, KW, 1, PT, true>(grid, s, p); \
        else if (two) launch_q4k_sliced<P, KW, 2, PT, false>(grid, s, p); \
        else launch_q4k_sliced<P, KW, 1, PT, false>(grid, s, p); \
    } while (0)
        if (kw == 4) KQ_STREAM4S(1, 4);
        else if (pp == 1) KQ_STREAM4S(1, 7);
        else KQ_STREAM4S(2, 7);
#undef KQ_STREAM4S
        return hipGetLastError();
    }
    constexpr int NW = 4;
    // a Q4_K workgroup is NW independent waves, each with its own rows
    uint32_t wgs = t.splits > 0 ? ((a.N + (uint32_t)t.splits - 1u) / (uint32_t)t.splits + NW - 1u) / NW
                                : stream_workgroups((a.N + NW - 1u) / NW, 1u, 0);
    wgs = (wgs + pairs * twins - 1u) / (pairs * twins);
    if (PT::kGrouped) wgs *= 2u;   // (as for Q6_K above)
    // ... and at least 512 workgroups in the launch, while a wave keeps four rows (a 128-expert layer of 768 x 2048
    // matrices: 2 tokens x 8 slots 27.7 -> 25.0 us for the layer, 8 tokens 63.6 -> 59.1, 10 tokens 97 -> 88)
    if (PT::kGrouped) wgs = max(wgs, min((512u + pairs * twins - 1u) / (pairs * twins), (a.N + 4u * NW - 1u) / (4u * NW)));
    int depth = t.depth > 0 ? t.depth : (a.N + wgs * NW - 1u) / (wgs * NW) <= 8u ? 2 : 4;
    if (q5 && depth > 2) depth = 2;
    if (PT::kFused) depth = depth >= 4 && !two ? 4 : 2;   // the fused forms come with two or four rows in flight
    const dim3 grid(wgs, pairs, twins);
#define KQ_STREAM_LAUNCH(P, D) \
    do { \
        if (q5 && two) launch_q4k_one<P, NW, D, 2, PT, true>(grid, s, p); \
        else if (q5) launch_q4k_one<P, NW, D, 1, PT, true>(grid, s, p); \
        else if (two) launch_q4k_one<P, NW, D, 2, PT, false>(grid, s, p); \
        else launch_q4k_one<P, NW, D, 1, PT, false>(grid, s, p); \
    } while (0)
    if constexpr (!PT::kGrouped) {
        // Matrices that give every wave six rows or more (gate|up: 28672 x 4096) run faster as eight waves
        // per workgroup with two rows in flight each than as four with four: 15.3 against 16.8 us there,
        // 14336 x 4096 9.1 against 9.4.  Shorter walks lose with it (8192 x 4096: 6.2 against 6.0 us,
        // 6144 x 4096: 6.1 against 5.1), so they keep the four-wave form.
        const bool eight = t.waves == 8 || (t.waves == 0 && t.depth == 0 && t.splits == 0 && a.N >= 6u * 8u * cu_count());
        if (eight && !q5 && !two && a.n_blocks > 8u) {
            const uint32_t wgs8 = stream_workgroups((a.N + 7u) / 8u, 1u, 0);
            launch_q4k_entry<2, 8, 2, 1, false, 1>(dim3(wgs8, 1, 1), dim3(512), s, p);
            return hipGetLastError();
        }
    }
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

template <typename PT>
static void stream_fill_common(PT& p, const MatmulArgs& a)
{
    p.X = (const float*)a.X;
    p.W = a.W;
    p.bias = a.bias;
    p.Y = a.Y;
    p.N = a.N; p.K = a.K;
    p.n_blocks = a.n_blocks;
    p.row_stride_bytes = a.row_stride_bytes;
    p.y_offset = a.y_offset;
    p.ldy = a.ldy;
    p.M = a.M;
}

bool stream_combine_supported(const MatmulArgs& a, uint32_t tokens)
{
    return a.type == KQ_TYPE_Q6_K && a.expert_idx && a.k_slots >= 1u && a.k_slots <= 8u && a.n_blocks <= 16u && tokens >= 1u &&
           tokens <= 65535u && a.M == tokens * a.k_slots && gemv_stream_supported(a) && !a.W2 && !a.bias;
}

// a = the grouped call of the last matvec (pairs, X per pair); out[token, r] = sum over slots of wt * result
hipError_t launch_stream_combine(const MatmulArgs& a, const float* wt, float* out, uint32_t tokens, const GemvTuning& t,
                                 hipStream_t s)
{
    StreamCombine p;
    stream_fill_common(p, a);
    p.expert_idx = a.expert_idx;
    p.k_slots = a.k_slots;
    p.x_per_slot = a.x_per_slot;
    p.W2 = nullptr;
    p.Y2 = nullptr;
    p.X2 = a.X2;
    p.wt = wt;
    p.Y = out;
    p.M = a.k_slots;
    // One workgroup per CU over all tokens (rounded down: a few workgroups more than fit at once run alone at the
    // end).  Measured on a 128-expert layer, 8 slots, 2048 x 768, with the two-rows form: one token 15.9-16.5 us
    // for the layer against 18.2 with twice and 26.8 with four times the workgroups (every workgroup loads its
    // slots' activations again: at four rows per wave they outweigh the weights), 17.1 with half; two tokens 19.2
    // against 22.2; 16 tokens 83-85 against 86, 93 at three quarters.
    uint32_t wgs = stream_workgroups(a.N, 1u, t.splits);
    if (t.splits == 0) wgs = max(1u, wgs / tokens);
    else wgs = (wgs + tokens - 1u) / tokens;
    const dim3 grid(wgs, tokens, 1);
    if (a.n_blocks <= 4u) launch_q6k_entry<1, 8, 2, 1, StreamCombine, 2>(grid, dim3(512), s, p);   // two rows per step
    else if (a.n_blocks <= 8u) launch_q6k_entry<1, 8, 2, 1>(grid, dim3(512), s, p);
    else launch_q6k_entry<2, 8, 2, 1>(grid, dim3(512), s, p);
    return hipGetLastError();
}

hipError_t launch_gemv_stream(const MatmulArgs& a, const GemvTuning& t, hipStream_t s)
{
    if (a.expert_idx) {
        StreamGrouped p;
        stream_fill_common(p, a);
        p.expert_idx = a.expert_idx;
        p.k_slots = a.k_slots;
        p.x_per_slot = a.x_per_slot;
        p.W2 = a.W2;
        p.Y2 = a.Y2;
        p.X2 = a.X2;
        return launch_stream_with(a, t, s, p, a.M, p.W2 ? 2u : 1u);   // grid.y = pairs, grid.z = twins
    }
    if (a.pro != STREAM_PRO_NONE || a.residual || a.epi) {
        StreamFused p;
        stream_fill_common(p, a);
        p.pro = a.pro;
        p.eps = a.eps;
        p.norm_w = a.norm_w;
        p.residual = a.residual;
        p.epi = a.epi;
        p.grid_x = 0;   // (the launch passes its own grid size)
        return launch_stream_with(a, t, s, p, 1u, 1u);
    }
    StreamDense p;
    stream_fill_common(p, a);
    p.grid_x = 0;
    return launch_stream_with(a, t, s, p, 1u, 1u);
}

}  // namespace kq
