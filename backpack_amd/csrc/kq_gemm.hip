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
// The 256 x 256 tile runs 8 waves (2 x 4, 128 x 64 each), two per SIMD, in two
// phases: waves 0..3 issue the global loads of step t+1, run the MFMAs of step
// t and then dequantise step t+1; waves 4..7 first dequantise step t+1 from
// registers loaded a step earlier, issue the loads of step t+2, then run the
// MFMAs of step t.  On every SIMD one wave's conversion arithmetic therefore
// overlaps the other wave's matrix work.  The 128 x 128 tile runs 4 waves
// (2 x 2) and fits twice on a CU, which gives the same overlap between
// workgroups.
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

namespace kq {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int GEMM_BK = 64;
constexpr int GEMM_LD = GEMM_BK * 2 + 16;   // bytes per LDS row

struct GemmParams {
    const uint16_t* X;   // bf16 [M,K]
    const uint8_t* W;
    const float* bias;
    float* Y;
    uint32_t M, N, K, n_blocks, row_stride_bytes, ldy;
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
    constexpr bool PHASED = NWAVES == 8;  // second half of the waves converts before it multiplies
    uint8_t* As = smem;
    uint8_t* Bs = smem + 2 * A_BYTES;

    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t wm = wave / WAVES_N, wn = wave % WAVES_N;
    const uint32_t m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const uint32_t nk = p.K / GEMM_BK;
    const bool convert_first = PHASED && wave >= NWAVES / 2;   // wave-uniform

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
    uint32_t w4[WI][12];
    Q6Raw w6[WI];

    auto load_tile = [&](uint32_t kt) {
#pragma unroll
        for (int i = 0; i < XP; ++i) xr[i] = *(const u32x4*)(xsrc[i] + (size_t)kt * (GEMM_BK * 2));
#pragma unroll
        for (int i = 0; i < WI; ++i) {
            if (TYPE == KQ_TYPE_Q4_K) q4k_load(wsrc[i], kt, w4[i]);
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
            if (TYPE == KQ_TYPE_Q4_K) q4k_expand(w4[i], kt, whf[i], dst);
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
    if (convert_first && nk > 1) load_tile(1);
    __syncthreads();

    for (uint32_t kt = 0; kt < nk; ++kt) {
        const uint32_t buf = kt & 1u;
        if (convert_first) {
            if (kt + 1 < nk) store_tile(kt + 1, buf ^ 1u);
            if (kt + 2 < nk) load_tile(kt + 2);
        } else {
            if (kt + 1 < nk) load_tile(kt + 1);
        }
        multiply(buf);
        if (!convert_first && kt + 1 < nk) store_tile(kt + 1, buf ^ 1u);
        __syncthreads();
    }

    // accumulator register r of lane l: token row 8*(r/4) + 4*(l/32) + r%4, weight row l%32
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const uint32_t n = n0 + wn * WN + j * 32u + (lane & 31u);
        if (n >= p.N) continue;
        const float bias = p.bias ? p.bias[n] : 0.0f;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t m = m0 + wm * WM + i * 32u + 8u * (r >> 2) + 4u * (lane >> 5) + (r & 3u);
                if (m < p.M) p.Y[(size_t)m * p.ldy + n] = acc[i][j][r] + bias;
            }
        }
    }
}

bool gemm_bf16_supported(const MatmulArgs& a)
{
    if (a.expert_idx) return false;
    if (a.type != KQ_TYPE_Q4_K && a.type != KQ_TYPE_Q6_K) return false;
    if ((uintptr_t)a.X & 15u) return false;            // 128-bit loads of bf16 rows (K % 256 == 0 already)
    if (a.type == KQ_TYPE_Q4_K && (((uintptr_t)a.W & 15u) || (a.row_stride_bytes & 15u))) return false;
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

hipError_t launch_gemm_bf16(const MatmulArgs& a, int tile, hipStream_t s)
{
    GemmParams p;
    p.X = (const uint16_t*)a.X;
    p.W = a.W;
    p.bias = a.bias;
    p.Y = a.Y;
    p.M = a.M; p.N = a.N; p.K = a.K;
    p.n_blocks = a.n_blocks;
    p.row_stride_bytes = a.row_stride_bytes;
    p.ldy = a.ldy;
    // big tiles when they still give every CU work, else 128 x 128
    const uint64_t big = (uint64_t)((a.M + 255u) / 256u) * ((a.N + 255u) / 256u);
    const bool use_big = tile == 256 || (tile == 0 && big >= 256u);
    const bool q4 = a.type == KQ_TYPE_Q4_K;
    if (use_big) return q4 ? launch_gemm<KQ_TYPE_Q4_K, 256, 256, 8>(p, s) : launch_gemm<KQ_TYPE_Q6_K, 256, 256, 8>(p, s);
    return q4 ? launch_gemm<KQ_TYPE_Q4_K, 128, 128, 4>(p, s) : launch_gemm<KQ_TYPE_Q6_K, 128, 128, 4>(p, s);
}

}  // namespace kq
