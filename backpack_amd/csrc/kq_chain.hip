// kq_chain.hip — a chain of decode matvecs (M = 1) in ONE launch.
//
// The reference records a token's dispatches once and replays the list (runtime/model_runner.cpp:5725-5759);
// between two attention blocks that list is nothing but k-quant matvecs and the small elementwise
// dispatches around them: o (+ residual), ffn norm -> gate|up -> act * up, down (+ residual), attn norm ->
// q|k|v of the next layer (runtime/model_runner.cpp:3324-3330, :3711-3793, :3206-3243).  Launched one by
// one, each of them pays several memory round trips in which no weight byte moves: the launch, the first
// waves' wait for x, the first fill of the weight ring, the last waves finishing alone.  A grid-wide
// barrier between ops inside one kernel costs as much (measured: 5 us each through an arrival counter:
// store acknowledgement, atomic, poll, load of x are four round trips of more than a microsecond).
// So this kernel has no barrier between ops.  One persistent grid (a workgroup of eight waves per compute
// unit) walks a device-side list of matvec descriptors, and
//
//  * the weights never stop moving: when a wave has requested the last row of op i it requests its first
//    rows of op i + 1 (weights do not depend on x) with loads whose destination is LDS, so nothing in
//    registers is in flight across the op boundary and the data is a few LDS reads away by the time x is;
//  * x travels with its own flags: every output is also stored, written through to memory, into a
//    "mailbox" copy whose lowest mantissa bit carries the parity of the run.  An op that reads what an
//    earlier op of the launch wrote loads the mailbox until every element shows the run's parity:
//    the load of x IS the wait, one store and one load instead of four round trips.  (The consumer
//    sees x with the lowest mantissa bit cleared, 2^-24 relative; the caller's Y is exact.)
//
// Every wait is bounded: a thread that has polled longer than the limit writes an error word and its
// workgroup leaves; every workgroup checks the word when it polls and when a launch starts, so the grid
// always drains; the host reads the word (bpk_chain_status).
//
// The per-lane arithmetic, the ring loads and their hand-placed waits are those of kq_stream.hip.
#include "kq_format.h"
#include "kq_kernels.h"
#include "kq_wave.h"
#include "kq_stream_core.h"   // hand-waited loads: KQ_REQUIRES_NO_SPILL (the build refuses this file if a kernel spills)

namespace kq {

namespace {

constexpr int CW = CHAIN_WAVES;                 // waves per workgroup
constexpr uint32_t CHAIN_THREADS = 64u * CW;
constexpr int CD = 2;                           // rows in flight per wave: 8 waves x 2 rows is the 30-40 KB per
                                                // compute unit at which these loops run best
static_assert(CD == 2, "the wait counts at an op boundary are written out for two slots");

__device__ __forceinline__ float ld_agent(const float* p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t ld_agent(const uint32_t* p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_agent(float* p, float v)
{
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float2 ld_agent2(const float* p)
{
    const uint64_t u = __hip_atomic_load((const uint64_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    float2 r;
    r.x = __builtin_bit_cast(float, (uint32_t)u);
    r.y = __builtin_bit_cast(float, (uint32_t)(u >> 32));
    return r;
}
__device__ __forceinline__ float tag(float v, uint32_t par)
{
    return __builtin_bit_cast(float, (__builtin_bit_cast(uint32_t, v) & ~1u) | par);
}
__device__ __forceinline__ bool tagged(float v, uint32_t par) { return (__builtin_bit_cast(uint32_t, v) & 1u) == par; }

// What a polling thread needs to give up in bounded time.
struct Patience {
    uint32_t* error;
    uint64_t ticks;
    uint32_t op;
};

// One failed poll: has the wait lasted too long, or has somebody else given up?  t0 == 0: first failure.
// Most failed polls return at once (the next poll is the wait): the clock and the error word, a memory
// round trip of its own, are looked at on every eighth.
__device__ __forceinline__ bool give_up(const Patience& pt, uint64_t& t0, uint32_t& tries)
{
    if ((++tries & 7u) != 0u) return false;
    if (ld_agent(pt.error) != 0u) return true;
    const uint64_t now = wall_clock64();
    if (t0 == 0) { t0 = now | 1u; return false; }
    if (now - t0 > pt.ticks) {
        __hip_atomic_store(pt.error, CHAIN_ERR_TIMEOUT | (pt.op << 8), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return true;
    }
    return false;
}

// Sum over the workgroup; every thread gets it.  red: CW floats of LDS.
__device__ __forceinline__ float block_sum(float v, float* red, uint32_t wave, uint32_t lane)
{
    v = wave_sum(v);
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = red[0];
#pragma unroll
    for (int w = 1; w < CW; ++w) t += red[w];
    __syncthreads();
    return t;
}

// A thread's share of the op's input: XB pairs of activations (pair tid + 512 u), 64-bit loads that are all
// in flight together: one memory round trip, not one per pair.  No branch around a load (with one the
// compiler waits for each load before it issues the next): a pair past the end re-reads the last one and is
// zeroed afterwards.  From the caller's buffer, or from the mailbox of the op of this launch that writes
// them: then the loads are repeated until every pair carries the run's parity.
template <int XB>
__device__ __forceinline__ void chain_x_load(float2 (&v)[XB], const float* plain, const float* mail, bool from_chain, uint32_t par,
                                             uint32_t half, const Patience& pt, int& bad)
{
    const uint32_t tid = threadIdx.x;
    uint32_t at[XB];
#pragma unroll
    for (int u = 0; u < XB; ++u) at[u] = 2u * min(tid + u * CHAIN_THREADS, half - 1u);
    if (!mail) {
#pragma unroll
        for (int u = 0; u < XB; ++u) v[u] = *(const float2*)(plain + at[u]);
    } else {
        uint64_t t0 = 0;
        uint32_t tries = 0;
        // While the producers are still at work, a workgroup polls a sample (one pair per thread, 4 KB instead
        // of the whole x): every compute unit reading all of x from memory again and again takes the
        // bandwidth the producers' last rows need.  Once the sample is there nearly everything is.
        for (;;) {
            const float2 probe = ld_agent2(mail + at[0]);
            if (tagged(probe.x, par) && tagged(probe.y, par)) break;
            if (give_up(pt, t0, tries)) { bad = 1; break; }
        }
        uint32_t pending = bad ? 0u : 1u;
        while (pending) {
            // (all of them again: the ones that had arrived are still there, and no load waits for another)
#pragma unroll
            for (int u = 0; u < XB; ++u) v[u] = ld_agent2(mail + at[u]);
            pending = 0;
#pragma unroll
            for (int u = 0; u < XB; ++u)
                if (!(tagged(v[u].x, par) && tagged(v[u].y, par))) pending |= 1u << u;
            if (pending && give_up(pt, t0, tries)) { bad = 1; break; }
        }
    }
#pragma unroll
    for (int u = 0; u < XB; ++u) {
        if (tid + u * CHAIN_THREADS >= half) v[u] = float2{0.0f, 0.0f};
        // the flag bit is cleared whatever the run's parity (the same x from run to run), also where the
        // values come from an op of the chain in an earlier launch (the same x wherever a chain is cut)
        else if (from_chain) { v[u].x = tag(v[u].x, 0u); v[u].y = tag(v[u].y, 0u); }
    }
}

// x of the op -> xs[0..K), prologue applied (runtime/kernels/norm/rms_norm.wgsl:15-20,
// fused/silu_mul_fused.wgsl:39-49, fused/gelu_mul_fused.wgsl:22-32), for K <= 1024 XB.  Returns false (for
// the whole workgroup) when a wait was given up.  Ends with a barrier.
template <int XB>
__device__ __forceinline__ bool chain_stage_x_n(const ChainOp& p, const float* mail, uint32_t par, const Patience& pt, float* xs,
                                                float* red, volatile uint32_t* gave_up, uint32_t wave, uint32_t lane)
{
    const uint32_t tid = threadIdx.x;
    const uint32_t half = p.K >> 1;   // K is a multiple of 256
    const bool fc = p.x_src != CHAIN_NO_SRC;
    int bad = 0;
    float2 v[XB];
    chain_x_load<XB>(v, p.X, mail, fc, par, half, pt, bad);
    if (p.pro == STREAM_PRO_SILU || p.pro == STREAM_PRO_GELU) {
        float2 up[XB];
        chain_x_load<XB>(up, p.X + p.K, mail ? mail + p.K : nullptr, fc, par, half, pt, bad);
#pragma unroll
        for (int u = 0; u < XB; ++u) {
            if (p.pro == STREAM_PRO_SILU) {
                v[u].x = stream_act<STREAM_PRO_SILU, true>(v[u].x, up[u].x);
                v[u].y = stream_act<STREAM_PRO_SILU, true>(v[u].y, up[u].y);
            } else {
                v[u].x = stream_act<STREAM_PRO_GELU, true>(v[u].x, up[u].x);
                v[u].y = stream_act<STREAM_PRO_GELU, true>(v[u].y, up[u].y);
            }
        }
    } else if (p.pro == STREAM_PRO_NORM) {
        // the norm's weights travel while the sum of squares is formed
        float2 nw[XB];
#pragma unroll
        for (int u = 0; u < XB; ++u) nw[u] = *(const float2*)(p.norm_w + 2u * min(tid + u * CHAIN_THREADS, half - 1u));
        float ss = 0.0f;
#pragma unroll
        for (int u = 0; u < XB; ++u) ss = __builtin_fmaf(v[u].x, v[u].x, __builtin_fmaf(v[u].y, v[u].y, ss));   // (pairs past the end are zero)
        const float tot = block_sum(ss, red, wave, lane);
        const float rstd = 1.0f / sqrtf(tot / (float)p.K + p.eps);
#pragma unroll
        for (int u = 0; u < XB; ++u) {
            v[u].x = v[u].x * rstd * nw[u].x;
            v[u].y = v[u].y * rstd * nw[u].y;
        }
    }
#pragma unroll
    for (int u = 0; u < XB; ++u) {
        const uint32_t i = tid + u * CHAIN_THREADS;
        if (i < half) *(float2*)(xs + 2u * i) = v[u];
    }
    if (bad) *gave_up = 1u;
    __syncthreads();
    return *gave_up == 0u;
}

// (three sizes, so that a short x is not loaded as a long one's worth of repeated pairs)
__device__ __forceinline__ bool chain_stage_x(const ChainOp& p, const float* mail, uint32_t par, const Patience& pt, float* xs,
                                              float* red, volatile uint32_t* gave_up, uint32_t wave, uint32_t lane)
{
    if (p.K <= 4096u) return chain_stage_x_n<4>(p, mail, par, pt, xs, red, gave_up, wave, lane);
    if (p.K <= 9216u) return chain_stage_x_n<9>(p, mail, par, pt, xs, red, gave_up, wave, lane);
    static_assert(18u * 2u * CHAIN_THREADS >= CHAIN_MAX_K, "the widest staging form must cover the longest row a chain accepts");
    return chain_stage_x_n<18>(p, mail, par, pt, xs, red, gave_up, wave, lane);
}

// Which rows of an op a wave walks.
struct Geo {
    uint32_t gw, stride;      // rows gw, gw + stride, ... (pairs of rows with an epilogue)
    uint32_t n_rows;          // rows this wave takes (twice the pairs)
    uint32_t n_walk_all;      // rows (pairs) of the op
    bool pairs;               // the wave alternates between a pair's gate row and its up row, n_walk_all further on
    bool active;              // the wave has rows, and its K slice lies inside them
    __device__ __forceinline__ size_t row_of(uint32_t i) const
    {
        i = min(i, n_rows - 1u);
        if (pairs) return (size_t)(gw + (i >> 1) * stride) + (size_t)(i & 1u) * n_walk_all;
        return (size_t)(gw + i * stride);
    }
};

__device__ __forceinline__ Geo chain_geo(const ChainOp& p, uint32_t wg, uint32_t G, uint32_t wave)
{
    Geo g;
    const bool sliced = (p.mode & CHAIN_MODE_SLICED) != 0u;
    const uint32_t pp = (p.mode & CHAIN_MODE_P2) ? 2u : 1u;
    g.gw = sliced ? wg : wg * CW + wave;
    g.stride = sliced ? G : G * CW;
    g.pairs = p.epi != 0u;
    g.n_walk_all = g.pairs ? p.N / 2u : p.N;
    const uint32_t n_walk = g.gw < g.n_walk_all ? (g.n_walk_all - g.gw + g.stride - 1u) / g.stride : 0u;
    g.n_rows = g.pairs ? 2u * n_walk : n_walk;
    g.active = g.n_rows > 0u && (!sliced || wave * 8u * pp < p.n_blocks);
    return g;
}

// Byte offsets, inside a row, of the superblock(s) a lane reads: pass s covers superblocks 8 s .. 8 s + 7 of
// the row (rows mode) or of the wave's K slice (sliced mode); lanes past the row's end re-read its last
// superblock against activations that are zero.
__device__ __forceinline__ void chain_offsets(const ChainOp& p, uint32_t wave, uint32_t lane, uint32_t (&off)[2], bool (&valid)[2],
                                              uint32_t (&blk)[2])
{
    const bool sliced = (p.mode & CHAIN_MODE_SLICED) != 0u;
    const uint32_t pp = (p.mode & CHAIN_MODE_P2) ? 2u : 1u;
    const uint32_t bytes = (p.mode & CHAIN_MODE_Q6) ? KQ_Q6K_BYTES : KQ_Q4K_BYTES;
#pragma unroll
    for (uint32_t s = 0; s < 2u; ++s) {
        uint32_t b = ((sliced ? wave * pp : 0u) + s) * 8u + (lane >> 3);
        valid[s] = b < p.n_blocks;
        b = valid[s] ? b : p.n_blocks - 1u;
        blk[s] = b;
        off[s] = b * bytes;
    }
}

// ---- the first CD rows of an op, through LDS -----------------------------------------------------------
// No register may be waiting for a load where the compiler is free to move registers about, and between two
// ops (a switch over the bodies, waits, the staging of x) it is: an earlier form of this kernel that handed
// the register ring from op to op computed wrong rows now and then, because the ring's registers were copied
// while their loads were in flight.  So the rows a wave needs first are requested with loads that write LDS
// (global_load_lds: lane l's bytes land at base + size * l; the compiler tracks them like any load) into a
// stage private to the wave: CD slots of cells, one cell per load of the slot.  Q4_K, per pass: the header and
// the lane's quant piece, 16 bytes per lane each.  Q6_K, per pass: nine cells of 4 bytes per lane (the two
// halves of ql, ql + 32, qh and the scales, then d).  They are requested when the op BEFORE has requested
// its last row, or, for the first op of a launch, when the launch starts.
typedef __attribute__((address_space(1))) const void* chain_gptr;
typedef __attribute__((address_space(3))) void* chain_lptr;
constexpr uint32_t CHAIN_CELL16 = 1024u, CHAIN_CELL4 = 256u;
constexpr uint32_t CHAIN_SLOT_STAGE = 2u * 9u * CHAIN_CELL4;   // two passes of Q6_K; two passes of Q4_K take 4 KB
constexpr uint32_t CHAIN_WAVE_STAGE = CD * CHAIN_SLOT_STAGE + CHAIN_CELL4;   // + a cell nobody reads, for the touches

__device__ __forceinline__ void lds_load16(const uint8_t* src, uint8_t* cell)
{
    __builtin_amdgcn_global_load_lds((chain_gptr)src, (chain_lptr)cell, 16, 0, 0);
}
__device__ __forceinline__ void lds_load4(const uint8_t* src, uint8_t* cell)
{
    __builtin_amdgcn_global_load_lds((chain_gptr)src, (chain_lptr)cell, 4, 0, 0);
}

// Requests rows 0 .. CD-1 of this wave's share of op p into the wave's stage, and touches the `ahead` rows
// behind them (4 bytes per lane into the spare cell): those lines are in this XCD's L2 when the ring's first
// refills ask for them.
__device__ __forceinline__ void chain_request_first_rows(const ChainOp& p, const Geo& g, uint8_t* stage, uint32_t wave, uint32_t lane,
                                                         uint32_t ahead)
{
    if (!g.active) return;
    uint32_t off[2], blk[2];
    bool valid[2];
    chain_offsets(p, wave, lane, off, valid, blk);
    const uint32_t t = lane & 7u, n = t >> 2, lg = t & 3u;
    const uint32_t passes = (p.mode & CHAIN_MODE_P2) ? 2u : 1u;
#pragma unroll
    for (int d = 0; d < CD; ++d) {
        const uint8_t* row = p.W + g.row_of((uint32_t)d) * p.row_stride_bytes;
        uint8_t* cell = stage + d * CHAIN_SLOT_STAGE;
        for (uint32_t pass = 0; pass < passes; ++pass) {
            const uint8_t* b = row + off[pass];
            if (p.mode & CHAIN_MODE_Q6) {
                uint8_t* c = cell + pass * 9u * CHAIN_CELL4;
                lds_load4(b + 64u * n + 8u * lg, c);
                lds_load4(b + 64u * n + 8u * lg + 4u, c + CHAIN_CELL4);
                lds_load4(b + 64u * n + 32u + 8u * lg, c + 2u * CHAIN_CELL4);
                lds_load4(b + 64u * n + 32u + 8u * lg + 4u, c + 3u * CHAIN_CELL4);
                lds_load4(b + 128u + 32u * n + 8u * lg, c + 4u * CHAIN_CELL4);
                lds_load4(b + 128u + 32u * n + 8u * lg + 4u, c + 5u * CHAIN_CELL4);
                lds_load4(b + 192u + 8u * n, c + 6u * CHAIN_CELL4);
                lds_load4(b + 192u + 8u * n + 4u, c + 7u * CHAIN_CELL4);
                lds_load4(b + 206u, c + 8u * CHAIN_CELL4);   // d in the upper half (the word ends with the block)
            } else {
                uint8_t* c = cell + pass * 2u * CHAIN_CELL16;
                lds_load16(b, c);
                lds_load16(b + 16u + 16u * t, c + CHAIN_CELL16);
            }
        }
    }
    uint8_t* dump = stage + CD * CHAIN_SLOT_STAGE;
    for (uint32_t k = 0; k < ahead; ++k) {
        if (CD + k >= g.n_rows) break;
        const uint8_t* row = p.W + g.row_of(CD + k) * p.row_stride_bytes;
        for (uint32_t pass = 0; pass < passes; ++pass) {
            if (p.mode & CHAIN_MODE_Q6) {
                lds_load4(row + off[pass] + 64u * n + 8u * lg, dump);            // ql: bytes 0 .. 127 of the block
                lds_load4(row + off[pass] + 128u + 32u * n + 8u * lg, dump);     // qh, and the scales behind it
            } else {
                lds_load4(row + off[pass] + 16u + 16u * t, dump);
            }
        }
    }
}

template <int P>
__device__ __forceinline__ void chain_take_first_rows(Q4Slot<P, false> (&ring)[CD], const uint8_t* stage, uint32_t lane)
{
#pragma unroll
    for (int d = 0; d < CD; ++d)
#pragma unroll
        for (int pass = 0; pass < P; ++pass) {
            const uint8_t* c = stage + d * CHAIN_SLOT_STAGE + pass * 2u * CHAIN_CELL16;
            ring[d].hdr[pass] = *(const s_u32x4*)(c + 16u * lane);
            ring[d].q[pass] = *(const s_u32x4*)(c + CHAIN_CELL16 + 16u * lane);
        }
}
template <int P>
__device__ __forceinline__ void chain_take_first_rows(Q6Slot<P> (&ring)[CD], const uint8_t* stage, uint32_t lane)
{
#pragma unroll
    for (int d = 0; d < CD; ++d)
#pragma unroll
        for (int pass = 0; pass < P; ++pass) {
            const uint32_t* c = (const uint32_t*)(stage + d * CHAIN_SLOT_STAGE + pass * 9u * CHAIN_CELL4) + lane;
            Q6Piece& v = ring[d].v[pass];
            v.a = s_u32x2{c[0], c[64]};
            v.b = s_u32x2{c[128], c[192]};
            v.h = s_u32x2{c[256], c[320]};
            v.sc = s_u32x2{c[384], c[448]};
            v.d = c[512] >> 16;
        }
}

// What a body needs besides its own op.
struct Ctx {
    const float* res_mail;    // mailbox the residual comes from, or nullptr (the caller's buffer)
    uint32_t res_par;
    float* y_mail;            // mailbox this op's outputs are copied to
    uint32_t y_par;
    Patience pt;
    float* xs;
    float (*part)[64];
    uint8_t* stage;           // the wave's LDS stage, holding its first CD rows of this op
    uint32_t wave, lane;
};

// Output n of the op: residual, the caller's Y, the mailbox.
__device__ __forceinline__ void chain_out(const ChainOp& p, const Ctx& c, uint32_t n, float y, bool with_residual, int& bad)
{
    const size_t at = (size_t)p.y_offset + n;
    if (with_residual && p.residual) {
        float r;
        if (c.res_mail) {
            uint64_t t0 = 0;
            uint32_t tries = 0;
            r = ld_agent(c.res_mail + n);
            while (!tagged(r, c.res_par)) {
                if (give_up(c.pt, t0, tries)) { bad = 1; break; }
                r = ld_agent(c.res_mail + n);
            }
            r = tag(r, 0u);
        } else {
            r = p.residual[at];
            if (p.res_src != CHAIN_NO_SRC) r = tag(r, 0u);   // (as through the mailbox)
        }
        y += r;
    }
    p.Y[at] = y;
    if (c.y_mail) st_agent(c.y_mail + n, tag(y, c.y_par));
}

// ---------------------------------------------------------------------------------------------------
// Q4_K.  SLICED == false: a wave owns whole rows (n_blocks <= 8 P); the waves of the grid walk rows gw,
// gw + stride, ...  SLICED == true: the CW waves of a workgroup each hold a K slice of 8 P superblocks of the
// workgroup's rows wg, wg + G, ... and their sums meet in LDS once per 64 rows.  On entry the wave's stage
// holds (or is about to receive) its first CD rows.  The row loop is the one of q4k_stream_kernel: no
// branch around a refill (past the end the last row is fetched again and dropped), so that every wait finds
// the same number of younger loads; the ring lives in this function only.
// ---------------------------------------------------------------------------------------------------
template <int P, bool SLICED>
__device__ __forceinline__ void chain_q4(const ChainOp& p, const Geo& g, const Ctx& c, int& bad)
{
    const uint32_t lane = c.lane, wave = c.wave;
    const uint32_t j = lane & 7u, gq = j >> 1, h = j & 1u;
    const bool sel_hi = gq >= 2u;
    const uint32_t sh = 16u * (gq & 1u);
    constexpr int S = 2 * P;   // loads per slot
    if (g.n_rows == 0u) return;   // SLICED: the whole workgroup

    float xlo[P][1][16], xhi[P][1][16], xs_lo[P][1], xs_hi[P][1];
    uint32_t off2[2], blk[2];
    bool valid[2];
    chain_offsets(p, wave, lane, off2, valid, blk);
    uint32_t off[P];
#pragma unroll
    for (int pass = 0; pass < P; ++pass) off[pass] = off2[pass];
    Q4Slot<P, false> ring[CD] = {};
    if (g.active) {
#pragma unroll
        for (int pass = 0; pass < P; ++pass) {
            const float4* xp = (const float4*)(c.xs + (size_t)blk[pass] * KQ_QK + 64u * gq + 16u * h);
            float sl = 0.0f, sh_ = 0.0f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float4 lo = xp[i], hi = xp[8 + i];
                if (!valid[pass]) { lo = float4{0, 0, 0, 0}; hi = lo; }
                xlo[pass][0][4 * i + 0] = lo.x; xlo[pass][0][4 * i + 1] = lo.y; xlo[pass][0][4 * i + 2] = lo.z; xlo[pass][0][4 * i + 3] = lo.w;
                xhi[pass][0][4 * i + 0] = hi.x; xhi[pass][0][4 * i + 1] = hi.y; xhi[pass][0][4 * i + 2] = hi.z; xhi[pass][0][4 * i + 3] = hi.w;
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) { sl += xlo[pass][0][i]; sh_ += xhi[pass][0][i]; }
            xs_lo[pass][0] = sl;
            xs_hi[pass][0] = sh_;
        }
        chain_take_first_rows<P>(ring, c.stage, lane);
    }
    for (uint32_t c0 = 0; c0 < g.n_rows; c0 += 64u) {
        const uint32_t cnt = min(64u, g.n_rows - c0);
        float res = 0.0f;
        if (g.active) {
            for (uint32_t i0 = 0; i0 < cnt; i0 += CD) {
#pragma unroll
                for (int d = 0; d < CD; ++d) {
                    const uint32_t i = i0 + d;
                    ring[d].template wait<(CD - 1) * S>();   // (the staged rows of the first pass are there already)
                    float acc[1] = {0.0f};
#pragma unroll
                    for (int pass = 0; pass < P; ++pass)
                        q4k_piece_dot<1, false>(ring[d].hdr[pass], ring[d].q[pass], xlo[pass], xhi[pass], xs_lo[pass], xs_hi[pass],
                                                sel_hi, sh, acc);
                    ring[d].fill(p.W + g.row_of(c0 + i + CD) * p.row_stride_bytes, off, j);
                    const float tot = wave_sum(acc[0]);
                    res = (lane == i && i < cnt) ? tot : res;
                }
            }
        }
        if (SLICED) {
            c.part[wave][lane] = res;
            __syncthreads();
        }
        if ((!SLICED || wave == 0) && lane < cnt) {
            const uint32_t r = (uint32_t)g.row_of(c0 + lane);
            float y = res;
            if (SLICED) {
                y = c.part[0][lane];
#pragma unroll
                for (int w = 1; w < CW; ++w) y += c.part[w][lane];
            }
            y += p.bias ? p.bias[r] : 0.0f;
            if (g.pairs) {
                // lanes 2j and 2j + 1 hold a pair's gate and up products (cnt is even): the even lane stores
                const float up = group_partner<1>(y);
                y = p.epi == STREAM_PRO_SILU ? stream_act<STREAM_PRO_SILU, true>(y, up)
                                             : stream_act<STREAM_PRO_GELU, true>(y, up);
                if (!(lane & 1u)) chain_out(p, c, r, y, false, bad);
            } else {
                chain_out(p, c, r, y, true, bad);
            }
        }
        if (SLICED) __syncthreads();
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the ring's last refills have landed
}

// ---------------------------------------------------------------------------------------------------
// Q6_K, the same forms; lane (b, t) takes 8 positions of one half block (see kq_stream.hip).
// ---------------------------------------------------------------------------------------------------
template <int P, bool SLICED>
__device__ __forceinline__ void chain_q6(const ChainOp& p, const Geo& g, const Ctx& c, int& bad)
{
    const uint32_t lane = c.lane, wave = c.wave;
    const uint32_t t = lane & 7u, n = t >> 2, lg = t & 3u;
    const uint32_t sc_shift = 8u * (lg >> 1);
    constexpr int S = 5 * P;
    if (g.n_rows == 0u) return;   // SLICED: the whole workgroup

    float x[P][1][4][8], m32xs[P][1][4];
    uint32_t off2[2], blk[2];
    bool valid[2];
    chain_offsets(p, wave, lane, off2, valid, blk);
    uint32_t off[P];
#pragma unroll
    for (int pass = 0; pass < P; ++pass) off[pass] = off2[pass];
    Q6Slot<P> ring[CD] = {};
    if (g.active) {
#pragma unroll
        for (int pass = 0; pass < P; ++pass) {
            const float4* xp = (const float4*)(c.xs + (size_t)blk[pass] * KQ_QK + 128u * n + 8u * lg);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                float4 lo = xp[8 * k], hi = xp[8 * k + 1];
                if (!valid[pass]) { lo = float4{0, 0, 0, 0}; hi = lo; }
                x[pass][0][k][0] = lo.x; x[pass][0][k][1] = lo.y; x[pass][0][k][2] = lo.z; x[pass][0][k][3] = lo.w;
                x[pass][0][k][4] = hi.x; x[pass][0][k][5] = hi.y; x[pass][0][k][6] = hi.z; x[pass][0][k][7] = hi.w;
                float sum = 0.0f;
#pragma unroll
                for (int i = 0; i < 8; ++i) sum += x[pass][0][k][i];
                m32xs[pass][0][k] = -32.0f * sum;
            }
        }
        chain_take_first_rows<P>(ring, c.stage, lane);
    }
    for (uint32_t c0 = 0; c0 < g.n_rows; c0 += 64u) {
        const uint32_t cnt = min(64u, g.n_rows - c0);
        float res = 0.0f;
        if (g.active) {
            for (uint32_t i0 = 0; i0 < cnt; i0 += CD) {
#pragma unroll
                for (int d = 0; d < CD; ++d) {
                    const uint32_t i = i0 + d;
                    ring[d].template wait<(CD - 1) * S>();
                    float acc[1] = {0.0f};
#pragma unroll
                    for (int pass = 0; pass < P; ++pass)
                        q6k_piece_dot<1>(ring[d].v[pass], x[pass], m32xs[pass], sc_shift, acc);
                    ring[d].fill(p.W + g.row_of(c0 + i + CD) * p.row_stride_bytes, off, n, lg);
                    const float tot = wave_sum(acc[0]);
                    res = (lane == i && i < cnt) ? tot : res;
                }
            }
        }
        if (SLICED) {
            c.part[wave][lane] = res;
            __syncthreads();
        }
        if ((!SLICED || wave == 0) && lane < cnt) {
            const uint32_t r = (uint32_t)g.row_of(c0 + lane);
            float y = res;
            if (SLICED) {
                y = c.part[0][lane];
#pragma unroll
                for (int w = 1; w < CW; ++w) y += c.part[w][lane];
            }
            y += p.bias ? p.bias[r] : 0.0f;
            chain_out(p, c, r, y, true, bad);
        }
        if (SLICED) __syncthreads();
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// Diagnostics: thread 0 of every workgroup leaves the wall clock at a few points of every op.
__device__ __forceinline__ void chain_stamp(uint64_t* trace, uint32_t count, uint32_t op, uint32_t point)
{
    if (trace && threadIdx.x == 0) trace[((size_t)blockIdx.x * count + op) * CHAIN_TRACE_POINTS + point] = wall_clock64();
}

// A descriptor out of the launch's LDS copy, as wave-uniform values.
constexpr uint32_t CHAIN_OP_WORDS = sizeof(ChainOp) / 4u;
static_assert(sizeof(ChainOp) % 4u == 0, "descriptors are copied word by word");
__device__ __forceinline__ ChainOp chain_op_at(const uint32_t* lds_ops, uint32_t i)
{
    uint32_t w[CHAIN_OP_WORDS];
#pragma unroll
    for (uint32_t k = 0; k < CHAIN_OP_WORDS; ++k)
        w[k] = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_ops[i * CHAIN_OP_WORDS + k]);
    ChainOp op;
    __builtin_memcpy(&op, w, sizeof op);
    return op;
}

}  // namespace

__global__ __launch_bounds__(CHAIN_THREADS) void chain_kernel(ChainLaunch a)
{
    extern __shared__ __align__(16) uint8_t smem[];
    float* xs = (float*)smem;
    float (*part)[64] = (float (*)[64])(xs + a.max_k);
    float* red = (float*)(part + CW);
    volatile uint32_t* flags = (volatile uint32_t*)(red + CW);   // [0]: a wait ran out; [1]: the chain's error word at the start
    uint32_t* lds_par = (uint32_t*)(red + CW + 8);               // parity of the launch's ops
    uint32_t* lds_ops = lds_par + CHAIN_MAX_PER_LAUNCH;          // their descriptors
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    uint8_t* stage = (uint8_t*)(lds_ops + CHAIN_MAX_PER_LAUNCH * CHAIN_OP_WORDS) + wave * CHAIN_WAVE_STAGE;
    const uint32_t wg = blockIdx.x, G = gridDim.x;

    chain_stamp(a.trace, a.count, 0, 3);
    // Everything the launch needs to know, in one round trip: descriptors, parities, the error word.
    {
        const uint32_t* src = (const uint32_t*)(a.ops + a.first);
        for (uint32_t k = threadIdx.x; k < a.count * CHAIN_OP_WORDS; k += CHAIN_THREADS) lds_ops[k] = src[k];
        for (uint32_t k = threadIdx.x; k < a.count; k += CHAIN_THREADS) lds_par[k] = a.parity[a.first + k];
        if (threadIdx.x == 0) {
            flags[0] = 0u;
            flags[1] = ld_agent(a.error);
        }
        __syncthreads();
        // a launch after one that gave up does nothing (until the host resets the chain)
        if (flags[1] != 0u) return;
    }

    int bad = 0;
    ChainOp p = chain_op_at(lds_ops, 0);
    Geo g = chain_geo(p, wg, G, wave);
    chain_request_first_rows(p, g, stage, wave, lane, a.ahead);
    for (uint32_t i = 0; i < a.count; ++i) {
        const uint32_t at = a.first + i;
        Ctx c;
        c.pt = Patience{a.error, a.spin_ticks, at};
        // inputs written by earlier ops of this launch come from those ops' mailboxes
        const bool x_here = p.x_src != CHAIN_NO_SRC && p.x_src >= a.first;
        const bool r_here = p.res_src != CHAIN_NO_SRC && p.res_src >= a.first;
        const uint32_t x_par = x_here ? lds_par[p.x_src - a.first] : 0u;
        c.res_mail = r_here ? p.res_mail : nullptr;
        c.res_par = r_here ? lds_par[p.res_src - a.first] : 0u;
        c.y_mail = a.hold ? nullptr : p.y_mail;   // (testing: nothing is handed on, every wait runs out)
        c.y_par = lds_par[i];
        c.xs = xs;
        c.part = part;
        c.stage = stage;
        c.wave = wave;
        // (the lane id through an opaque statement, per op: what a body derives from it is recomputed there
        // instead of being held in registers across the other bodies)
        uint32_t lane_i = lane;
        asm volatile("" : "+v"(lane_i));
        c.lane = lane_i;
        chain_stamp(a.trace, a.count, i, 0);
        if (!chain_stage_x(p, x_here ? p.x_mail : nullptr, x_par, c.pt, xs, red, flags, wave, lane)) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // no load may outlive the wave
            return;
        }
        chain_stamp(a.trace, a.count, i, 1);
        switch (p.mode) {
        case 0: chain_q4<1, false>(p, g, c, bad); break;
        case CHAIN_MODE_P2: chain_q4<2, false>(p, g, c, bad); break;
        case CHAIN_MODE_SLICED: chain_q4<1, true>(p, g, c, bad); break;
        case CHAIN_MODE_SLICED | CHAIN_MODE_P2: chain_q4<2, true>(p, g, c, bad); break;
        case CHAIN_MODE_Q6: chain_q6<1, false>(p, g, c, bad); break;
        case CHAIN_MODE_Q6 | CHAIN_MODE_P2: chain_q6<2, false>(p, g, c, bad); break;
        case CHAIN_MODE_Q6 | CHAIN_MODE_SLICED: chain_q6<1, true>(p, g, c, bad); break;
        default: chain_q6<2, true>(p, g, c, bad); break;
        }
        chain_stamp(a.trace, a.count, i, 2);
        if (i + 1u < a.count) {
            // the next op's first rows start moving before anybody waits for its x
            p = chain_op_at(lds_ops, i + 1u);
            g = chain_geo(p, wg, G, wave);
            chain_request_first_rows(p, g, stage, wave, lane_i, a.ahead);
        }
    }
    // (a lane that gave up waiting for a residual has set the error word; the launch still ends normally)
    __syncthreads();
    chain_stamp(a.trace, a.count, 0, 4);
    if (threadIdx.x == 0)
        flags[1] = __hip_atomic_fetch_add(a.arrivals, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    // the last workgroup to finish flips the parity of the mailboxes this launch has filled (nobody polls
    // them any more), a thread per op, and re-arms the counter
    if (flags[1] == G - 1u) {
        if (threadIdx.x < a.count) a.parity[a.first + threadIdx.x] = lds_par[threadIdx.x] ^ 1u;
        if (threadIdx.x == 0) __hip_atomic_store(a.arrivals, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// ---- host side -------------------------------------------------------------------------------------

int chain_mode_for(int type, uint32_t n_blocks, int epi)
{
    if (n_blocks == 0 || n_blocks > 16u * CW || n_blocks * KQ_QK > CHAIN_MAX_K) return -1;
    if (type != KQ_TYPE_Q4_K && type != KQ_TYPE_Q6_K) return -1;
    // rows of up to 16 superblocks are held whole by a wave, longer ones as K slices of 8 or 16 per wave
    uint32_t mode = type == KQ_TYPE_Q6_K ? CHAIN_MODE_Q6 : 0u;
    if (n_blocks > 16u) mode |= CHAIN_MODE_SLICED;
    // the act(gate) * up epilogue pairs the rows of a wave: Q4_K rows that a wave holds whole
    if (epi && mode != 0u && mode != CHAIN_MODE_P2) return -1;
    if (n_blocks > ((mode & CHAIN_MODE_SLICED) ? 8u * CW : 8u)) mode |= CHAIN_MODE_P2;
    return (int)mode;
}

// (the kernel also has a few hundred bytes of static LDS: the dynamic part stays 4 KB under the unit's 160 KB)
size_t chain_lds_bytes(uint32_t max_k)
{
    return ((size_t)max_k + 64u * CW + CW + 8u + CHAIN_MAX_PER_LAUNCH * (1u + sizeof(ChainOp) / 4u)) * sizeof(float) +
           (size_t)CW * CHAIN_WAVE_STAGE;
}

hipError_t launch_chain(const ChainLaunch& a, uint32_t workgroups, hipStream_t s)
{
    // A workgroup takes more than half of a compute unit's LDS, so the dispatcher puts one on each unit
    // and all of them run at once (an op's wait for the ops before it relies on the workgroups that
    // produce them being resident; the waits are bounded anyway).
    size_t shmem = chain_lds_bytes(a.max_k);
    if (shmem < (size_t)84 << 10) shmem = (size_t)84 << 10;
    static bool raised[64];
    int dev = 0;
    (void)hipGetDevice(&dev);
    if (dev >= 0 && dev < 64 && !raised[dev]) {
        const hipError_t e = hipFuncSetAttribute((const void*)chain_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)CHAIN_MAX_LDS);
        if (e != hipSuccess) return e;
        raised[dev] = true;
    }
    hipLaunchKernelGGL(chain_kernel, dim3(workgroups), dim3(CHAIN_THREADS), shmem, s, a);
    return hipGetLastError();
}

}  // namespace kq
