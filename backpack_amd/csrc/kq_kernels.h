// kq_kernels.h — launch entry points of the HIP kernels (internal to the library).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace kq {

struct MatmulArgs {
    int type;               // KQ_TYPE_*
    const void* X;          // f32 [M,K] or bf16 [M,K]
    const uint8_t* W;       // packed rows
    const float* bias;      // [N] or nullptr
    float* Y;               // f32
    uint32_t M, N, K;
    uint32_t n_blocks;
    uint32_t row_stride_bytes;
    uint32_t y_offset;
    uint32_t ldy;           // elements between consecutive rows of Y
    // expert indirection (nullptr for the dense case): pair p uses weight rows
    // expert_idx[p]*N .. +N-1 and X row p / k_slots (x_per_slot == 0) or p.
    const uint32_t* expert_idx;
    uint32_t k_slots;
    int x_per_slot;
    // fusions of the MoE FFN, honoured by the grouped lanes-along-K launch (and W2 by the grouped tile launch,
    // which then stores silu(W x) * (W2 x) to Y): a twin matrix W2 of the
    // same shape whose products go to Y2 (gate and up in one launch), and X2: x = silu(X) * X2
    const uint8_t* W2;
    float* Y2;
    const float* X2;
    uint32_t tile_iters;   // grouped tile launch of one chunk of K: tiles a wave walks with X staged once (0: chosen by the launcher)
    // fused forms of the dense decode matvec, honoured by the lanes-along-K launch only (other launches
    // must be given pro == 0 and residual == nullptr): pro 1 = RMSNorm of the X row with weight norm_w,
    // 2 / 3 = X rows are gate | up (2K floats) and x = silu / gelu_tanh (gate) * up; residual is added to
    // every output (indexed like Y, may alias it)
    int pro = 0;
    const float* norm_w = nullptr;
    float eps = 0.0f;
    const float* residual = nullptr;
    // 2 / 3: W is gate | up stacked (N rows, N/2 outputs), Y[n] = silu / gelu_tanh (gate_n . x) * (up_n . x);
    // Y rows are ldy apart
    int epi = 0;
};

// Per-device scratch for split-K partial sums and arrival counters.
struct SplitScratch {
    float* partial;        // capacity_floats floats
    uint32_t* counters;    // n_counters words, zero between launches
    size_t capacity_floats;
    uint32_t n_counters;
};

hipError_t launch_dequant_rows(int type, const uint8_t* W, uint32_t row_stride_bytes,
                               const int32_t* rows, uint32_t M, uint32_t K, float* out,
                               hipStream_t s);

// Stand-alone RMSNorm (pro 1) / silu-mul (2) / gelu-mul (3) of M rows into out [M,K], and
// Y[m, y_offset + n] = T[m, n] + R[m, y_offset + n].
hipError_t launch_prologue_rows(int pro, const float* X, const float* norm_w, float eps, uint32_t M, uint32_t K,
                                float* out, hipStream_t s);
// The same prologues with bf16 rows as their output (pro 0: plain conversion): X of the prefill GEMM.
hipError_t launch_prologue_rows_bf16(int pro, const float* X, const float* norm_w, float eps, uint32_t M, uint32_t K,
                                     uint16_t* out, hipStream_t s);
hipError_t launch_add_residual(const float* T, const float* R, float* Y, uint32_t M, uint32_t N, uint32_t ldy,
                               uint32_t y_offset, hipStream_t s);

// MoE router stage: per token the k largest of n_experts logits (iterated argmax, lowest index on ties)
// and the softmax over them; and the same behind an fp32 router matvec.  n_experts <= 1024, k <= 16.
hipError_t launch_topk_softmax(const float* logits, uint32_t T, uint32_t n_experts, uint32_t k, int normalize,
                               uint32_t* idx, float* wt, hipStream_t s);
constexpr uint32_t ROUTE_SPREAD_TOKENS = 64;   // fewer tokens: experts spread over workgroups, two launches
constexpr uint32_t ROUTE_SCRATCH_FLOATS = 1u << 20;   // the library's own place for router logits (4 MB)
hipError_t launch_route(const float* X, const float* router_w, uint32_t T, uint32_t hidden, uint32_t n_experts,
                        uint32_t k, int normalize, float* logits_out, float* logits_scratch, uint32_t* idx, float* wt,
                        hipStream_t s);

// Index (and value) of the largest element of each of M rows of N floats, rows ld apart; one launch per
// ARGMAX_MAX_ROWS rows.  Scratch: ARGMAX_MAX_ROWS * ARGMAX_PARTS partial values and indices, and
// ARGMAX_MAX_ROWS tickets that are zero between launches.
constexpr uint32_t ARGMAX_PARTS = 64, ARGMAX_MAX_ROWS = 256;
hipError_t launch_argmax_rows(const float* logits, uint32_t M, uint32_t N, uint32_t ld, int32_t* out_idx,
                              float* out_val, float* part_val, uint32_t* part_idx, uint32_t* tickets, hipStream_t s);
// Device address, on the current device, of a scratch of ARGMAX_STATIC_WORDS words in that layout which
// lives in the library's code object (no allocation): looked up once per device at set-up.
constexpr size_t ARGMAX_STATIC_WORDS = (size_t)ARGMAX_MAX_ROWS * (2u * ARGMAX_PARTS + 1u);
hipError_t argmax_static_scratch(uint32_t** out);

// Any shape with K % 256 == 0, any 4-byte aligned W.  M tiled by 4 inside.
hipError_t launch_matmul_generic(const MatmulArgs& a, hipStream_t s);

// Row-per-lane decode GEMV (M <= 4): Q4_K and Q6_K with 16-byte aligned rows.
struct GemvTuning {
    int splits = 0;   // workgroups along K, 0 = automatic
    int waves = 0;    // waves per workgroup (2, 4 or 8), 0 = automatic
    int depth = 0;    // superblocks a wave keeps in flight (1, 2 or 4), 0 = automatic
};
bool gemv_rows_supported(const MatmulArgs& a);
size_t gemv_rows_scratch_floats(const MatmulArgs& a, const GemvTuning& t);
// The greedy pick folded into a matvec launch: every workgroup leaves the best (value, index) of the outputs it
// stored, per token, in part_val / part_idx[token * groups + group]; the last one to take the ticket reduces them
// into out_idx / out_val (lowest index among equal maxima, index 0 when nothing exceeds -1e30) and re-arms
// the ticket.  cells: capacity of the partial arrays.
struct ArgmaxFold {
    int32_t* out_idx;
    float* out_val;       // may be null
    float* part_val;
    uint32_t* part_idx;
    uint32_t* ticket;     // zero between launches
    uint32_t cells;
};
bool gemv_rows_can_fold(const MatmulArgs& a, const ArgmaxFold& f);
hipError_t launch_gemv_rows(const MatmulArgs& a, const SplitScratch& sc, const GemvTuning& t,
                            hipStream_t s, const ArgmaxFold* fold = nullptr);

// Lanes-along-K decode GEMV (M = 1): a wave owns whole rows, activations stay
// in registers.  t.splits, when set, overrides the rows per wave.
bool gemv_stream_supported(const MatmulArgs& a);
hipError_t launch_gemv_stream(const MatmulArgs& a, const GemvTuning& t, hipStream_t s);
// The grouped call `a` (Q6_K, up to 8 slots per token) with the weighted sum over each token's slots folded into
// the launch: out[token, r] = sum over slots, in slot order, of wt[pair] * (W[expert_idx[pair]] x[pair])[r].
bool stream_combine_supported(const MatmulArgs& a, uint32_t tokens);
hipError_t launch_stream_combine(const MatmulArgs& a, const float* wt, float* out, uint32_t tokens, const GemvTuning& t,
                                 hipStream_t s);

// One token on the matrix cores: Q4_K rows of up to 16 superblocks, 16-byte aligned (kq_mgemv.hip).
bool mgemv_supported(const MatmulArgs& a);
// form 1: sixteen waves of one superblock each (four waves per SIMD); otherwise eight waves of two
hipError_t launch_mgemv(const MatmulArgs& a, uint32_t cus, int form, hipStream_t s);

// 16-row x 16-token MFMA tiles for M = 2..16 (dense): weights read once for all tokens.
bool mtile_supported(const MatmulArgs& a);
hipError_t launch_mtile(const MatmulArgs& a, const SplitScratch& sc, hipStream_t s);
// grouped by expert: records {expert, count, pair ids...} of up to cap pairs, as launch_moe_group
// writes them with sets = cap / 2; cap at most mtile_group_cap(type)
uint32_t mtile_group_cap(int type);
// the fused forms (MatmulArgs pro / residual / epi) on the tile kernel, up to 16 tokens, one launch
bool mtile_fused_supported(const MatmulArgs& a);
hipError_t launch_mtile_fused(const MatmulArgs& a, const SplitScratch& sc, hipStream_t s);
bool mtile_grouped_dual_supported(const MatmulArgs& a);   // a.W2 honoured: Y = silu(W x) * (W2 x)
hipError_t launch_mtile_grouped(const MatmulArgs& a, const uint32_t* tiles, const uint32_t* n_tiles,
                                uint32_t tiles_bound, uint32_t cap, hipStream_t s);

// Row-per-lane matvec on the matrix cores, M <= 16 dense or grouped by expert.
bool mrow_supported(const MatmulArgs& a);
size_t mrow_scratch_floats(const MatmulArgs& a, const GemvTuning& t);
hipError_t launch_mrow(const MatmulArgs& a, const SplitScratch& sc, const GemvTuning& t, const uint32_t* tiles,
                       const uint32_t* n_tiles, uint32_t tiles_bound, int sets, hipStream_t s);

// MoE: bucket (token, slot) pairs by expert into tiles of 2*sets pairs, the
// activation between gate/up and down, and the weighted combine.
int moe_sets_for(uint32_t n_pairs, uint32_t n_experts);
uint32_t moe_tiles_bound(uint32_t n_pairs, uint32_t n_experts, int sets);
size_t moe_tiles_words(uint32_t n_pairs, uint32_t n_experts, int sets);
hipError_t launch_moe_group(const uint32_t* expert_idx, uint32_t n_pairs, uint32_t n_experts, int sets, uint32_t* tiles,
                            uint32_t* n_tiles, hipStream_t s);
double moe_expected_records(uint32_t n_pairs, uint32_t n_experts, uint32_t cap);
hipError_t launch_moe_silu_mul(const float* gate, const float* up, float* act, size_t n, hipStream_t s);
hipError_t launch_moe_combine(const float* down, const float* wt, float* out, uint32_t T, uint32_t k, uint32_t hidden,
                              hipStream_t s);

// Prefill GEMM on the matrix cores: X bf16 [M,K], Y f32.  tile = 0 (automatic),
// 128 or 256 (square workgroup tile); split (256-tile only) = 0 (automatic),
// 1 (one tile per workgroup) or 2 (the walk cut into equal shares per CU).
bool gemm_bf16_supported(const MatmulArgs& a);
hipError_t launch_gemm_bf16(const MatmulArgs& a, int tile, int split, const SplitScratch& gemm_scratch, hipStream_t s);

// A chain of decode matvecs (M = 1) in one launch: a persistent grid walks ops[first .. first + count).
struct ChainOp {                 // device-resident, written once when the chain is created
    const uint8_t* W;            // packed rows
    const float* X;              // f32 [K]; [2K] (gate | up) for the act prologues
    const float* bias;           // [N] or nullptr
    float* Y;
    const float* norm_w;         // [K], pro == 1
    const float* residual;       // indexed like Y, or nullptr
    // Mailboxes (owned by the chain): a copy of an op's outputs, written through to memory, whose lowest
    // mantissa bit carries the parity of the run.  y_mail: this op's; x_mail / res_mail: where, in the mailbox
    // of op x_src / res_src, this op's X row / its residual elements start (used when that op belongs to
    // the same launch; otherwise X / residual are read from the caller's buffers).
    float* y_mail;
    const float* x_mail;
    const float* res_mail;
    uint32_t x_src, res_src;     // op indices, or CHAIN_NO_SRC
    uint32_t N;                  // rows of W (twice the outputs with an epilogue)
    uint32_t K, n_blocks, row_stride_bytes, y_offset;
    uint32_t pro, epi;           // as MatmulArgs
    float eps;
    uint32_t mode;               // CHAIN_MODE_* bits, from chain_mode_for
};
constexpr uint32_t CHAIN_NO_SRC = 0xFFFFFFFFu;
constexpr uint32_t CHAIN_MODE_P2 = 1u;     // two passes of eight superblocks per wave (else one)
constexpr uint32_t CHAIN_MODE_SLICED = 2u; // the waves of a workgroup share rows, a K slice each (else a wave per row)
constexpr uint32_t CHAIN_MODE_Q6 = 4u;     // Q6_K (else Q4_K)
constexpr int CHAIN_WAVES = 8;
constexpr uint32_t CHAIN_MAX_OPS = 1024;
constexpr uint32_t CHAIN_TRACE_POINTS = 8;
constexpr uint32_t CHAIN_MAX_PER_LAUNCH = 64;   // ops one launch walks (their descriptors sit in LDS)
constexpr size_t CHAIN_MAX_LDS = (size_t)156 << 10;   // dynamic LDS a chain launch may ask for
// longest X row a chain op may have: what the widest staging form (18 pairs per thread of 512) covers, and what
// fits the dynamic LDS beside the descriptors and the waves' staging windows
constexpr uint32_t CHAIN_MAX_K = 18432;
constexpr uint32_t CHAIN_ERR_TIMEOUT = 1u; // low byte of the error word; the op index sits above it
struct ChainLaunch {
    const ChainOp* ops;
    uint32_t* parity;            // per op: the bit this run's mailbox entries carry (flipped when a launch ends)
    uint32_t* arrivals;          // workgroups that have finished the launch; zero between launches
    uint32_t* error;             // 0, or CHAIN_ERR_* | op << 8 once a thread gave up waiting
    uint32_t first, count;
    uint32_t max_k;              // floats of x the LDS holds
    uint32_t hold;               // testing: 1 keeps the ops from filling their mailboxes, so every wait runs out
    uint32_t ahead;              // rows per wave touched into L2 behind the staged first rows of the next op
    uint64_t spin_ticks;         // bound of a wait, in ticks of the 100 MHz wall clock
    uint64_t* trace;             // diagnostics: [workgroup][op][CHAIN_TRACE_POINTS] wall-clock stamps, or nullptr
};
// CHAIN_MODE_* bits for a matrix, or -1 where the chain kernel has no form for it.
int chain_mode_for(int type, uint32_t n_blocks, int epi);
size_t chain_lds_bytes(uint32_t max_k);
hipError_t launch_chain(const ChainLaunch& a, uint32_t workgroups, hipStream_t s);

// Compute units of the current device (cached per device id).
inline uint32_t device_cu_count()
{
    static int cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256u;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev] = n;
    }
    return (uint32_t)cached[dev];
}

}  // namespace kq
