/*
 * bpk_kquant.h — C ABI of the MI355X (gfx950) k-quant dequant-matmul library.
 *
 * Plain pointers and sizes only.  Device pointers are ordinary HIP device
 * addresses; a caller that holds a buffer + byte offset view (the reference's
 * GPUBuffer{handle,size,offset}, runtime/gpu_context.h:47-51) passes
 * base + offset.  `stream` is a hipStream_t passed as void* (NULL = the null
 * stream).  Every launch is asynchronous on that stream and in order with the
 * other work on it; the library never synchronises the device.
 *
 * Every function returns BPK_OK (0) or a negative BPK_ERR_* code, and stores a
 * human-readable message retrievable with bpk_last_error() (thread-local).
 * The reference's ops return void and print to stderr on failure
 * (runtime/ops/matmul.cpp:211-212, runtime/model_runner.cpp:154-157); a host
 * wrapper that wants that behaviour prints bpk_last_error() and returns.
 *
 * One host thread per stream, as in the reference (runtime/model_runner.h:27-30).
 */
#ifndef BPK_KQUANT_H
#define BPK_KQUANT_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#if defined(__GNUC__)
#define BPK_API __attribute__((visibility("default")))
#else
#define BPK_API
#endif

/* GGUF tensor type codes (runtime/gguf_loader.h:29-30). */
#define BPK_TYPE_Q4_K 12
#define BPK_TYPE_Q5_K 13
#define BPK_TYPE_Q6_K 14

enum {
    BPK_OK = 0,
    BPK_ERR_TYPE = -1,      /* not a type this entry point serves            */
    BPK_ERR_SHAPE = -2,     /* K not a multiple of 256, zero sizes, overflow  */
    BPK_ERR_NULL = -3,      /* required pointer is NULL                       */
    BPK_ERR_ALIGN = -4,     /* pointer or stride alignment not met            */
    BPK_ERR_HIP = -5,       /* a HIP runtime call failed                      */
    BPK_ERR_DEVICE = -6,    /* the current device is not gfx950               */
    BPK_ERR_WORKSPACE = -7, /* workspace missing or too small                 */
    BPK_ERR_IO = -8,        /* a file could not be opened or mapped           */
    BPK_ERR_FORMAT = -9,    /* not a GGUF file, or truncated / inconsistent   */
    BPK_ERR_NOT_FOUND = -10,/* no tensor / metadata element of that name      */
    BPK_ERR_TIMEOUT = -11   /* a chain launch gave up a wait between its ops  */
};

/* Library version, major*10000 + minor*100 + patch. */
BPK_API int bpk_version(void);

/* Message of the last failing call on this thread ("" when none). */
BPK_API const char *bpk_last_error(void);

/* Checks that `device` is a gfx950 part and creates the library's per-device
 * state (split-K scratch, counters).  Optional: the first launch on a device
 * does the same — but it allocates, so call it before capturing a HIP graph
 * on that device.  Replaces GPUContext device bring-up for this path
 * (runtime/gpu_context.h:86-145). */
BPK_API int bpk_init(int device);

/* Frees the per-device state of every device.  Outstanding work must have
 * completed. */
BPK_API int bpk_shutdown(void);

/* ---- layout: replaces the descriptor half of pack_q4k / pack_q6k ----------
 * runtime/gguf_loader.cpp:359-379, :403-424; struct KQuantPacked
 * (runtime/gguf_loader.h:108-113).  n_blocks = ceil(K/256);
 * row_stride_words = 36*n_blocks (Q4_K), 44*n_blocks (Q5_K, pack_q5k,
 * gguf_loader.cpp:381-401) or ceil(210*n_blocks/4) (Q6_K). */
BPK_API int bpk_kq_layout(int type, uint32_t K, uint32_t *n_blocks,
                          uint32_t *row_stride_words);

/* Host-side packer: N rows of raw GGUF blocks -> N*row_stride_words words,
 * pad bytes zero.  Replaces the copy half of pack_q4k / pack_q6k. */
BPK_API int bpk_kq_pack_host(int type, const void *raw, uint32_t N, uint32_t K,
                             uint32_t *out_words);

/* ---- weights: replaces uploadKQWeight / fuseKQ ------------------------------
 * runtime/model_runner.cpp:958-963 (createBuffer + writeBuffer of the packed
 * words) and :1002-1012 (row-wise concatenation of matrices with equal K).
 * The handle owns one device allocation that lives until destroy. */
typedef struct bpk_weight bpk_weight;

typedef struct bpk_weight_desc {
    int type;                  /* BPK_TYPE_*                     */
    uint32_t N, K;             /* rows (outputs), columns        */
    uint32_t n_blocks;         /* superblocks per row            */
    uint32_t row_stride_words; /* words per packed row           */
    void *data;                /* device address of row 0        */
    size_t bytes;              /* N*row_stride_words*4, the packed rows; the allocation
                                  holds 16 readable zero bytes more (see bpk_kq_matmul) */
} bpk_weight_desc;

/* parts[i] points at raw GGUF bytes (host) of an n_rows[i] x K matrix; the
 * parts are stacked in order (n_parts = 1 for a plain upload).  Synchronous:
 * the host buffers may be released on return. */
BPK_API int bpk_weight_create(int type, uint32_t K, uint32_t n_parts,
                              const void *const *parts, const uint32_t *n_rows,
                              bpk_weight **out);
BPK_API int bpk_weight_describe(const bpk_weight *w, bpk_weight_desc *out);
BPK_API int bpk_weight_destroy(bpk_weight *w);

/* ---- GGUF container: replaces GGUFFile for this path ----------------------
 * runtime/gguf_loader.h:49-86 (GGUFFile, its getters) and
 * runtime/gguf_loader.cpp:90-182 (open: magic "GGUF", version, tensor and
 * key-value counts, typed key-value pairs, tensor table, data section at the
 * next aligned offset).  The file is memory-mapped read-only and every length
 * and offset in it is checked against the file size.  Versions 2 and 3.
 * `general.alignment` is honoured when present (default 32, the constant of
 * gguf_loader.cpp:151).  Pointers returned (names, data) stay valid until
 * bpk_gguf_close. */
typedef struct bpk_gguf bpk_gguf;

typedef struct bpk_gguf_tensor {
    const char *name;   /* NUL-terminated                                   */
    uint32_t type;      /* GGUF tensor type code (runtime/gguf_loader.h:23-36) */
    uint32_t n_dims;    /* 0..4                                             */
    uint64_t dims[4];   /* dims[0] = row length (K); unused entries are 1   */
    uint64_t offset;    /* from the start of the data section               */
    uint64_t bytes;     /* size of the data; 0 when the type is not known here */
    const void *data;   /* host address inside the mapping                  */
} bpk_gguf_tensor;

BPK_API int bpk_gguf_open(const char *path, bpk_gguf **out);
BPK_API int bpk_gguf_close(bpk_gguf *g);
/* Any of the out pointers may be NULL. */
BPK_API int bpk_gguf_info(const bpk_gguf *g, uint32_t *version,
                          uint64_t *n_tensors, uint64_t *n_kv,
                          uint64_t *data_offset);
/* Tensors in file order / by name (GGUFFile::tensors, ::tensor_index). */
BPK_API int bpk_gguf_tensor_at(const bpk_gguf *g, uint64_t index,
                               bpk_gguf_tensor *out);
BPK_API int bpk_gguf_find_tensor(const bpk_gguf *g, const char *name,
                                 bpk_gguf_tensor *out);

/* Metadata getters with the reference's defaults-and-coercions behaviour
 * (runtime/gguf_loader.cpp:155-182): a missing key or a value of another kind
 * yields `def`, never an error.  get_u32 accepts integers of any width and, for
 * an int32/uint32 array, returns its largest element (gguf_loader.cpp:158-166).
 * get_f32 accepts f32 and f64.  has_key returns 1 or 0. */
BPK_API int bpk_gguf_has_key(const bpk_gguf *g, const char *key);
/* GGUF metadata value type code of the key (0 u8 .. 8 string, 9 array, 10 u64,
 * 11 i64, 12 f64), or -1 when absent. */
BPK_API int bpk_gguf_key_type(const bpk_gguf *g, const char *key);
BPK_API int bpk_gguf_get_u32(const bpk_gguf *g, const char *key, uint32_t def,
                             uint32_t *out);
BPK_API int bpk_gguf_get_f32(const bpk_gguf *g, const char *key, float def,
                             float *out);
BPK_API int bpk_gguf_get_bool(const bpk_gguf *g, const char *key, int def,
                              int *out);
/* Copies at most cap-1 bytes into buf and terminates it; *len (may be NULL)
 * receives the full length, 0 when the key is absent or not a string. */
BPK_API int bpk_gguf_get_string(const bpk_gguf *g, const char *key, char *buf,
                                size_t cap, size_t *len);
/* Arrays (GGUFFile::getStringArray etc., runtime/gguf_loader.h:73-85): element
 * count and element type code (0 when absent), one string element, and the
 * address of the packed elements of a fixed-size-element array. */
BPK_API int bpk_gguf_array_len(const bpk_gguf *g, const char *key, uint64_t *n,
                               uint32_t *elem_type);
BPK_API int bpk_gguf_array_string(const bpk_gguf *g, const char *key,
                                  uint64_t index, char *buf, size_t cap,
                                  size_t *len);
BPK_API int bpk_gguf_array_data(const bpk_gguf *g, const char *key,
                                const void **data, uint64_t *n,
                                uint32_t *elem_type);

/* Model hyper-parameters (extractModelConfig, runtime/gguf_loader.cpp:184-317;
 * ModelConfig, runtime/gguf_loader.h:164-218): the reference's keys under
 * "<general.architecture>.", its defaults, and its probes of the tensor
 * directory (vocabulary from token_embd.weight, QK norm, sandwich norm, MTP).
 * layer_types (may be NULL) receives n_layer_attn_types entries, 0 = global
 * attention, 1 = sliding window (Gemma 2 / 3 / 4 patterns); cap is its size. */
enum { BPK_ACT_SILU = 0, BPK_ACT_GELU = 1 };
typedef struct bpk_model_config {
    char arch[64];
    uint32_t n_layer, n_head, n_kv_heads, n_embd, intermediate_size, n_vocab;
    uint32_t head_dim, kv_head_dim;
    float rms_norm_eps, rope_theta;
    int tie_word_embeddings, has_qk_norm;
    int activation;                 /* BPK_ACT_*                                */
    float embedding_scale;          /* sqrt(n_embd) for the Gemma family, else 0 */
    float logit_softcap;
    uint32_t sliding_window;
    uint32_t n_layer_attn_types;    /* n_layer when sliding_window > 0, else 0  */
    int has_sandwich_norm;
    uint32_t ple_size, shared_kv_layers;
    int has_mtp;
    uint32_t mtp_num_layers;
    uint32_t num_experts, num_experts_per_tok, moe_intermediate_size,
        moe_shared_intermediate_size;
    uint32_t ssm_inner_size, ssm_state_size, ssm_conv_kernel, ssm_group_count,
        ssm_time_step_rank, full_attention_interval;
    int32_t rope_sections[4];       /* default 11, 11, 10, 0                    */
} bpk_model_config;
BPK_API int bpk_gguf_model_config(const bpk_gguf *g, bpk_model_config *out,
                                  uint8_t *layer_types,
                                  uint32_t layer_types_cap);

/* Named Q4_K / Q6_K matrices of the file (GGUF shape {K, N}) -> one device
 * weight with the rows stacked in the order given: the tensor -> packKQ ->
 * fuseKQ -> uploadKQWeight sequence of runtime/model_runner.cpp:1275-1338
 * (q|k|v and gate|up are stacked that way there).  All parts must share type
 * and K; another tensor type fails with BPK_ERR_TYPE. */
BPK_API int bpk_gguf_weight_create(const bpk_gguf *g, const char *const *names,
                                   uint32_t n_names, bpk_weight **out);

/* ---- matmul: replaces the q4k_matmul* / q6k_matmul* dispatches -------------
 * Bindings 0:X 1:W 2:Bias 3:Y 4:P of runtime/kernels/quant_kq/q4k_matmul.wgsl:20-95,
 * q4k_matmul_128.wgsl:8-17, q4k_matmul_batched4/8.wgsl, q6k_matmul.wgsl:25-114,
 * q6k_matmul_batched4.wgsl, q6k_matmul_wide.wgsl, with
 * P = {K, N, nBlocks, rowStrideWords, yOffset} (runtime/model_runner.cpp:2404-2413)
 * or {K, N, M, nBlocks, rowStrideWords} (:5843-5844).  One entry point serves
 * every M; the kernel choice the reference makes in kqPipelineFor / mmk
 * (runtime/model_runner.cpp:2043-2054, :5841-5845) happens inside.
 *
 *   Y[m*N + y_offset + n] = bias[n] + sum_k X[m*K + k] * dequant(W)[n, k]
 *
 * X: f32 [M,K] (device).  W: packed rows (device, 4-byte aligned; 16-byte
 * aligned rows take the fast kernels).  Q6_K blocks are 210 bytes and are
 * fetched in 16-byte pieces: the buffer must stay readable for 16 bytes past
 * the end of the last row (bpk_weight_create allocates them).  bias: f32 [N] or NULL (= zeros).
 * Y: f32, caller-owned, not cleared.  fp32 accumulation throughout.  Up to 16
 * tokens (8 on Q6_K matrices) every weight byte is read once per call; more
 * tokens run in groups of that size, each reading the weights again (prefill
 * chunks belong on bpk_prefill_rows_bf16 + bpk_kq_matmul_bf16). */
BPK_API int bpk_kq_matmul(int type, const float *X, const void *W,
                          const float *bias, float *Y, uint32_t M, uint32_t N,
                          uint32_t K, uint32_t n_blocks,
                          uint32_t row_stride_words, uint32_t y_offset,
                          void *stream);

/* ---- fused decode forms: replace the dispatches either side of the matvec ----
 * What the reference wrote as q4k_matmul_norm / q6k_matmul_norm
 * (runtime/kernels/quant_kq/q4k_matmul_norm.wgsl:50-91: RMSNorm of the X row
 * inside the matvec, bindings 5:NormW 6:{K,0,0,eps}) and q4k_down_gelu /
 * q6k_down_gelu (quant_kq/q4k_down_gelu.wgsl:11-56: binding 0 is the fused
 * gate|up buffer), and the dispatches it still issues separately: rms_norm
 * (kernels/norm/rms_norm.wgsl:15-20), silu_mul_fused / gelu_mul_fused
 * (kernels/fused/silu_mul_fused.wgsl:39-49, gelu_mul_fused.wgsl:22-32) before
 * down, add_inplace after it (runtime/model_runner.cpp:3748-3793).
 *
 *   x[m,k] = X[m,k]                                              BPK_PRO_NONE
 *          = X[m,k] * rsqrt(mean_k(X[m,:]^2) + eps) * norm_w[k]  BPK_PRO_RMS_NORM
 *          = silu(X[m,k]) * X[m,K+k],  X rows are 2K floats      BPK_PRO_SILU_MUL
 *          = gelu_tanh(X[m,k]) * X[m,K+k]                        BPK_PRO_GELU_MUL
 *   Y[m*N + y_offset + n] = bias[n] + residual[m*N + y_offset + n]
 *                           + sum_k x[m,k] * dequant(W)[n,k]
 *
 * silu(g) = g / (1 + exp(-g)); gelu_tanh(g) = 0.5 g (1 + tanh(0.7978845608 (g +
 * 0.044715 g^3))).  residual may be NULL (= zeros) and may be Y itself (the
 * in-place add).  M <= 2 with rows the decode kernel holds in registers
 * (K <= 28672 for one token, K <= 14336 for two; N <= 32768) is one launch
 * and needs no workspace; so are verify batches, M <= 16, on the tile kernel
 * (X, W and norm_w 16-byte aligned; not Q6_K with M > 8 under an act * up
 * prologue).  Other shapes run the same function as prologue, matmul and add
 * launches through `workspace` (device memory, 16-byte aligned, at least
 * bpk_kq_matmul_fused_workspace_bytes(M, N, K) bytes) and fail with
 * BPK_ERR_WORKSPACE without it.
 *
 * Epilogue BPK_EPI_SILU_MUL / BPK_EPI_GELU_MUL folds the same activation into
 * the gate|up matvec instead: W is the stacked gate|up matrix of 2N rows
 * (gate rows first), N counts the outputs, and
 *   Y[m*N + y_offset + n] = act(bias[n] + gate_n . x[m]) * (bias[N+n] + up_n . x[m])
 * so the 2N-float gate|up buffer is never written (the down matvec then takes
 * Y as a plain X).  bias is f32 [2N] or NULL; residual must be NULL.  One launch
 * for Q4_K / Q5_K with M <= 2, and for every type with M <= 16 when N is a
 * multiple of 16; other shapes go through the workspace. */
enum { BPK_PRO_NONE = 0, BPK_PRO_RMS_NORM = 1, BPK_PRO_SILU_MUL = 2, BPK_PRO_GELU_MUL = 3 };
enum { BPK_EPI_NONE = 0, BPK_EPI_SILU_MUL = 2, BPK_EPI_GELU_MUL = 3 };

typedef struct bpk_kq_fusion {
    int prologue;          /* BPK_PRO_*                               */
    const float *norm_w;   /* f32 [K] (device), BPK_PRO_RMS_NORM only */
    float eps;             /* BPK_PRO_RMS_NORM only                   */
    const float *residual; /* f32 (device), indexed like Y, or NULL   */
    int epilogue;          /* BPK_EPI_*                               */
} bpk_kq_fusion;

BPK_API size_t bpk_kq_matmul_fused_workspace_bytes(uint32_t M, uint32_t N,
                                                   uint32_t K);
BPK_API int bpk_kq_matmul_fused(int type, const float *X, const void *W,
                                const float *bias, float *Y, uint32_t M,
                                uint32_t N, uint32_t K, uint32_t n_blocks,
                                uint32_t row_stride_words, uint32_t y_offset,
                                const bpk_kq_fusion *fusion, void *workspace,
                                size_t workspace_bytes, void *stream);

/* ---- chains of decode matvecs: replaces a recorded stretch of the dispatch list ----
 * EXPERIMENTAL, not on the default path: measured slower per token than the same
 * ops as separate bpk_kq_matmul_fused launches; what it buys is one launch per
 * stretch.
 * The reference records one token's dispatches once (buildDecodePipeline) and
 * replays the list per token (runtime/model_runner.cpp:5725-5759).  Between two
 * attention blocks that list is k-quant matvecs and the elementwise dispatches
 * around them: o + add_inplace (runtime/model_runner.cpp:3324-3330), rms_norm,
 * gate|up, act_mul, down + add_inplace (:3711-3793), rms_norm and q|k|v of the
 * next layer (:3206-3243).  A chain holds such a list as bpk_kq_matmul_fused
 * calls with M = 1 and runs any stretch of it, ops [first, first + count), as
 * ONE launch: a persistent grid walks the ops in order without draining between
 * them; an op whose X (or residual) is the output of an earlier op of the launch
 * starts as soon as those outputs have arrived, and the next op's weights are
 * already being fetched while it waits.  Which op feeds which is found from the
 * pointers: an input that lies inside an earlier op's output range comes from
 * that op.  Results are those of the same bpk_kq_matmul_fused calls issued one
 * after the other, except that an input handed from op to op inside a launch
 * has its lowest mantissa bit cleared (a relative 2^-24; Y itself is exact).
 *
 * Each op: the arguments of bpk_kq_matmul_fused with M = 1 (N counts outputs; W
 * has 2N rows with an epilogue).  Served: Q4_K and Q6_K, K <= 18432 (the longest
 * row a workgroup stages in LDS), X and norm_w
 * 16-byte aligned, Q4_K rows 16-byte aligned; the act(gate)*up epilogue for Q4_K
 * with K <= 4096.  An input must lie wholly inside one earlier op's outputs or
 * outside all of them; bpk_chain_create refuses anything else with
 * BPK_ERR_SHAPE / BPK_ERR_TYPE / BPK_ERR_ALIGN (issue such ops as separate
 * calls).  Inside one launch an op may overwrite a buffer an earlier op of that
 * launch uses only if it follows that op through its X (as x += down(...)
 * follows o); bpk_chain_run refuses a range where that is not so with
 * BPK_ERR_SHAPE (cut the launch there).  Pointers are captured at
 * creation, like the reference's bind groups; the buffers must stay valid while
 * the chain lives.
 *
 * bpk_chain_run is asynchronous on `stream`, allocates nothing and may be
 * captured into a HIP graph.  Launches of one chain must not overlap in time,
 * and nothing else should occupy the GPU's compute units while one runs: an op
 * waits for the workgroups that produce its input, every wait is bounded (about
 * two seconds), and a launch whose workgroups were not all resident gives up,
 * leaves outputs unwritten and records the fact.  bpk_chain_status
 * (synchronises with the device) returns BPK_ERR_TIMEOUT once that has
 * happened, and launches do nothing until bpk_chain_reset. */
typedef struct bpk_chain bpk_chain;

typedef struct bpk_chain_op {
    int type;                  /* BPK_TYPE_Q4_K or BPK_TYPE_Q6_K              */
    const float *X;            /* f32 [K], or [2K] for the act prologues      */
    const void *W;
    const float *bias;         /* f32 [rows of W] or NULL                     */
    float *Y;
    uint32_t N, K, n_blocks, row_stride_words, y_offset;
    bpk_kq_fusion fusion;      /* prologue, norm_w, eps, residual, epilogue   */
} bpk_chain_op;

BPK_API int bpk_chain_create(const bpk_chain_op *ops, uint32_t n_ops,
                             bpk_chain **out);
BPK_API int bpk_chain_run(bpk_chain *c, uint32_t first, uint32_t count,
                          void *stream);
BPK_API int bpk_chain_status(bpk_chain *c);
BPK_API int bpk_chain_reset(bpk_chain *c);
BPK_API int bpk_chain_destroy(bpk_chain *c);
/* Diagnostics: the next bpk_chain_run calls on this thread make every workgroup
 * leave wall-clock stamps (100 MHz ticks) in `stamps`, device memory for
 * [workgroups (one per compute unit)][ops of the launch][8] uint64: [0] the op
 * begins, [1] its x is staged, [2] its rows are done; for the launch's first op
 * also [3] the workgroup starts and [4] it has finished its last op.  NULL
 * switches it off. */
BPK_API int bpk_chain_trace(void *stamps);

/* ---- greedy sampling tail: replaces argmax + argmax_reduce -----------------
 * The two dispatches after the lm_head matvec (kernels argmax.wgsl /
 * argmax_reduce.wgsl, wired in runtime/model_runner.cpp:2441-2453), as one
 * launch: out_idx[m] = index of the largest of logits[m*ld .. +N-1], the
 * lowest index among equal maxima (the reference leaves ties to its lane
 * order), 0 when nothing exceeds -1e30 (the reference's starting value).
 * out_val (may be NULL) receives the maximum.  Launches on one device share a
 * scratch area and must not overlap. */
BPK_API int bpk_argmax_rows(const float *logits, uint32_t M, uint32_t N,
                            uint32_t ld, int32_t *out_idx, float *out_val,
                            void *stream);

/* bpk_argmax_rows for callers that cannot allocate device memory: code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It
 * has no counterpart in the reference (whose dispatches bind buffers made at
 * load time).  Same function and same
 * kernel as bpk_argmax_rows; the per-row partial maxima and arrival tickets live
 * in an array inside the library's code object (132 096 bytes per GPU, held
 * until the process ends) instead of allocated scratch, and the call itself
 * allocates and frees nothing.  bpk_init(device) must have run on the current
 * device (that is where the array's address is looked up); otherwise
 * BPK_ERR_DEVICE.  At most BPK_ARGMAX_STATIC_MAX_ROWS rows per call
 * (BPK_ERR_SHAPE beyond); any N.  All calls on one GPU share the array: calls
 * on different streams of one GPU that overlap in time race.  The tickets are
 * zero when the library is loaded and each launch leaves them zero again. */
#define BPK_ARGMAX_STATIC_MAX_ROWS 256u
BPK_API int bpk_argmax_rows_static(const float *logits, uint32_t M, uint32_t N,
                                   uint32_t ld, int32_t *out_idx,
                                   float *out_val, void *stream);

/* lm_head and its argmax in one call (runtime/model_runner.cpp:4124-4135 then
 * :2441-2453): bpk_kq_matmul with y_offset 0 into `logits` (f32 [M,N], kept for
 * the caller) followed by bpk_argmax_rows on it. */
BPK_API int bpk_kq_matmul_argmax(int type, const float *X, const void *W,
                                 const float *bias, float *logits, uint32_t M,
                                 uint32_t N, uint32_t K, uint32_t n_blocks,
                                 uint32_t row_stride_words, int32_t *out_idx,
                                 float *out_val, void *stream);

/* Prefill form: X is bf16 [M,K] (raw 16-bit patterns), Y f32 [M,N].  Weight
 * tiles are dequantised to bf16 in LDS and contracted on the matrix cores
 * with fp32 accumulation.  The reference has no such kernel: its k-quant
 * prefill loops the M=1 path (runtime/model_runner.cpp:6148-6158); the
 * contract is the same formula as bpk_kq_matmul. */
BPK_API int bpk_kq_matmul_bf16(int type, const uint16_t *X, const void *W,
                               const float *bias, float *Y, uint32_t M,
                               uint32_t N, uint32_t K, uint32_t n_blocks,
                               uint32_t row_stride_words, void *stream);

/* Activation rows for bpk_kq_matmul_bf16 from the engine's fp32 buffers:
 *   out[m*K + k] = bf16(x[m,k]), round to nearest even, with x the prologue
 * forms of bpk_kq_matmul_fused (BPK_PRO_NONE: X as it is; BPK_PRO_RMS_NORM:
 * norm/rms_norm.wgsl:15-20; BPK_PRO_SILU_MUL / BPK_PRO_GELU_MUL: X rows are
 * gate | up, 2K floats, fused/silu_mul_fused.wgsl:39-49 and
 * fused/gelu_mul_fused.wgsl:22-32), evaluated in fp32.  The reference keeps
 * activations in fp32 and has no bf16 path; this is the one pass its norm and
 * act*mul dispatches become in front of a prefill GEMM.  X f32 (device),
 * out bf16 [M,K] (device, 2-byte aligned); K any positive size. */
BPK_API int bpk_prefill_rows_bf16(int prologue, const float *X,
                                  const float *norm_w, float eps, uint32_t M,
                                  uint32_t K, uint16_t *out, void *stream);

/* ---- dequantised rows: replaces q6k_gather / q6k_gather_batched -------------
 * runtime/kernels/quant_kq/q6k_gather.wgsl:15-44, q6k_gather_batched.wgsl:9-21.
 * out[m*K + k] = dequant(W)[max(rows[m],0), k], bit-identical to
 * dequant_kquant (runtime/gguf_loader.cpp:455-573).  rows: i32 [M] (device);
 * NULL selects rows 0..M-1. */
BPK_API int bpk_kq_dequant_rows(int type, const void *W,
                                uint32_t row_stride_words, const int32_t *rows,
                                uint32_t M, uint32_t K, float *out,
                                void *stream);

/* ---- MoE expert matmul: replaces the *_matmul_moe indirection ---------------
 * runtime/kernels/quant_kq/iq4xs_matmul_moe.wgsl:55-66 with offsets from
 * runtime/kernels/moe/compute_offsets.wgsl:25-36 (decode), and the per-token
 * form of runtime/ops/moe.cpp:486-592 (expert = expert_indices[tok*k + slot]).
 * W is the stacked matrix [n_experts*N, K]; expert e owns rows e*N..e*N+N-1.
 *
 *   Y[(t*k+s)*N + n] = sum_k X[xrow*K + k] * dequant(W)[idx[t*k+s]*N + n, k]
 *   xrow = t            when x_per_slot == 0 (gate / up: one X row per token)
 *        = t*k + s      when x_per_slot != 0 (down: one X row per pair)
 *
 * expert_idx: u32 [T*k] (device).  Pairs are grouped by expert on the GPU so
 * each touched expert's weights are streamed once; no host synchronisation. */
BPK_API int bpk_kq_moe_matmul(int type, const float *X, const void *W,
                              const uint32_t *expert_idx, float *Y, uint32_t T,
                              uint32_t k, uint32_t n_experts, uint32_t N,
                              uint32_t K, uint32_t n_blocks,
                              uint32_t row_stride_words, int x_per_slot,
                              void *stream);

/* ---- MoE router stage: replaces moe_topk_softmax (and the router matmul) ----
 * runtime/kernels/moe/topk_softmax.wgsl:23-67, dispatched after the router
 * matmul in runtime/model_runner.cpp:3532-3548; its outputs are the expert_idx /
 * expert_wt inputs of the calls above and below.  Per token: k passes of argmax
 * over the experts not yet taken (`v > best` with best starting at -3.4e38 and
 * index 0, so the lowest index wins a tie), then wt = exp(v - max) over the
 * selected, times 1/sum when `normalize` is set and the sum is positive.
 * logits: f32 [T, n_experts]; idx: u32 [T, k]; wt: f32 [T, k] (all device).
 * n_experts <= 1024 (the reference's mask array), k <= 16 (its MAX_K). */
BPK_API int bpk_moe_topk_softmax(const float *logits, uint32_t T,
                                 uint32_t n_experts, uint32_t k, int normalize,
                                 uint32_t *idx, float *wt, void *stream);

/* The same behind the router matvec, one call (two launches): logits[t, e] = sum_h X[t, h] *
 * router_w[e, h] in fp32 (GGUF keeps `ffn_gate_inp.weight` as F32 [hidden,
 * n_experts]; the reference requantises it to Q8 for its Q8 matmul,
 * model_runner.cpp:3532-3540).  `logits` may be NULL when the caller does not
 * need them.  hidden % 4 == 0; X and router_w 16-byte aligned. */
BPK_API int bpk_moe_route(const float *X, const float *router_w, uint32_t T,
                          uint32_t hidden, uint32_t n_experts, uint32_t k,
                          int normalize, float *logits, uint32_t *idx, float *wt,
                          void *stream);

/* Whole routed-expert FFN for T tokens, replacing the per-slot dispatch list of
 * runtime/model_runner.cpp:3584-3651 (gate, up, silu*mul, down, weighted
 * accumulate) and the batched form in runtime/ops/moe.cpp:486-592:
 *   act = silu(gate_e x) * (up_e x);  out[t] = sum_s wt[t,s] * (down_e act)
 * gate/up: [n_experts*inter, hidden] of type_gu; down: [n_experts*hidden, inter]
 * of type_dn.  out: f32 [T, hidden], overwritten.  scratch: device memory of
 * at least bpk_kq_moe_ffn_scratch_bytes(T, k, hidden, inter) bytes. */
BPK_API size_t bpk_kq_moe_ffn_scratch_bytes(uint32_t T, uint32_t k,
                                            uint32_t hidden, uint32_t inter);
BPK_API int bpk_kq_moe_ffn(int type_gu, int type_dn, const float *X,
                           const void *gate, const void *up, const void *down,
                           const uint32_t *expert_idx, const float *expert_wt,
                           float *out, uint32_t T, uint32_t k,
                           uint32_t n_experts, uint32_t hidden, uint32_t inter,
                           void *scratch, size_t scratch_bytes, void *stream);

/* ---- introspection for tests and benchmarks --------------------------------
 * Name of the kernel the last bpk_kq_matmul* call on this thread launched
 * ("" before the first). */
BPK_API const char *bpk_last_kernel(void);

/* Force a kernel family for the next calls on this thread (testing only):
 * 0 = automatic, 1 = generic, 2 = row-per-lane GEMV (M <= 4), 3 = row-per-lane
 * kernel on the 4x4x4 matrix-core op (M <= 16), 4 = matrix-core tiled GEMM
 * (bf16 X only), 5 = lanes-along-K GEMV (M = 1), 6 = 16-row x 16-token
 * matrix-core tiles (M <= 16), 7 = one token on the matrix cores (Q4_K rows of
 * up to 16 superblocks).  A forced family that cannot serve the call's
 * shape fails with BPK_ERR_SHAPE instead of falling back. */
BPK_API int bpk_force_kernel(int family);

/* Tuning knobs for experiments on this thread.  "gemv_splits": number of
 * K-range splits of the row-per-lane GEMV, or rows per wave of the
 * lanes-along-K GEMV; "gemv_waves": waves per workgroup of the row-per-lane
 * kernels (2, 4 or 8); "gemv_depth": rows a wave of the lanes-along-K GEMV
 * keeps in flight (1, 2 or 4); "gemm_tile": workgroup tile of the bf16
 * GEMM (128 or 256: square; 129: 256 tokens x 128 weight rows; 192: 256 tokens
 * x 192 weight rows); "gemm_split": how the 256-tile GEMM hands out work
 * (1 = one tile per workgroup, 2 = the walk over tiles and k steps cut into
 * equal shares per compute unit; the runs of a tile cut between workgroups go
 * through a per-device workspace and are added in the order of the walk, so
 * results repeat bit for bit); "fused_separate": 1 makes bpk_kq_matmul_fused run its prologue,
 * matmul and add as separate launches for every shape (needs the workspace);
 * "mgemv": which one-token Q4_K matvecs go to the matrix-core kernel instead of
 * the lanes-along-K kernel: 0 none, 1 (default) matrices of 49152 rows and more,
 * 2 from 16384 rows on (gate|up: level on most parts, ahead where the clock runs low);
 * "moe_fold": 0 keeps the weighted sum over a token's slots behind the expert FFN
 * a launch of its own (default 1: inside the last matvec's launch where its
 * kernel can: a few pairs, Q6_K down projection, at most 8 slots per token),
 * and the batched tile path's gate and up two launches and an activation
 * kernel (default: one launch that stores silu(gate x) * (up x), where hidden
 * spans more than four superblocks); "moe_tile_iters": tiles of 16 rows a wave
 * of the batched tile path walks with a record's activations staged once, where
 * K is at most four superblocks (1, 2, 4 or 8; 0 = chosen per call from the
 * expected number of records, so that the workgroups fill whole rounds);
 * "chain_spin_us": bound of a wait between the ops of a chain in microseconds
 * (at most ten seconds);
 * "chain_hold" (test hook, refused unless chain_spin_us is 1..100000): 1 keeps
 * the ops of a chain from handing their outputs on, so that every wait for them
 * runs out (the way the tests reach the give-up path with every workgroup
 * exiting normally); "chain_ahead": 1 + the rows per wave
 * of the next op touched into L2 while an op finishes.  0 = automatic. */
BPK_API int bpk_set_option(const char *name, int value);

/* Which form of the bf16 dequant-GEMM bpk_kq_matmul_bf16 takes for a shape on a
 * part of `compute_units` CUs, with this thread's "gemm_tile" / "gemm_split"
 * options: host arithmetic only, no device is touched (diagnostic; the reference
 * has no such kernel, its prefill loops M = 1, runtime/model_runner.cpp:6148-6158).
 * *form: 0 = 128 x 128 tiles; 1 = 256 x 256 tiles, one workgroup each; 2 = the
 * walk over the 256-tiles' k steps cut into equal shares (*share k steps each);
 * 3 = tiles of 256 tokens x 128 weight rows; 4 = the full rounds of 256-tiles
 * over the first *rows_first weight rows, then the rest as in 3; 5 = tiles of
 * 256 tokens x 192 weight rows. */
BPK_API int bpk_gemm_plan(int type, uint32_t M, uint32_t N, uint32_t K, uint32_t compute_units,
                          int *form, uint32_t *share, uint32_t *rows_first);

#ifdef __cplusplus
}
#endif
#endif /* BPK_KQUANT_H */
