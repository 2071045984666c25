// bpk_api.hip — the C ABI (include/bpk_kquant.h): argument checking, per-device
// state, kernel-family choice, launches.  No arithmetic lives here.
#include "../../include/bpk_kquant.h"

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <new>
#include <thread>
#include <vector>

#include "kq_format.h"
#include "kq_gemm_plan.h"
#include "kq_kernels.h"

namespace {

constexpr int kMaxDevices = 16;
constexpr size_t kPartialFloats = size_t(4) << 20;  // 16 MiB of split-K partial sums
constexpr uint32_t kCounters = 1u << 16;
// bf16 GEMM: two 256 x 256 fp32 slots per workgroup for the runs of cut tiles, a workgroup per CU
constexpr size_t kGemmPartialFloats = size_t(2) * 256 * 65536;  // 128 MiB
constexpr size_t kMoeWords = size_t(4) << 20;       // 16 MiB of tile records for bpk_kq_moe_matmul
static_assert(BPK_ARGMAX_STATIC_MAX_ROWS == kq::ARGMAX_MAX_ROWS, "the header's limit is the scratch array's");

thread_local char t_err[512] = "";
thread_local const char* t_kernel = "";
thread_local int t_family = 0;
thread_local kq::GemvTuning t_gemv;
thread_local int t_gemm_tile = 0;
thread_local int t_gemm_split = 0;
thread_local int t_moe_tile_iters = 0; // option "moe_tile_iters": tiles a wave of the grouped tile kernel walks per staged X (0: chosen per call)
thread_local bool t_moe_fold = true;    // option "moe_fold": the slots' weighted sum inside the last matvec where its kernel can
thread_local int t_fused_separate = 0;
thread_local int t_chain_spin_us = 0;    // 0 = default
thread_local int t_chain_ahead = 0;      // 1 + rows touched ahead; 0 = default
thread_local void* t_chain_trace = nullptr;   // device buffer for the chain kernel's time stamps (diagnostics)
thread_local int t_chain_hold = 0;
thread_local int t_mgemv_auto = 1;       // option "mgemv": 0 never, 1 from 49152 rows on, 2 from 16384 rows on

int fail(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(t_err, sizeof t_err, fmt, ap);
    va_end(ap);
    return code;
}

}  // namespace

// The same for the library's other sources: stores the message bpk_last_error() returns.
namespace kq {
int api_fail(int code, const char* fmt, va_list ap)
{
    vsnprintf(t_err, sizeof t_err, fmt, ap);
    return code;
}
}  // namespace kq

namespace {

int hip_fail(hipError_t e, const char* what)
{
    return fail(BPK_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

// Pinned double buffer of the weight upload: one half is filled by host threads while the other is in
// flight to the device.
constexpr size_t kStageBytes = size_t(32) << 20;
struct UploadStage {
    void* buf[2] = {nullptr, nullptr};
    hipEvent_t sent[2] = {nullptr, nullptr};
    hipStream_t stream = nullptr;
};

struct DeviceState {
    bool ready = false;
    kq::SplitScratch split{};
    kq::SplitScratch gemm_split{};   // of the bf16 GEMM's cut tiles (its own, so that it can run beside a GEMV)
    uint32_t* moe_tiles = nullptr;   // kMoeWords words
    uint32_t* argmax_scratch = nullptr;   // partial values | partial indices | tickets of bpk_argmax_rows
    float* route_logits = nullptr;   // ROUTE_SCRATCH_FLOATS router logits of a route call that does not return them
    uint32_t* argmax_static = nullptr;    // this device's copy of the scratch array in the code object (not allocated)
    UploadStage up{};                // created by the first upload on the device
};

std::mutex g_mu;
DeviceState g_dev[kMaxDevices];

// Frees every device buffer of the state (hipFree(nullptr) is a no-op); the device must be current.
void free_device_buffers(DeviceState& st)
{
    (void)hipFree(st.split.partial);
    (void)hipFree(st.split.counters);
    (void)hipFree(st.gemm_split.partial);
    (void)hipFree(st.moe_tiles);
    (void)hipFree(st.route_logits);
    (void)hipFree(st.argmax_scratch);
}

int ensure_device(int device, DeviceState** out)
{
    if (device < 0 || device >= kMaxDevices) return fail(BPK_ERR_DEVICE, "device %d out of range", device);
    std::lock_guard<std::mutex> lk(g_mu);
    DeviceState& st = g_dev[device];
    if (!st.ready) {
        hipDeviceProp_t prop;
        hipError_t e = hipGetDeviceProperties(&prop, device);
        if (e != hipSuccess) return hip_fail(e, "hipGetDeviceProperties");
        if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
            return fail(BPK_ERR_DEVICE, "device %d is %s; this library is built for gfx950 only", device,
                        prop.gcnArchName);
        int cur = -1;
        (void)hipGetDevice(&cur);
        if (cur != device) (void)hipSetDevice(device);
        e = hipMalloc((void**)&st.split.partial, kPartialFloats * sizeof(float));
        if (e == hipSuccess) e = hipMalloc((void**)&st.split.counters, kCounters * sizeof(uint32_t));
        if (e == hipSuccess) e = hipMemset(st.split.counters, 0, kCounters * sizeof(uint32_t));
        if (e == hipSuccess) e = hipMalloc((void**)&st.gemm_split.partial, kGemmPartialFloats * sizeof(float));
        if (e == hipSuccess) e = hipMalloc((void**)&st.moe_tiles, kMoeWords * sizeof(uint32_t));
        constexpr size_t kArgmaxWords = (size_t)kq::ARGMAX_MAX_ROWS * (2u * kq::ARGMAX_PARTS + 1u);
        if (e == hipSuccess) e = hipMalloc((void**)&st.argmax_scratch, kArgmaxWords * sizeof(uint32_t));
        if (e == hipSuccess) e = hipMemset(st.argmax_scratch, 0, kArgmaxWords * sizeof(uint32_t));
        if (e == hipSuccess) e = hipMalloc((void**)&st.route_logits, kq::ROUTE_SCRATCH_FLOATS * sizeof(float));
        if (e == hipSuccess) e = kq::argmax_static_scratch(&st.argmax_static);   // with `device` current
        if (e != hipSuccess) {
            // nothing half-made stays behind: a later call starts from scratch
            free_device_buffers(st);
            st = DeviceState{};
        }
        if (cur != device && cur >= 0) (void)hipSetDevice(cur);
        if (e != hipSuccess) return hip_fail(e, "allocating the per-device scratch");
        st.split.capacity_floats = kPartialFloats;
        st.split.n_counters = kCounters;
        st.gemm_split.capacity_floats = kGemmPartialFloats;
        st.gemm_split.n_counters = 0;   // the sum kernel needs no arrival counters
        st.ready = true;
    }
    if (out) *out = &st;
    return BPK_OK;
}

int current_state(DeviceState** out)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
    return ensure_device(dev, out);
}

bool known_type(int type) { return type == BPK_TYPE_Q4_K || type == BPK_TYPE_Q5_K || type == BPK_TYPE_Q6_K; }

int check_matmul(int type, const void* X, const void* W, const void* Y, uint32_t M, uint32_t N, uint32_t K,
                 uint32_t n_blocks, uint32_t row_stride_words)
{
    if (!known_type(type)) return fail(BPK_ERR_TYPE, "unsupported GGUF type %d (Q4_K=12, Q5_K=13, Q6_K=14)", type);
    if (!X || !W || !Y) return fail(BPK_ERR_NULL, "X, W and Y must be non-null");
    if (K == 0 || K % KQ_QK) return fail(BPK_ERR_SHAPE, "K=%u is not a positive multiple of 256", K);
    if (N == 0) return fail(BPK_ERR_SHAPE, "N must be positive");
    if (n_blocks != K / KQ_QK) return fail(BPK_ERR_SHAPE, "n_blocks=%u does not match K/256=%u", n_blocks, K / KQ_QK);
    const uint64_t row_bytes = (uint64_t)n_blocks * kq::block_bytes(type);
    if ((uint64_t)row_stride_words * 4u < row_bytes)
        return fail(BPK_ERR_SHAPE, "row_stride_words=%u is smaller than a row (%llu bytes)", row_stride_words,
                    (unsigned long long)row_bytes);
    if ((uint64_t)row_stride_words * 4u > 0xFFFFFFFFull) return fail(BPK_ERR_SHAPE, "row stride too large");
    if ((uintptr_t)W & 3u) return fail(BPK_ERR_ALIGN, "W must be 4-byte aligned");
    if ((uintptr_t)X & 3u || (uintptr_t)Y & 3u) return fail(BPK_ERR_ALIGN, "X and Y must be 4-byte aligned");
    (void)M;
    return BPK_OK;
}

}  // namespace

extern "C" {

int bpk_version(void) { return 100; }

const char* bpk_last_error(void) { return t_err; }

const char* bpk_last_kernel(void) { return t_kernel; }

int bpk_force_kernel(int family)
{
    if (family < 0 || family > 7) return fail(BPK_ERR_SHAPE, "kernel family %d unknown", family);
    t_family = family;
    return BPK_OK;
}

int bpk_set_option(const char* name, int value)
{
    if (!name) return fail(BPK_ERR_NULL, "option name is null");
    if (!strcmp(name, "gemv_splits")) { t_gemv.splits = value; return BPK_OK; }
    if (!strcmp(name, "gemv_waves")) {
        if (value != 0 && value != 2 && value != 4 && value != 8)
            return fail(BPK_ERR_SHAPE, "gemv_waves must be 0, 2, 4 or 8");
        t_gemv.waves = value;
        return BPK_OK;
    }
    if (!strcmp(name, "gemv_depth")) {
        if (value < 0 || value > 8) return fail(BPK_ERR_SHAPE, "gemv_depth must be 0..8");
        t_gemv.depth = value;
        return BPK_OK;
    }
    if (!strcmp(name, "gemm_tile")) {
        if (value != 0 && value != 128 && value != 129 && value != 192 && value != 256)
            return fail(BPK_ERR_SHAPE, "gemm_tile must be 0, 128, 129, 192 or 256");
        t_gemm_tile = value;
        return BPK_OK;
    }
    if (!strcmp(name, "fused_separate")) {
        t_fused_separate = value != 0;
        return BPK_OK;
    }
    if (!strcmp(name, "chain_ahead")) {
        if (value < 0 || value > 9) return fail(BPK_ERR_SHAPE, "chain_ahead must be 0..9");
        t_chain_ahead = value;
        return BPK_OK;
    }
    if (!strcmp(name, "chain_spin_us")) {
        if (value < 0 || value > 10000000) return fail(BPK_ERR_SHAPE, "chain_spin_us must lie in 0 .. 10000000 (ten seconds)");
        t_chain_spin_us = value;
        return BPK_OK;
    }
    if (!strcmp(name, "mgemv")) {
        if (value < 0 || value > 2) return fail(BPK_ERR_SHAPE, "mgemv must be 0, 1 or 2");
        t_mgemv_auto = value;
        return BPK_OK;
    }
    if (!strcmp(name, "chain_hold")) {
        t_chain_hold = value != 0;
        return BPK_OK;
    }
    if (!strcmp(name, "moe_tile_iters")) {
        if (value != 0 && value != 1 && value != 2 && value != 4 && value != 8) return fail(BPK_ERR_SHAPE, "moe_tile_iters must be 0, 1, 2, 4 or 8");
        t_moe_tile_iters = value;
        return BPK_OK;
    }
    if (!strcmp(name, "moe_fold")) {
        t_moe_fold = value != 0;
        return BPK_OK;
    }
    if (!strcmp(name, "gemm_split")) {
        if (value < 0 || value > 2) return fail(BPK_ERR_SHAPE, "gemm_split must be 0, 1 or 2");
        t_gemm_split = value;
        return BPK_OK;
    }
    return fail(BPK_ERR_SHAPE, "unknown option '%s'", name);
}

int bpk_gemm_plan(int type, uint32_t M, uint32_t N, uint32_t K, uint32_t compute_units, int* form, uint32_t* share,
                  uint32_t* rows_first)
{
    if (!known_type(type)) return fail(BPK_ERR_TYPE, "unsupported GGUF type (Q4_K=12, Q5_K=13, Q6_K=14)");
    if (!form || !share || !rows_first) return fail(BPK_ERR_NULL, "form, share and rows_first must be non-null");
    if (M == 0 || N == 0 || K == 0 || K % KQ_QK || compute_units == 0)
        return fail(BPK_ERR_SHAPE, "M, N, compute_units must be positive and K a positive multiple of 256");
    const kq::GemmPlan pl = kq::plan_gemm_bf16(type, M, N, K, compute_units, t_gemm_tile, t_gemm_split);
    *form = pl.form;
    *share = pl.share;
    *rows_first = pl.rows_first;
    return BPK_OK;
}

int bpk_init(int device) { return ensure_device(device, nullptr); }

int bpk_shutdown(void)
{
    std::lock_guard<std::mutex> lk(g_mu);
    int cur = -1;
    (void)hipGetDevice(&cur);
    for (int d = 0; d < kMaxDevices; ++d) {
        DeviceState& st = g_dev[d];
        if (!st.ready) continue;
        (void)hipSetDevice(d);
        free_device_buffers(st);
        for (int b = 0; b < 2; ++b) {
            if (st.up.buf[b]) (void)hipHostFree(st.up.buf[b]);
            if (st.up.sent[b]) (void)hipEventDestroy(st.up.sent[b]);
        }
        if (st.up.stream) (void)hipStreamDestroy(st.up.stream);
        st = DeviceState{};
    }
    if (cur >= 0) (void)hipSetDevice(cur);
    return BPK_OK;
}

int bpk_kq_layout(int type, uint32_t K, uint32_t* n_blocks, uint32_t* row_stride_words)
{
    if (!known_type(type)) return fail(BPK_ERR_TYPE, "unsupported GGUF type %d", type);
    const uint32_t nb = (K + KQ_QK - 1) / KQ_QK;
    if (n_blocks) *n_blocks = nb;
    if (row_stride_words) *row_stride_words = (nb * kq::block_bytes(type) + 3u) / 4u;
    return BPK_OK;
}

int bpk_kq_pack_host(int type, const void* raw, uint32_t N, uint32_t K, uint32_t* out_words)
{
    if (!known_type(type)) return fail(BPK_ERR_TYPE, "unsupported GGUF type %d", type);
    if (!raw || !out_words) return fail(BPK_ERR_NULL, "raw and out_words must be non-null");
    uint32_t nb, rs;
    bpk_kq_layout(type, K, &nb, &rs);
    const size_t row_bytes = (size_t)nb * kq::block_bytes(type), stride = (size_t)rs * 4u;
    const uint8_t* src = (const uint8_t*)raw;
    uint8_t* dst = (uint8_t*)out_words;
    for (uint32_t n = 0; n < N; ++n) {
        memcpy(dst + n * stride, src + n * row_bytes, row_bytes);
        memset(dst + n * stride + row_bytes, 0, stride - row_bytes);
    }
    return BPK_OK;
}

struct bpk_weight {
    bpk_weight_desc d;
    int device;
};

// Packed rows [row0, row0+n) of the stacked matrix -> dst (n*stride bytes).  Parts are raw GGUF rows of
// row_bytes each; a packed row is the raw row plus zero padding to the word boundary.
static void pack_stacked_rows(const void* const* parts, const uint32_t* n_rows, uint32_t n_parts, uint64_t row0,
                              uint64_t n, size_t row_bytes, size_t stride, uint8_t* dst)
{
    uint64_t first = 0;
    for (uint32_t i = 0; i < n_parts && n; first += n_rows[i], ++i) {
        if (row0 >= first + n_rows[i]) continue;
        const uint64_t r = row0 - first;
        const uint64_t take = n_rows[i] - r < n ? n_rows[i] - r : n;
        const uint8_t* src = (const uint8_t*)parts[i] + r * row_bytes;
        if (stride == row_bytes) {
            memcpy(dst, src, take * row_bytes);
        } else {
            for (uint64_t k = 0; k < take; ++k) {
                memcpy(dst + k * stride, src + k * row_bytes, row_bytes);
                memset(dst + k * stride + row_bytes, 0, stride - row_bytes);
            }
        }
        dst += take * stride;
        row0 += take;
        n -= take;
    }
}

int bpk_weight_create(int type, uint32_t K, uint32_t n_parts, const void* const* parts, const uint32_t* n_rows,
                      bpk_weight** out)
{
    if (!known_type(type)) return fail(BPK_ERR_TYPE, "unsupported GGUF type %d", type);
    if (!parts || !n_rows || !out) return fail(BPK_ERR_NULL, "parts, n_rows and out must be non-null");
    if (K == 0 || K % KQ_QK) return fail(BPK_ERR_SHAPE, "K=%u is not a positive multiple of 256", K);
    uint64_t N = 0;
    for (uint32_t i = 0; i < n_parts; ++i) {
        if (!parts[i]) return fail(BPK_ERR_NULL, "parts[%u] is null", i);
        N += n_rows[i];
    }
    if (N == 0 || N > 0xFFFFFFFFull) return fail(BPK_ERR_SHAPE, "total rows %llu out of range", (unsigned long long)N);
    DeviceState* st;
    if (int rc = current_state(&st)) return rc;
    uint32_t nb, rs;
    bpk_kq_layout(type, K, &nb, &rs);
    const size_t row_bytes = (size_t)nb * kq::block_bytes(type), stride = (size_t)rs * 4u;
    if (stride > kStageBytes) return fail(BPK_ERR_SHAPE, "a row of %zu bytes exceeds the upload stage", stride);
    const size_t bytes = (size_t)N * stride;

    // One upload at a time per process: the stage is shared.
    static std::mutex up_mu;
    std::lock_guard<std::mutex> lk(up_mu);
    UploadStage& up = st->up;
    hipError_t e = hipSuccess;
    if (!up.stream) {
        e = hipStreamCreateWithFlags(&up.stream, hipStreamNonBlocking);
        for (int b = 0; b < 2 && e == hipSuccess; ++b) {
            e = hipHostMalloc(&up.buf[b], kStageBytes, hipHostMallocDefault);
            if (e == hipSuccess) e = hipEventCreateWithFlags(&up.sent[b], hipEventDisableTiming);
        }
        if (e != hipSuccess) return hip_fail(e, "creating the upload stage");
    }
    void* dptr = nullptr;
    // 16 trailing bytes let 128-bit loads of the last row's tail stay in bounds
    e = hipMalloc(&dptr, bytes + 16);
    if (e != hipSuccess) return hip_fail(e, "hipMalloc(weights)");

    const uint64_t rows_per_chunk = kStageBytes / stride;
    const unsigned hw = std::thread::hardware_concurrency();
    const unsigned n_threads = hw >= 8 ? 8 : (hw ? hw : 1);
    uint64_t row = 0;
    for (uint64_t c = 0; row < N && e == hipSuccess; ++c) {
        const int b = (int)(c & 1);
        if (c >= 2) e = hipEventSynchronize(up.sent[b]);
        if (e != hipSuccess) break;
        const uint64_t n = N - row < rows_per_chunk ? N - row : rows_per_chunk;
        uint8_t* dst = (uint8_t*)up.buf[b];
        // host threads share the chunk's rows; small chunks are not worth a thread each
        const unsigned t_use = n * stride >= (size_t(4) << 20) ? n_threads : 1;
        if (t_use == 1) {
            pack_stacked_rows(parts, n_rows, n_parts, row, n, row_bytes, stride, dst);
        } else {
            std::vector<std::thread> pool;
            const uint64_t per = (n + t_use - 1) / t_use;
            for (unsigned t = 0; t < t_use; ++t) {
                const uint64_t r0 = t * per;
                if (r0 >= n) break;
                const uint64_t cnt = n - r0 < per ? n - r0 : per;
                pool.emplace_back(pack_stacked_rows, parts, n_rows, n_parts, row + r0, cnt, row_bytes, stride,
                                  dst + r0 * stride);
            }
            for (auto& th : pool) th.join();
        }
        e = hipMemcpyAsync((uint8_t*)dptr + row * stride, dst, n * stride, hipMemcpyHostToDevice, up.stream);
        if (e == hipSuccess) e = hipEventRecord(up.sent[b], up.stream);
        row += n;
    }
    if (e == hipSuccess) e = hipMemsetAsync((uint8_t*)dptr + bytes, 0, 16, up.stream);
    const hipError_t e_sync = hipStreamSynchronize(up.stream);   // also on failure: the stage must be idle on return
    if (e == hipSuccess) e = e_sync;
    if (e != hipSuccess) {
        (void)hipFree(dptr);
        return hip_fail(e, "uploading weights");
    }
    bpk_weight* w = new (std::nothrow) bpk_weight;
    if (!w) {
        (void)hipFree(dptr);
        return fail(BPK_ERR_SHAPE, "out of host memory");
    }
    w->d = bpk_weight_desc{type, (uint32_t)N, K, nb, rs, dptr, bytes};
    (void)hipGetDevice(&w->device);
    *out = w;
    return BPK_OK;
}

int bpk_weight_describe(const bpk_weight* w, bpk_weight_desc* out)
{
    if (!w || !out) return fail(BPK_ERR_NULL, "weight and out must be non-null");
    *out = w->d;
    return BPK_OK;
}

int bpk_weight_destroy(bpk_weight* w)
{
    if (!w) return BPK_OK;
    hipError_t e = hipFree(w->d.data);
    delete w;
    return e == hipSuccess ? BPK_OK : hip_fail(e, "hipFree(weights)");
}

// fold: the greedy pick over the outputs, taken along by the launch where its kernel can (*folded says so)
static int matmul_impl(int type, const float* X, const void* W, const float* bias, float* Y, uint32_t M, uint32_t N,
                       uint32_t K, uint32_t n_blocks, uint32_t row_stride_words, uint32_t y_offset, void* stream,
                       const kq::ArgmaxFold* fold, bool* folded)
{
    if (int rc = check_matmul(type, X, W, Y, M, N, K, n_blocks, row_stride_words)) return rc;
    if (M == 0) return BPK_OK;
    DeviceState* st;
    if (int rc = current_state(&st)) return rc;
    kq::MatmulArgs a{};
    a.type = type; a.X = X; a.W = (const uint8_t*)W; a.bias = bias; a.Y = Y;
    a.M = M; a.N = N; a.K = K; a.n_blocks = n_blocks;
    a.row_stride_bytes = row_stride_words * 4u;
    a.y_offset = y_offset;
    a.ldy = N;
    hipStream_t s = (hipStream_t)stream;
    hipError_t e;
    const bool rows_ok = kq::gemv_rows_supported(a);
    const bool mrow_ok = kq::mrow_supported(a);
    if (t_family == 2 && !rows_ok) return fail(BPK_ERR_SHAPE, "row-per-lane GEMV cannot serve this call");
    if (t_family == 3 && !mrow_ok) return fail(BPK_ERR_SHAPE, "matrix-core row kernel cannot serve this call");
    const bool stream_ok = kq::gemv_stream_supported(a);
    const bool mtile_ok = kq::mtile_supported(a);
    if (t_family == 6 && !mtile_ok) return fail(BPK_ERR_SHAPE, "16x16 tile kernel cannot serve this call");
    // three and four tokens on the smaller matrices stay on the lanes-along-K kernel (four tokens share every
    // weight load and its unpack).  Measured at M = 4: Q4_K 4096x4096 8.5 against 10.6 us on the tile
    // kernel, 6144x4096 10.8 against 11.8, 28672x4096 32.6 against 19.2; Q6_K 4096x14336 23.2 against 27.0.
    const uint64_t weights = (uint64_t)N * K;
    const bool stream_four = stream_ok && M >= 3 && M <= 4 && N <= 32768u &&
                             weights <= (type == BPK_TYPE_Q6_K ? (64ull << 20) : (32ull << 20));
    // two tokens on a Q4_K / Q5_K matrix of gate|up's size: the tile kernel's form for up to 8 tokens (hi and lo
    // parts as token slots) beats two tokens on the vector units there (28672x4096: 19.6 against 22.7 us; 6144x4096:
    // 11.1 against 8.5, so smaller matrices stay)
    const bool tile_two = M == 2 && type != BPK_TYPE_Q6_K && weights >= (64ull << 20);
    if (t_family == 6 || (t_family == 0 && mtile_ok && ((M >= 3 && !stream_four) || tile_two))) {
        t_kernel = "mtile";
        e = kq::launch_mtile(a, st->split, s);
        return e == hipSuccess ? BPK_OK : hip_fail(e, t_kernel);
    }
    // One token on a Q4_K matrix of very many rows: the contraction on the matrix cores.  Its steady state is
    // faster than the lanes-along-K kernel's (6.5 against 5.7-6.0 TB/s: 114688 x 4096 takes 44.3 against 48.7 us,
    // 57344 x 4096 23.9 against 25.3), its start and end are not (x is split and laid out as operands before the
    // first product, the waves meet before the stores), and on gate|up's 28672 x 4096 the two are level — 13.9
    // against 13.9-14.0 us alone; inside the decode step the lanes-along-K kernel is 0.3 us ahead per launch, and
    // every other kernel of the step ran 1 % slower next to this one (1.219 against 1.210 ms on four boxes).  On
    // parts whose clock runs low the order flips (14.4 against 15.8-16.4 us).  So: from 49152 rows on.
    const bool mgemv_ok = kq::mgemv_supported(a);
    if (t_family == 7 && !mgemv_ok) return fail(BPK_ERR_SHAPE, "matrix-core GEMV cannot serve this call");
    if (t_family == 7 || (t_family == 0 && mgemv_ok && N >= (t_mgemv_auto == 2 ? 16384u : 49152u) && t_mgemv_auto)) {
        t_kernel = "mgemv";
        e = kq::launch_mgemv(a, kq::device_cu_count(), t_gemv.splits, s);
        return e == hipSuccess ? BPK_OK : hip_fail(e, t_kernel);
    }
    if (t_family == 5 && !stream_ok) return fail(BPK_ERR_SHAPE, "lanes-along-K GEMV cannot serve this call");
    if (t_family == 4) return fail(BPK_ERR_SHAPE, "kernel family %d is not available for fp32 X", t_family);
    // The lanes-along-K kernel (no LDS staging, no K split to fold) wins everywhere except on Q6_K matrices
    // of more than a few tens of thousands of rows at one token, where the row-per-lane kernel reaches a
    // faster steady state (128256 x 4096: 90 against 97 us; at two tokens 129 against 102 us, and Q4_K of
    // that size 152 against 82 us).
    const bool stream_rows_ok = N <= 32768u || M == 2u || type != BPK_TYPE_Q6_K;
    if (t_family == 5 || (t_family == 0 && stream_ok && ((M <= 2 && stream_rows_ok) || stream_four))) {
        t_kernel = "gemv_stream";
        e = kq::launch_gemv_stream(a, t_gemv, s);
        return e == hipSuccess ? BPK_OK : hip_fail(e, t_kernel);
    }
    // automatic choice: M <= 2 on the VALU row kernel (the 4x4x4 MFMA does not
    // overlap with VALU work on this part), M = 3..16 on the matrix-core row kernel
    const bool use_rows = rows_ok && (t_family == 2 || (t_family == 0 && (M <= 2 || !mrow_ok)));
    const bool use_mrow = mrow_ok && !use_rows && (t_family == 0 || t_family == 3);
    if (use_rows) {
        const bool take = fold && kq::gemv_rows_can_fold(a, *fold);
        t_kernel = take ? "gemv_rows_argmax" : "gemv_rows";
        e = kq::launch_gemv_rows(a, st->split, t_gemv, s, take ? fold : nullptr);
        if (take && e == hipSuccess) *folded = true;
    } else if (use_mrow) {
        t_kernel = "mrow";
        e = kq::launch_mrow(a, st->split, t_gemv, nullptr, nullptr, 1, 0, s);
    } else {
        t_kernel = "generic";
        e = kq::launch_matmul_generic(a, s);
    }
    return e == hipSuccess ? BPK_OK : hip_fail(e, t_kernel);
}

int bpk_kq_matmul(int type, const float* X, const void* W, const float* bias, float* Y, uint32_t M, uint32_t N,
                  uint32_t K, uint32_t n_blocks, uint32_t row_stride_words, uint32_t y_offset, void* stream)
{
    return matmul_impl(type, X, W, bias, Y, M, N, K, n_blocks, row_stride_words, y_offset, stream, nullptr, nullptr);
}

size_t bpk_kq_matmul_fused_workspace_bytes(uint32_t M, uint32_t N, uint32_t K)
{
    // the prologue's output [M, K] and the matmul's own output: [M, N], or [M, 2N] in front of an epilogue
    const size_t x = ((size_t)M * K * sizeof(float) + 255u) & ~(size_t)255u;
    return x + 2u * (size_t)M * N * sizeof(float);
}

int bpk_kq_matmul_fused(int type, const float* X, const void* W, const float* bias, float* Y, uint32_t M, uint32_t N,
                        uint32_t K, uint32_t n_blocks, uint32_t row_stride_words, uint32_t y_offset,
                        const bpk_kq_fusion* f, void* workspace, size_t workspace_bytes, void* stream)
{
    if (!f) return fail(BPK_ERR_NULL, "fusion descriptor must be non-null");
    if (f->prologue < BPK_PRO_NONE || f->prologue > BPK_PRO_GELU_MUL)
        return fail(BPK_ERR_SHAPE, "prologue %d unknown", f->prologue);
    if (f->epilogue != BPK_EPI_NONE && f->epilogue != BPK_EPI_SILU_MUL && f->epilogue != BPK_EPI_GELU_MUL)
        return fail(BPK_ERR_SHAPE, "epilogue %d unknown", f->epilogue);
    if (f->prologue == BPK_PRO_RMS_NORM && !f->norm_w) return fail(BPK_ERR_NULL, "norm_w must be non-null for the norm prologue");
    const bool epi = f->epilogue != BPK_EPI_NONE;
    if (epi && f->residual) return fail(BPK_ERR_SHAPE, "an epilogue takes no residual");
    if (epi && N > 0x7FFFFFFFu) return fail(BPK_ERR_SHAPE, "N too large");
    if (f->prologue == BPK_PRO_NONE && !f->residual && !epi)
        return bpk_kq_matmul(type, X, W, bias, Y, M, N, K, n_blocks, row_stride_words, y_offset, stream);
    const uint32_t w_rows = epi ? 2u * N : N;   // rows of W
    if (int rc = check_matmul(type, X, W, Y, M, w_rows, K, n_blocks, row_stride_words)) return rc;
    if (((uintptr_t)f->norm_w | (uintptr_t)f->residual) & 3u) return fail(BPK_ERR_ALIGN, "norm_w and residual must be 4-byte aligned");
    if (M == 0) return BPK_OK;
    DeviceState* st;
    if (int rc = current_state(&st)) return rc;
    hipStream_t s = (hipStream_t)stream;
    kq::MatmulArgs a{};
    a.type = type; a.X = X; a.W = (const uint8_t*)W; a.bias = bias; a.Y = Y;
    a.M = M; a.N = w_rows; a.K = K; a.n_blocks = n_blocks;
    a.row_stride_bytes = row_stride_words * 4u;
    a.y_offset = y_offset;
    a.ldy = N;
    // one launch where the lanes-along-K kernel takes the shape
    if (!t_fused_separate && (t_family == 0 || t_family == 5)) {
        a.pro = f->prologue; a.norm_w = f->norm_w; a.eps = f->eps; a.residual = f->residual; a.epi = f->epilogue;
        if (kq::gemv_stream_supported(a) && w_rows <= 32768u) {
            t_kernel = "gemv_stream_fused";
            const hipError_t e = kq::launch_gemv_stream(a, t_gemv, s);
            return e == hipSuccess ? BPK_OK : hip_fail(e, t_kernel);
        }
        if (t_family == 5) return fail(BPK_ERR_SHAPE, "lanes-along-K GEMV cannot serve this call");
    }
    // verify batches: one launch of the tile kernel
    if (!t_fused_separate && (t_family == 0 || t_family == 6)) {
        a.pro = f->prologue; a.norm_w = f->norm_w; a.eps = f->eps; a.residual = f->residual; a.epi = f->epilogue;
        if (kq::mtile_fused_supported(a)) {
            t_kernel = "mtile_fused";
            const hipError_t e = kq::launch_mtile_fused(a, st->split, s);
            return e == hipSuccess ? BPK_OK : hip_fail(e, t_kernel);
        }
        if (t_family == 6) return fail(BPK_ERR_SHAPE, "16x16 tile kernel cannot serve this call");
    }
    // otherwise the same function in up to three launches through the caller's workspace
    const size_t x_bytes = ((size_t)M * K * sizeof(float) + 255u) & ~(size_t)255u;
    const bool need_x = f->prologue != BPK_PRO_NONE, need_y = f->residual != nullptr || epi;
    const size_t need = (need_x ? x_bytes : 0) + (need_y ? (size_t)M * w_rows * sizeof(float) : 0);
    if (!workspace || workspace_bytes < need || ((uintptr_t)workspace & 15u))
        return fail(BPK_ERR_WORKSPACE, "this shape needs a 16-byte aligned workspace of %zu bytes (given %zu)", need,
                    workspace ? workspace_bytes : (size_t)0);
    float* wx = (float*)workspace;
    float* wy = (float*)((uint8_t*)workspace + (need_x ? x_bytes : 0));
    if (need_x) {
        const hipError_t e = kq::launch_prologue_rows(f->prologue, X, f->norm_w, f->eps, M, K, wx, s);
        if (e != hipSuccess) return hip_fail(e, "prologue_rows");
    }
    if (int rc = bpk_kq_matmul(type, need_x ? wx : X, W, bias, need_y ? wy : Y, M, w_rows, K, n_blocks, row_stride_words,
                               need_y ? 0u : y_offset, stream))
        return rc;
    if (epi) {
        // act(gate) * up of the [M, 2N] product rows -> Y rows (N apart, at y_offset)
        const hipError_t e = kq::launch_prologue_rows(f->epilogue, wy, nullptr, 0.0f, M, N, Y + y_offset, s);
        if (e != hipSuccess) return hip_fail(e, "act_mul_rows");
    } else if (need_y) {
        const hipError_t e = kq::launch_add_residual(wy, f->residual, Y, M, N, N, y_offset, s);
        if (e != hipSuccess) return hip_fail(e, "add_residual");
    }
    return BPK_OK;
}

int bpk_prefill_rows_bf16(int prologue, const float* X, const float* norm_w, float eps, uint32_t M, uint32_t K,
                          uint16_t* out, void* stream)
{
    if (prologue < BPK_PRO_NONE || prologue > BPK_PRO_GELU_MUL) return fail(BPK_ERR_SHAPE, "unknown prologue");
    if (!X || !out) return fail(BPK_ERR_NULL, "X and out are required");
    if (prologue == BPK_PRO_RMS_NORM && !norm_w) return fail(BPK_ERR_NULL, "BPK_PRO_RMS_NORM needs norm_w");
    if (K == 0) return fail(BPK_ERR_SHAPE, "K must be positive");
    if (M > 65535u && prologue != BPK_PRO_RMS_NORM) return fail(BPK_ERR_SHAPE, "at most 65535 rows per call");
    if (M == 0) return BPK_OK;
    if (int rc = current_state(nullptr)) return rc;
    t_kernel = "prefill_rows_bf16";
    const hipError_t e = kq::launch_prologue_rows_bf16(prologue, X, norm_w, eps, M, K, out, (hipStream_t)stream);
    return e == hipSuccess ? BPK_OK : hip_fail(e, t_kernel);
}

int bpk_kq_matmul_bf16(int type, const uint16_t* X, const void* W, const float* bias, float* Y, uint32_t M,
                       uint32_t N, uint32_t K, uint32_t n_blocks, uint32_t row_stride_words, void* stream)
{
    if (int rc = check_matmul(type, X, W, Y, M, N, K, n_blocks, row_stride_words)) return rc;
    if (M == 0) return BPK_OK;
    DeviceState* st = nullptr;
    if (int rc = current_state(&st)) return rc;
    kq::MatmulArgs a{};
    a.type = type; a.X = X; a.W = (const uint8_t*)W; a.bias = bias; a.Y = Y;
    a.M = M; a.N = N; a.K = K; a.n_blocks = n_blocks;
    a.row_stride_bytes = row_stride_words * 4u;
    a.y_offset = 0;
    a.ldy = N;
    if (!kq::gemm_bf16_supported(a))
        return fail(BPK_ERR_ALIGN, "bf16 GEMM needs 16-byte aligned X and (for Q4_K) 16-byte aligned W rows");
    t_kernel = "gemm_bf16";
    hipError_t e = kq::launch_gemm_bf16(a, t_gemm_tile, t_gemm_split, st->gemm_split, (hipStream_t)stream);
    return e == hipSuccess ? BPK_OK : hip_fail(e, t_kernel);
}

int bpk_kq_dequant_rows(int type, const void* W, uint32_t row_stride_words, const int32_t* rows, uint32_t M,
                        uint32_t K, float* out, void* stream)
{
    if (!known_type(type)) return fail(BPK_ERR_TYPE, "unsupported GGUF type %d", type);
    if (!W || !out) return fail(BPK_ERR_NULL, "W and out must be non-null");
    if (K == 0 || K % KQ_QK) return fail(BPK_ERR_SHAPE, "K=%u is not a positive multiple of 256", K);
    if ((uint64_t)row_stride_words * 4u < (uint64_t)(K / KQ_QK) * kq::block_bytes(type))
        return fail(BPK_ERR_SHAPE, "row_stride_words=%u is smaller than a row", row_stride_words);
    if (M == 0) return BPK_OK;
    if (int rc = current_state(nullptr)) return rc;
    hipError_t e = kq::launch_dequant_rows(type, (const uint8_t*)W, row_stride_words * 4u, rows, M, K, out,
                                           (hipStream_t)stream);
    return e == hipSuccess ? BPK_OK : hip_fail(e, "dequant_rows");
}

int bpk_kq_moe_matmul(int type, const float* X, const void* W, const uint32_t* expert_idx, float* Y, uint32_t T,
                      uint32_t k, uint32_t n_experts, uint32_t N, uint32_t K, uint32_t n_blocks,
                      uint32_t row_stride_words, int x_per_slot, void* stream)
{
    if (int rc = check_matmul(type, X, W, Y, T, N, K, n_blocks, row_stride_words)) return rc;
    if (!expert_idx) return fail(BPK_ERR_NULL, "expert_idx must be non-null");
    if (k == 0 || n_experts == 0) return fail(BPK_ERR_SHAPE, "k and n_experts must be positive");
    if ((uint64_t)T * k > 0xFFFFFFFFull) return fail(BPK_ERR_SHAPE, "T*k overflows");
    if (T == 0) return BPK_OK;
    DeviceState* st;
    if (int rc = current_state(&st)) return rc;
    kq::MatmulArgs a{};
    a.type = type; a.X = X; a.W = (const uint8_t*)W; a.bias = nullptr; a.Y = Y;
    a.M = T * k; a.N = N; a.K = K; a.n_blocks = n_blocks;
    a.row_stride_bytes = row_stride_words * 4u;
    a.y_offset = 0;
    a.ldy = N;
    a.expert_idx = expert_idx;
    a.k_slots = k;
    a.x_per_slot = x_per_slot;
    hipStream_t s = (hipStream_t)stream;
    const int sets = kq::moe_sets_for(T * k, n_experts);
    hipError_t e;
    // two or more pairs per expert on average: records of 8 pairs on the 16x16 tile kernel
    const bool dense = (uint64_t)T * k >= 2ull * n_experts;
    const bool tile_ok = (t_family == 0 || t_family == 6) && kq::mtile_supported(a) && N >= 128u && n_experts <= 8192u &&
                         kq::moe_tiles_bound(T * k, n_experts, 4) <= 65535u &&
                         kq::moe_tiles_words(T * k, n_experts, 4) <= kMoeWords;
    // a handful of pairs (decode): one lanes-along-K matvec per pair, no grouping pass
    const bool stream_path = (t_family == 0 || t_family == 5) && !(tile_ok && dense) && (uint64_t)T * k <= 64u &&
                             kq::gemv_stream_supported(a);
    // (Q5_K has no matrix-core row kernel: its thinly spread pairs take the tile kernel too)
    const bool tile_path = tile_ok && !stream_path && (dense || !kq::mrow_supported(a));
    if (stream_path) {
        t_kernel = "stream_grouped";
        e = kq::launch_gemv_stream(a, t_gemv, s);
    } else if (tile_path) {
        t_kernel = "mtile_grouped";
        uint32_t* n_tiles = st->moe_tiles;
        uint32_t* tiles = st->moe_tiles + 1;
        e = kq::launch_moe_group(expert_idx, T * k, n_experts, 4, tiles, n_tiles, s);
        if (e == hipSuccess)
            e = kq::launch_mtile_grouped(a, tiles, n_tiles, kq::moe_tiles_bound(T * k, n_experts, 4), 8, s);
    } else if (t_family != 1 && kq::mrow_supported(a) && n_experts <= 8192u &&
        kq::moe_tiles_bound(T * k, n_experts, sets) <= 65535u &&
        kq::moe_tiles_words(T * k, n_experts, sets) <= kMoeWords) {
        t_kernel = "mrow_grouped";
        uint32_t* n_tiles = st->moe_tiles;
        uint32_t* tiles = st->moe_tiles + 1;
        e = kq::launch_moe_group(expert_idx, T * k, n_experts, sets, tiles, n_tiles, s);
        if (e == hipSuccess)
            e = kq::launch_mrow(a, st->split, t_gemv, tiles, n_tiles, kq::moe_tiles_bound(T * k, n_experts, sets), sets, s);
    } else {
        t_kernel = "generic_indirect";
        e = kq::launch_matmul_generic(a, s);
    }
    return e == hipSuccess ? BPK_OK : hip_fail(e, t_kernel);
}

struct bpk_chain {
    int device = 0;
    uint32_t n_ops = 0;
    uint32_t max_k = 0;
    kq::ChainOp* d_ops = nullptr;      // n_ops descriptors
    uint32_t* d_words = nullptr;       // n_ops parity words, the arrival counter, the error word
    float* d_mail = nullptr;           // the ops' mailboxes, back to back
    size_t mail_floats = 0;
    // host copies for the check a launch makes of its range of ops
    std::vector<uintptr_t> span;       // per op: x, output and residual ranges, [lo, hi) each (6 words)
    std::vector<uint32_t> x_src;
    std::vector<uint64_t> checked;     // (first << 32 | count) of ranges already found sound
};

namespace {

struct Span {
    uintptr_t lo, hi;   // [lo, hi)
    bool overlaps(const Span& o) const { return lo < o.hi && o.lo < hi; }
    bool inside(const Span& o) const { return lo >= o.lo && hi <= o.hi; }
};

// Words of a fresh chain: every mailbox entry carries parity 0, so the first run writes parity 1.
hipError_t chain_arm(bpk_chain* c)
{
    std::vector<uint32_t> w(c->n_ops + 2u, 1u);
    w[c->n_ops] = 0;        // arrivals
    w[c->n_ops + 1u] = 0;   // error
    hipError_t e = hipMemcpy(c->d_words, w.data(), w.size() * sizeof(uint32_t), hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemset(c->d_mail, 0, c->mail_floats * sizeof(float));
    return e;
}

}  // namespace

int bpk_chain_create(const bpk_chain_op* ops, uint32_t n_ops, bpk_chain** out)
{
    if (!ops || !out) return fail(BPK_ERR_NULL, "ops and out must be non-null");
    if (n_ops == 0 || n_ops > kq::CHAIN_MAX_OPS) return fail(BPK_ERR_SHAPE, "n_ops=%u out of range (1..%u)", n_ops, kq::CHAIN_MAX_OPS);
    DeviceState* st;
    if (int rc = current_state(&st)) return rc;
    std::vector<kq::ChainOp> h(n_ops);
    std::vector<Span> out_span(n_ops), x_span(n_ops), r_span(n_ops);
    std::vector<size_t> mail_at(n_ops);
    uint32_t max_k = 0;
    size_t mail_floats = 0;
    for (uint32_t i = 0; i < n_ops; ++i) {
        const bpk_chain_op& o = ops[i];
        const bpk_kq_fusion& f = o.fusion;
        if (o.type != BPK_TYPE_Q4_K && o.type != BPK_TYPE_Q6_K)
            return fail(BPK_ERR_TYPE, "op %u: a chain takes Q4_K and Q6_K (type %d)", i, o.type);
        if (f.prologue < BPK_PRO_NONE || f.prologue > BPK_PRO_GELU_MUL) return fail(BPK_ERR_SHAPE, "op %u: prologue %d unknown", i, f.prologue);
        if (f.epilogue != BPK_EPI_NONE && f.epilogue != BPK_EPI_SILU_MUL && f.epilogue != BPK_EPI_GELU_MUL)
            return fail(BPK_ERR_SHAPE, "op %u: epilogue %d unknown", i, f.epilogue);
        const bool epi = f.epilogue != BPK_EPI_NONE;
        if (epi && f.residual) return fail(BPK_ERR_SHAPE, "op %u: an epilogue takes no residual", i);
        if (epi && o.N > 0x7FFFFFFFu) return fail(BPK_ERR_SHAPE, "op %u: N too large", i);
        if (f.prologue == BPK_PRO_RMS_NORM && !f.norm_w) return fail(BPK_ERR_NULL, "op %u: norm_w must be non-null for the norm prologue", i);
        const uint32_t w_rows = epi ? 2u * o.N : o.N;
        if (int rc = check_matmul(o.type, o.X, o.W, o.Y, 1, w_rows, o.K, o.n_blocks, o.row_stride_words)) return rc;
        if (((uintptr_t)o.X | (uintptr_t)f.norm_w) & 15u) return fail(BPK_ERR_ALIGN, "op %u: X and norm_w must be 16-byte aligned", i);
        if (o.type == BPK_TYPE_Q4_K && (((uintptr_t)o.W & 15u) || ((o.row_stride_words * 4u) & 15u)))
            return fail(BPK_ERR_ALIGN, "op %u: Q4_K rows must be 16-byte aligned", i);
        const int mode = kq::chain_mode_for(o.type, o.n_blocks, f.epilogue);
        if (mode < 0)
            return fail(BPK_ERR_SHAPE, "op %u: a chain has no kernel form for type %d with K=%u%s", i, o.type, o.K,
                        epi ? " and an epilogue" : "");
        const size_t x_len = (f.prologue >= BPK_PRO_SILU_MUL ? 2u : 1u) * (size_t)o.K;
        x_span[i] = Span{(uintptr_t)o.X, (uintptr_t)(o.X + x_len)};
        out_span[i] = Span{(uintptr_t)(o.Y + o.y_offset), (uintptr_t)(o.Y + o.y_offset + o.N)};
        r_span[i] = f.residual ? Span{(uintptr_t)(f.residual + o.y_offset), (uintptr_t)(f.residual + o.y_offset + o.N)} : Span{0, 0};
        kq::ChainOp& d = h[i];
        d = kq::ChainOp{};
        d.W = (const uint8_t*)o.W; d.X = o.X; d.bias = o.bias; d.Y = o.Y;
        d.norm_w = f.prologue == BPK_PRO_RMS_NORM ? f.norm_w : nullptr;
        d.residual = f.residual;
        d.x_src = d.res_src = kq::CHAIN_NO_SRC;
        d.N = w_rows; d.K = o.K; d.n_blocks = o.n_blocks; d.row_stride_bytes = o.row_stride_words * 4u;
        d.y_offset = o.y_offset;
        d.pro = (uint32_t)f.prologue; d.epi = (uint32_t)f.epilogue; d.eps = f.eps;
        d.mode = (uint32_t)mode;
        if (o.K > max_k) max_k = o.K;
        mail_at[i] = mail_floats;
        mail_floats += ((size_t)o.N + 63u) & ~(size_t)63u;
        // who writes what this op reads: the latest earlier op whose outputs overlap the range
        for (int pass = 0; pass < 2; ++pass) {
            const Span& rd = pass == 0 ? x_span[i] : r_span[i];
            if (rd.lo == rd.hi) continue;
            for (uint32_t j = i; j-- > 0;) {
                if (!rd.overlaps(out_span[j])) continue;
                const size_t delta = (rd.lo - out_span[j].lo) / sizeof(float);
                if (!rd.inside(out_span[j]) || (pass == 0 && (delta & 1u)))
                    return fail(BPK_ERR_SHAPE, "op %u reads part of the outputs of op %u: an input must lie inside one earlier "
                                "op's outputs (at an even element) or outside all of them", i, j);
                if (pass == 0) { d.x_src = j; d.x_mail = (const float*)0 + mail_at[j] + delta; }
                else { d.res_src = j; d.res_mail = (const float*)0 + mail_at[j] + delta; }
                break;
            }
        }
    }
    if (max_k > kq::CHAIN_MAX_K || kq::chain_lds_bytes(max_k) > kq::CHAIN_MAX_LDS)
        return fail(BPK_ERR_SHAPE, "K=%u exceeds what a workgroup can stage (K <= %u)", max_k, kq::CHAIN_MAX_K);
    bpk_chain* c = new (std::nothrow) bpk_chain;
    if (!c) return fail(BPK_ERR_SHAPE, "out of host memory");
    (void)hipGetDevice(&c->device);
    c->n_ops = n_ops;
    c->max_k = max_k;
    c->mail_floats = mail_floats;
    c->span.resize((size_t)n_ops * 6u);
    c->x_src.resize(n_ops);
    for (uint32_t i = 0; i < n_ops; ++i) {
        uintptr_t* w = &c->span[(size_t)i * 6u];
        w[0] = x_span[i].lo; w[1] = x_span[i].hi; w[2] = out_span[i].lo; w[3] = out_span[i].hi; w[4] = r_span[i].lo; w[5] = r_span[i].hi;
        c->x_src[i] = h[i].x_src;
    }
    hipError_t e = hipMalloc((void**)&c->d_ops, n_ops * sizeof(kq::ChainOp));
    if (e == hipSuccess) e = hipMalloc((void**)&c->d_words, (n_ops + 2u) * sizeof(uint32_t));
    if (e == hipSuccess) e = hipMalloc((void**)&c->d_mail, mail_floats * sizeof(float));
    if (e == hipSuccess) {
        for (uint32_t i = 0; i < n_ops; ++i) {
            h[i].y_mail = c->d_mail + mail_at[i];
            if (h[i].x_src != kq::CHAIN_NO_SRC) h[i].x_mail = c->d_mail + (h[i].x_mail - (const float*)0);
            if (h[i].res_src != kq::CHAIN_NO_SRC) h[i].res_mail = c->d_mail + (h[i].res_mail - (const float*)0);
        }
        e = hipMemcpy(c->d_ops, h.data(), n_ops * sizeof(kq::ChainOp), hipMemcpyHostToDevice);
    }
    if (e == hipSuccess) e = chain_arm(c);
    if (e != hipSuccess) {
        (void)hipFree(c->d_ops);
        (void)hipFree(c->d_words);
        (void)hipFree(c->d_mail);
        delete c;
        return hip_fail(e, "creating a chain");
    }
    *out = c;
    return BPK_OK;
}

int bpk_chain_run(bpk_chain* c, uint32_t first, uint32_t count, void* stream)
{
    if (!c) return fail(BPK_ERR_NULL, "chain must be non-null");
    if (count == 0) return BPK_OK;
    if (first >= c->n_ops || count > c->n_ops - first)
        return fail(BPK_ERR_SHAPE, "ops [%u, %u + %u) outside the chain's %u", first, first, count, c->n_ops);
    if (count > kq::CHAIN_MAX_PER_LAUNCH) return fail(BPK_ERR_SHAPE, "a launch walks at most %u ops (asked for %u)", kq::CHAIN_MAX_PER_LAUNCH, count);
    int dev = -1;
    (void)hipGetDevice(&dev);
    if (dev != c->device) return fail(BPK_ERR_DEVICE, "the chain was created on device %d, current is %d", c->device, dev);
    // What an op overwrites must not be in use by an earlier op of the same launch that may still be running
    // somewhere.  An op starts once the whole mailbox of the op that writes its X is filled, which every
    // reader and writer of that op's buffers precedes; so the ops ordered before op i are the chain of its
    // X's producers inside the launch, and only those may share a buffer with its output.
    const uint64_t key = ((uint64_t)first << 32) | count;
    bool known = false;
    for (uint64_t k : c->checked) known = known || k == key;
    if (!known) {
        auto overlap = [](const uintptr_t* a, const uintptr_t* b) { return a[0] < b[1] && b[0] < a[1]; };
        for (uint32_t i = first + 1u; i < first + count; ++i) {
            const uintptr_t* wi = &c->span[(size_t)i * 6u];
            for (uint32_t k = first; k < i; ++k) {
                const uintptr_t* wk = &c->span[(size_t)k * 6u];
                if (!(overlap(wi + 2, wk) || overlap(wi + 2, wk + 2) || (wk[5] && overlap(wi + 2, wk + 4)))) continue;
                bool ordered = false;
                for (uint32_t j = c->x_src[i]; j != kq::CHAIN_NO_SRC && j >= k && j >= first; j = c->x_src[j])
                    if (j == k) { ordered = true; break; }
                if (!ordered)
                    return fail(BPK_ERR_SHAPE, "op %u writes a buffer that op %u of the same launch reads or writes, and nothing "
                                "orders the two (an op follows the ops that lead to its X): launch them separately", i, k);
            }
        }
        if (c->checked.size() < 4096u) c->checked.push_back(key);
    }
    // the hold hook exists for the tests of the give-up path: it is taken only with a short bound on the waits,
    // so that a stray setting cannot make every launch spin for the default two seconds
    if (t_chain_hold && (t_chain_spin_us <= 0 || t_chain_spin_us > 100000))
        return fail(BPK_ERR_SHAPE, "chain_hold is a test hook and needs chain_spin_us set to 1 .. 100000 first");
    kq::ChainLaunch a{};
    a.ops = c->d_ops;
    a.parity = c->d_words;
    a.arrivals = c->d_words + c->n_ops;
    a.error = c->d_words + c->n_ops + 1u;
    a.first = first;
    a.count = count;
    a.max_k = c->max_k;
    a.hold = (uint32_t)t_chain_hold;
    a.ahead = t_chain_ahead > 0 ? (uint32_t)t_chain_ahead - 1u : 0u;   // (measured: touching ahead gains nothing)
    a.trace = (uint64_t*)t_chain_trace;
    a.spin_ticks = (uint64_t)(t_chain_spin_us > 0 ? t_chain_spin_us : 2000000) * 100u;   // 100 MHz wall clock
    t_kernel = "chain";
    const hipError_t e = kq::launch_chain(a, kq::device_cu_count(), (hipStream_t)stream);
    return e == hipSuccess ? BPK_OK : hip_fail(e, t_kernel);
}

int bpk_chain_trace(void* stamps)
{
    t_chain_trace = stamps;
    return BPK_OK;
}

int bpk_chain_status(bpk_chain* c)
{
    if (!c) return fail(BPK_ERR_NULL, "chain must be non-null");
    int dev = -1;
    (void)hipGetDevice(&dev);
    if (dev != c->device) return fail(BPK_ERR_DEVICE, "the chain was created on device %d, current is %d", c->device, dev);
    // every stream of the device, non-blocking ones included: a launch that is still waiting may yet give up
    hipError_t e = hipDeviceSynchronize();
    if (e != hipSuccess) return hip_fail(e, "waiting for the chain's launches");
    uint32_t word = 0;
    e = hipMemcpy(&word, c->d_words + c->n_ops + 1u, sizeof word, hipMemcpyDeviceToHost);
    if (e != hipSuccess) return hip_fail(e, "reading the chain's error word");
    if (word == 0) return BPK_OK;
    return fail(BPK_ERR_TIMEOUT, "a launch of the chain gave up waiting for the inputs of op %u (the grid was not all "
                "resident, or the ops that write them were not part of the launch's past); its outputs are incomplete", word >> 8);
}

int bpk_chain_reset(bpk_chain* c)
{
    if (!c) return fail(BPK_ERR_NULL, "chain must be non-null");
    hipError_t e = hipDeviceSynchronize();
    if (e == hipSuccess) e = chain_arm(c);
    return e == hipSuccess ? BPK_OK : hip_fail(e, "resetting a chain");
}

int bpk_chain_destroy(bpk_chain* c)
{
    if (!c) return BPK_OK;
    hipError_t e = hipFree(c->d_ops);
    const hipError_t e2 = hipFree(c->d_words), e3 = hipFree(c->d_mail);
    delete c;
    if (e == hipSuccess) e = e2;
    if (e == hipSuccess) e = e3;
    return e == hipSuccess ? BPK_OK : hip_fail(e, "hipFree(chain)");
}

int bpk_argmax_rows(const float* logits, uint32_t M, uint32_t N, uint32_t ld, int32_t* out_idx, float* out_val,
                    void* stream)
{
    if (!logits || !out_idx) return fail(BPK_ERR_NULL, "logits and out_idx must be non-null");
    if (N == 0 || ld < N) return fail(BPK_ERR_SHAPE, "N=%u must be positive and ld=%u at least N", N, ld);
    if (M == 0) return BPK_OK;
    DeviceState* st;
    if (int rc = current_state(&st)) return rc;
    float* pv = (float*)st->argmax_scratch;
    uint32_t* pi = st->argmax_scratch + (size_t)kq::ARGMAX_MAX_ROWS * kq::ARGMAX_PARTS;
    uint32_t* tickets = pi + (size_t)kq::ARGMAX_MAX_ROWS * kq::ARGMAX_PARTS;
    const hipError_t e = kq::launch_argmax_rows(logits, M, N, ld, out_idx, out_val, pv, pi, tickets, (hipStream_t)stream);
    return e == hipSuccess ? BPK_OK : hip_fail(e, "argmax_rows");
}

int bpk_argmax_rows_static(const float* logits, uint32_t M, uint32_t N, uint32_t ld, int32_t* out_idx, float* out_val,
                           void* stream)
{
    if (!logits || !out_idx) return fail(BPK_ERR_NULL, "logits and out_idx must be non-null");
    if (N == 0 || ld < N) return fail(BPK_ERR_SHAPE, "N=%u must be positive and ld=%u at least N", N, ld);
    if (M > BPK_ARGMAX_STATIC_MAX_ROWS)
        return fail(BPK_ERR_SHAPE, "M=%u exceeds the %u rows the built-in scratch holds; split the call or use bpk_argmax_rows",
                    M, (unsigned)BPK_ARGMAX_STATIC_MAX_ROWS);
    if (M == 0) return BPK_OK;
    int dev = -1;
    const hipError_t eg = hipGetDevice(&dev);
    if (eg != hipSuccess) return hip_fail(eg, "hipGetDevice");
    uint32_t* base = nullptr;
    if (dev >= 0 && dev < kMaxDevices) {
        std::lock_guard<std::mutex> lk(g_mu);
        if (g_dev[dev].ready) base = g_dev[dev].argmax_static;
    }
    // (never ensure_device here: that allocates)
    if (!base)
        return fail(BPK_ERR_DEVICE, "bpk_init(%d) must have run before bpk_argmax_rows_static: this call allocates nothing", dev);
    float* pv = (float*)base;
    uint32_t* pi = base + (size_t)kq::ARGMAX_MAX_ROWS * kq::ARGMAX_PARTS;
    uint32_t* tickets = pi + (size_t)kq::ARGMAX_MAX_ROWS * kq::ARGMAX_PARTS;
    const hipError_t e = kq::launch_argmax_rows(logits, M, N, ld, out_idx, out_val, pv, pi, tickets, (hipStream_t)stream);
    return e == hipSuccess ? BPK_OK : hip_fail(e, "argmax_rows_static");
}

int bpk_kq_matmul_argmax(int type, const float* X, const void* W, const float* bias, float* logits, uint32_t M,
                         uint32_t N, uint32_t K, uint32_t n_blocks, uint32_t row_stride_words, int32_t* out_idx,
                         float* out_val, void* stream)
{
    if (!out_idx) return fail(BPK_ERR_NULL, "out_idx must be non-null");
    DeviceState* st;
    if (int rc = current_state(&st)) return rc;
    // the row-per-lane kernel (one or two tokens over a vocabulary-sized Q6_K matrix) picks as it stores;
    // other launches are followed by the pick as a launch of its own
    const uint32_t cells = kq::ARGMAX_MAX_ROWS * kq::ARGMAX_PARTS;
    const kq::ArgmaxFold fold{out_idx, out_val, (float*)st->argmax_scratch, st->argmax_scratch + cells,
                              st->argmax_scratch + 2u * (size_t)cells, cells};
    bool folded = false;
    if (int rc = matmul_impl(type, X, W, bias, logits, M, N, K, n_blocks, row_stride_words, 0, stream, &fold, &folded)) return rc;
    if (folded || M == 0) return BPK_OK;
    return bpk_argmax_rows(logits, M, N, N, out_idx, out_val, stream);
}

static int check_route(uint32_t T, uint32_t n_experts, uint32_t k, const void* idx, const void* wt)
{
    if (!idx || !wt) return fail(BPK_ERR_NULL, "idx and wt must be non-null");
    if (n_experts == 0 || n_experts > 1024u) return fail(BPK_ERR_SHAPE, "n_experts=%u out of range (1..1024)", n_experts);
    if (k == 0 || k > 16u || k > n_experts) return fail(BPK_ERR_SHAPE, "k=%u out of range (1..min(16, n_experts))", k);
    if ((uint64_t)T * n_experts > 0xFFFFFFFFull) return fail(BPK_ERR_SHAPE, "T * n_experts too large");
    return BPK_OK;
}

int bpk_moe_topk_softmax(const float* logits, uint32_t T, uint32_t n_experts, uint32_t k, int normalize,
                         uint32_t* idx, float* wt, void* stream)
{
    if (!logits) return fail(BPK_ERR_NULL, "logits must be non-null");
    if (int rc = check_route(T, n_experts, k, idx, wt)) return rc;
    if (T == 0) return BPK_OK;
    DeviceState* st;
    if (int rc = current_state(&st)) return rc;
    t_kernel = "moe_topk_softmax";
    const hipError_t e = kq::launch_topk_softmax(logits, T, n_experts, k, normalize, idx, wt, (hipStream_t)stream);
    return e == hipSuccess ? BPK_OK : hip_fail(e, t_kernel);
}

int bpk_moe_route(const float* X, const float* router_w, uint32_t T, uint32_t hidden, uint32_t n_experts, uint32_t k,
                  int normalize, float* logits, uint32_t* idx, float* wt, void* stream)
{
    if (!X || !router_w) return fail(BPK_ERR_NULL, "X and router_w must be non-null");
    if (int rc = check_route(T, n_experts, k, idx, wt)) return rc;
    if (hidden == 0 || hidden % 4u) return fail(BPK_ERR_SHAPE, "hidden=%u is not a positive multiple of 4", hidden);
    if (((uintptr_t)X | (uintptr_t)router_w) & 15u) return fail(BPK_ERR_ALIGN, "X and router_w must be 16-byte aligned");
    if (T == 0) return BPK_OK;
    DeviceState* st;
    if (int rc = current_state(&st)) return rc;
    t_kernel = "moe_route";
    const hipError_t e = kq::launch_route(X, router_w, T, hidden, n_experts, k, normalize, logits, st->route_logits,
                                          idx, wt, (hipStream_t)stream);
    return e == hipSuccess ? BPK_OK : hip_fail(e, t_kernel);
}

size_t bpk_kq_moe_ffn_scratch_bytes(uint32_t T, uint32_t k, uint32_t hidden, uint32_t inter)
{
    // gate, up (the activation overwrites gate), per-pair down outputs, tile records
    const size_t P = (size_t)T * k;
    return (P * inter * 2 + P * hidden) * sizeof(float) + (P * 10 + 4) * sizeof(uint32_t);
}

int bpk_kq_moe_ffn(int type_gu, int type_dn, const float* X, const void* gate, const void* up, const void* down,
                   const uint32_t* expert_idx, const float* expert_wt, float* out, uint32_t T, uint32_t k,
                   uint32_t n_experts, uint32_t hidden, uint32_t inter, void* scratch, size_t scratch_bytes,
                   void* stream)
{
    if (!known_type(type_gu) || !known_type(type_dn)) return fail(BPK_ERR_TYPE, "unsupported GGUF type (Q4_K=12, Q5_K=13, Q6_K=14)");
    if (!X || !gate || !up || !down || !expert_idx || !expert_wt || !out)
        return fail(BPK_ERR_NULL, "X, gate, up, down, expert_idx, expert_wt and out must be non-null");
    if (k == 0 || n_experts == 0) return fail(BPK_ERR_SHAPE, "k and n_experts must be positive");
    if (hidden == 0 || hidden % KQ_QK || inter == 0 || inter % KQ_QK)
        return fail(BPK_ERR_SHAPE, "hidden=%u and inter=%u must be positive multiples of 256", hidden, inter);
    if ((uint64_t)T * k > 0x0FFFFFFFull) return fail(BPK_ERR_SHAPE, "T*k too large");
    if (T == 0) return BPK_OK;
    if (!scratch || scratch_bytes < bpk_kq_moe_ffn_scratch_bytes(T, k, hidden, inter))
        return fail(BPK_ERR_WORKSPACE, "scratch must hold %zu bytes", bpk_kq_moe_ffn_scratch_bytes(T, k, hidden, inter));
    if ((uintptr_t)scratch & 15u) return fail(BPK_ERR_ALIGN, "scratch must be 16-byte aligned");
    DeviceState* st;
    if (int rc = current_state(&st)) return rc;
    hipStream_t s = (hipStream_t)stream;
    const uint32_t P = T * k;
    float* G = (float*)scratch;
    float* U = G + (size_t)P * inter;
    float* D = U + (size_t)P * inter;
    uint32_t* n_tiles = (uint32_t*)(D + (size_t)P * hidden);
    uint32_t* tiles = n_tiles + 4;
    const int sets = kq::moe_sets_for(P, n_experts);
    const uint32_t bound = kq::moe_tiles_bound(P, n_experts, sets);

    uint32_t nb_gu, rs_gu, nb_dn, rs_dn;
    bpk_kq_layout(type_gu, hidden, &nb_gu, &rs_gu);
    bpk_kq_layout(type_dn, inter, &nb_dn, &rs_dn);
    kq::MatmulArgs a{};
    a.type = type_gu; a.X = X; a.W = (const uint8_t*)gate; a.Y = G;
    a.M = P; a.N = inter; a.K = hidden; a.n_blocks = nb_gu; a.row_stride_bytes = rs_gu * 4u; a.ldy = inter;
    a.expert_idx = expert_idx; a.k_slots = k; a.x_per_slot = 0;
    kq::MatmulArgs d{};
    d.type = type_dn; d.X = G; d.W = (const uint8_t*)down; d.Y = D;
    d.M = P; d.N = hidden; d.K = inter; d.n_blocks = nb_dn; d.row_stride_bytes = rs_dn * 4u; d.ldy = hidden;
    d.expert_idx = expert_idx; d.k_slots = k; d.x_per_slot = 1;
    a.tile_iters = d.tile_iters = (uint32_t)t_moe_tile_iters;
    const bool fast = t_family != 1 && n_experts <= 8192u && bound <= 65535u && kq::mrow_supported(a) &&
                      kq::mrow_supported(d);
    hipError_t e = hipSuccess;
    const uint32_t bound8 = kq::moe_tiles_bound(P, n_experts, 4);
    // Pairs per expert from which the tile kernel's records (every touched expert's matrices read once per record
    // of pairs) beat one lanes-along-K matvec per pair.  Measured on 128 experts x 8 slots, 2048 / 768: 128 pairs 119
    // against 104 us, 160 pairs 142 against 150-159, 192 pairs 145 against 179.
    const bool dense = 4ull * P >= 5ull * n_experts;
    const bool tile_ok = (t_family == 0 || t_family == 6) && n_experts <= 8192u && bound8 <= 65535u && inter >= 128u &&
                         hidden >= 128u && kq::mtile_supported(a) && kq::mtile_supported(d);
    const bool stream_path = (t_family == 0 || t_family == 5) && !(tile_ok && dense) && P <= 256u &&
                             kq::gemv_stream_supported(a) && kq::gemv_stream_supported(d);
    // (Q5_K has no matrix-core row kernel: its thinly spread pairs take the tile kernel too)
    const bool tile_path = tile_ok && !stream_path && (dense || !fast);
    if (stream_path) {
        // a handful of pairs (decode): one lanes-along-K matvec per pair, no grouping pass
        // gate and up in one launch (they read the same x), the activation folded into down's load of x
        t_kernel = "moe_ffn_stream";
        a.W2 = (const uint8_t*)up; a.Y2 = U;
        e = kq::launch_gemv_stream(a, t_gemv, s);
        d.X2 = U;
        if (e == hipSuccess && t_moe_fold && kq::stream_combine_supported(d, T)) {
            // ... and the weighted sum over the slots into down's launch: its waves are a token's slots
            e = kq::launch_stream_combine(d, expert_wt, out, T, t_gemv, s);
            return e == hipSuccess ? BPK_OK : hip_fail(e, t_kernel);
        }
        if (e == hipSuccess) e = kq::launch_gemv_stream(d, t_gemv, s);
    } else if (tile_path) {
        // two or more pairs per expert on average: records of 8 pairs (16 from four pairs per expert on),
        // every expert matrix read once per record (Q6_K: once per 8 pairs of it)
        t_kernel = "moe_ffn_mtile";
        const bool wide = (uint64_t)P >= 4ull * n_experts && kq::moe_tiles_bound(P, n_experts, 8) <= 65535u;
        const int rsets = wide ? 8 : 4;
        const uint32_t rbound = kq::moe_tiles_bound(P, n_experts, rsets), rcap = 2u * (uint32_t)rsets;
        e = kq::launch_moe_group(expert_idx, P, n_experts, rsets, tiles, n_tiles, s);
        a.W2 = (const uint8_t*)up;
        if (t_moe_fold && kq::mtile_grouped_dual_supported(a)) {
            // gate and up in one launch that converts the records' X once and stores silu(gate x) * (up x)
            if (e == hipSuccess) e = kq::launch_mtile_grouped(a, tiles, n_tiles, rbound, rcap, s);
        } else {
            a.W2 = nullptr;
            if (e == hipSuccess) e = kq::launch_mtile_grouped(a, tiles, n_tiles, rbound, rcap, s);
            a.W = (const uint8_t*)up; a.Y = U;
            if (e == hipSuccess) e = kq::launch_mtile_grouped(a, tiles, n_tiles, rbound, rcap, s);
            if (e == hipSuccess) e = kq::launch_moe_silu_mul(G, U, G, (size_t)P * inter, s);
        }
        if (e == hipSuccess) e = kq::launch_mtile_grouped(d, tiles, n_tiles, rbound, rcap, s);
    } else if (fast) {
        t_kernel = "moe_ffn_mrow";
        e = kq::launch_moe_group(expert_idx, P, n_experts, sets, tiles, n_tiles, s);
        if (e == hipSuccess) e = kq::launch_mrow(a, st->split, t_gemv, tiles, n_tiles, bound, sets, s);
        a.W = (const uint8_t*)up; a.Y = U;
        if (e == hipSuccess) e = kq::launch_mrow(a, st->split, t_gemv, tiles, n_tiles, bound, sets, s);
        if (e == hipSuccess) e = kq::launch_moe_silu_mul(G, U, G, (size_t)P * inter, s);
        if (e == hipSuccess) e = kq::launch_mrow(d, st->split, t_gemv, tiles, n_tiles, bound, sets, s);
    } else {
        t_kernel = "moe_ffn_generic";
        e = kq::launch_matmul_generic(a, s);
        a.W = (const uint8_t*)up; a.Y = U;
        if (e == hipSuccess) e = kq::launch_matmul_generic(a, s);
        if (e == hipSuccess) e = kq::launch_moe_silu_mul(G, U, G, (size_t)P * inter, s);
        if (e == hipSuccess) e = kq::launch_matmul_generic(d, s);
    }
    if (e == hipSuccess) e = kq::launch_moe_combine(D, expert_wt, out, T, k, hidden, s);
    return e == hipSuccess ? BPK_OK : hip_fail(e, t_kernel);
}

}  // extern "C"
