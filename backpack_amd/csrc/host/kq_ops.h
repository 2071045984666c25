// kq_ops.h — C++ host layer over the C ABI, shaped like the reference's k-quant
// operator interface so that a ModelRunner-style caller can switch to it:
//
//   KQuantPacked, pack_q4k/q5k/q6k       runtime/gguf_loader.h:108-124
//   GGUFFile and its getters             runtime/gguf_loader.h:49-86
//   GPUBuffer {handle, size, offset}     runtime/gpu_context.h:47-51 (non-owning view)
//   uploadKQWeight, fuseKQ               runtime/model_runner.cpp:958-963, :1002-1012
//   makeKQParams  P = {K,N,nBlocks,rowStrideWords,yOffset}   runtime/model_runner.cpp:2404-2413
//   Dispatch {pipeline, bindGroup, gx,gy,gz, name}           runtime/gpu_context.h:36-44
//
// A KQDispatch is the counterpart of one recorded dispatch: the binding set
// {0:X 1:W 2:Bias 3:Y 4:P} plus M, replayed with run(stream).  Kernel choice
// (the reference's kqPipelineFor / mmk) happens inside the library.  Errors
// follow the reference's convention: a message on stderr and an early return;
// run() additionally returns the library's status code.
#pragma once
#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

#include "../../../include/bpk_kquant.h"

namespace bp {

enum GGUFType : uint32_t { GGUF_TYPE_Q4_K = BPK_TYPE_Q4_K, GGUF_TYPE_Q5_K = BPK_TYPE_Q5_K, GGUF_TYPE_Q6_K = BPK_TYPE_Q6_K };

struct KQuantPacked {
    std::vector<uint32_t> data;   // raw block data as u32 words, rows padded to 4 bytes
    uint32_t N = 0, K = 0;        // output rows, input columns
    uint32_t rowStrideWords = 0;
    uint32_t nBlocks = 0;
    GGUFType type = GGUF_TYPE_Q4_K;
};

KQuantPacked pack_q4k(const void* raw_data, uint32_t N, uint32_t K);
KQuantPacked pack_q5k(const void* raw_data, uint32_t N, uint32_t K);
KQuantPacked pack_q6k(const void* raw_data, uint32_t N, uint32_t K);

// Row-wise concatenation of packed matrices with equal K and type (q|k|v, gate|up).
KQuantPacked fuseKQ(const std::vector<const KQuantPacked*>& parts);

struct GPUBuffer {
    void* handle = nullptr;   // device allocation
    size_t size = 0;
    size_t offset = 0;        // bind offset in bytes
    void* ptr() const { return handle ? (char*)handle + offset : nullptr; }
};

GPUBuffer createBuffer(const std::string& name, size_t bytes);
void writeBuffer(const GPUBuffer& b, const void* src, size_t bytes);
void readBuffer(const GPUBuffer& b, void* dst, size_t bytes);   // synchronises the device
void releaseBuffer(GPUBuffer& b);

// Packed rows are fetched in 16-byte pieces and Q6_K blocks are 210 bytes, so a Q6_K weight must stay readable
// for this many bytes behind its last row (include/bpk_kquant.h, bpk_kq_matmul).  uploadKQWeight allocates and
// zeroes them; a buffer made some other way has to provide them itself.
constexpr size_t KQ_WEIGHT_TAIL_BYTES = 16;
GPUBuffer uploadKQWeight(const std::string& name, const KQuantPacked& w);
// Host-side check every dispatch below runs before it launches: the view W must hold `rows` packed rows and,
// for Q6_K, the readable tail.  Returns BPK_OK or BPK_ERR_SHAPE (message on stderr); touches no device.
int checkKQWeightView(GGUFType type, const GPUBuffer& W, uint32_t rows, uint32_t rowStrideWords, const std::string& name);

struct KQParams { uint32_t v[5]; };
inline KQParams makeKQParams(uint32_t K, uint32_t N, uint32_t nBlocks, uint32_t rowStride, uint32_t yOffset = 0)
{
    return KQParams{{K, N, nBlocks, rowStride, yOffset}};
}

struct KQDispatch {
    GGUFType type;
    GPUBuffer X, W, Bias, Y;   // Bias.handle == nullptr binds zeros
    KQParams P;
    uint32_t M = 1;
    std::string name;
    int run(void* stream = nullptr) const;
};

// The dispatch group around a decode matvec as one dispatch: RMSNorm of X (NormW bound, eps set), or
// act(gate) * up with X bound to the fused gate|up buffer, and Residual added to Y (may be Y's buffer).
// Counterpart of the reference's q4k_matmul_norm / q4k_down_gelu binding sets
// (runtime/kernels/quant_kq/q4k_matmul_norm.wgsl:12-22, q4k_down_gelu.wgsl:11-15).
struct KQFusedDispatch {
    KQDispatch base;
    int prologue = BPK_PRO_NONE;
    int epilogue = BPK_EPI_NONE;   // base.W is then gate|up stacked and base.P.v[1] the number of outputs
    GPUBuffer NormW, Residual, Workspace;   // Workspace only for shapes that need separate launches
    float eps = 0.0f;
    int run(void* stream = nullptr) const;
};

// A recorded stretch of the decode dispatch list whose entries are fused k-quant matvecs feeding each other
// (the per-token command buffer, runtime/model_runner.cpp:5725-5759, between two attention blocks): record the
// dispatches once, then run(first, count) issues a range of them as ONE launch.  An entry whose X or Residual is
// the Y of an earlier entry follows it inside the launch.
struct KQChain {
    KQChain() = default;
    KQChain(const KQChain&) = delete;
    KQChain& operator=(const KQChain&) = delete;
    ~KQChain();
    void add(const KQFusedDispatch& d) { ops_.push_back(d); }
    size_t size() const { return ops_.size(); }
    int build();                                                      // after the last add
    int run(uint32_t first, uint32_t count, void* stream = nullptr);  // needs build()
    int status();                                                     // BPK_OK, or what a bounded wait gave up on
    int reset();

private:
    std::vector<KQFusedDispatch> ops_;
    bpk_chain* c_ = nullptr;
};

// Read-only view of a GGUF file with the reference's member names.  Tensor data pointers stay valid
// until the object is destroyed.
struct GGUFTensorInfo {
    std::string name;
    std::vector<uint64_t> shape;
    uint32_t type = 0;
    uint64_t offset = 0;
    const void* data = nullptr;   // host address of the tensor's bytes
    uint64_t bytes = 0;
};

struct GGUFFile {
    uint32_t version = 0;
    uint64_t n_tensors = 0;
    uint64_t data_offset = 0;
    std::vector<GGUFTensorInfo> tensors;

    GGUFFile() = default;
    GGUFFile(const GGUFFile&) = delete;
    GGUFFile& operator=(const GGUFFile&) = delete;
    ~GGUFFile();
    bool open(const std::string& path);
    const GGUFTensorInfo* find(const std::string& name) const;
    std::string getString(const std::string& key, const std::string& def = "") const;
    uint32_t getU32(const std::string& key, uint32_t def = 0) const;
    float getFloat(const std::string& key, float def = 0.0f) const;
    bool getBool(const std::string& key, bool def = false) const;
    bool hasKey(const std::string& key) const;
    // Named k-quant tensors stacked into one device weight (q|k|v, gate|up); W.handle is the library's
    // allocation and is released with releaseWeight.
    bool loadKQWeight(const std::vector<std::string>& names, GPUBuffer& W, KQuantPacked& desc, bpk_weight** owner) const;
    const bpk_gguf* handle() const { return g_; }

private:
    bpk_gguf* g_ = nullptr;
};
void releaseWeight(bpk_weight* owner);

// The model's hyper-parameters with the reference's field names (ModelConfig, runtime/gguf_loader.h:164-218;
// extractModelConfig, runtime/gguf_loader.cpp:184-317).
enum class ActivationType { SiLU, GELU };
enum class AttnLayerType : uint8_t { Global, SlidingWindow };
struct ModelConfig {
    std::string arch;
    uint32_t nLayer = 0, nHead = 0, nKvHeads = 0, nEmbd = 0, intermediateSize = 0, nVocab = 0, headDim = 0, kvHeadDim = 0;
    float rmsNormEps = 1e-6f, ropeTheta = 1e6f;
    bool tieWordEmbeddings = true, hasQkNorm = false;
    ActivationType activation = ActivationType::SiLU;
    float embeddingScale = 0.0f, logitSoftcap = 0.0f;
    uint32_t slidingWindow = 0;
    std::vector<AttnLayerType> layerAttnTypes;
    bool hasSandwichNorm = false;
    uint32_t pleSize = 0, sharedKvLayers = 0;
    bool hasMtp = false;
    uint32_t mtpNumLayers = 0;
    uint32_t numExperts = 0, numExpertsPerTok = 0, moeIntermediateSize = 0, moeSharedIntermediateSize = 0;
    uint32_t ssmInnerSize = 0, ssmStateSize = 0, ssmConvKernel = 0, ssmGroupCount = 0, ssmTimeStepRank = 0,
             fullAttentionInterval = 0;
    std::vector<int32_t> ropeSections = {11, 11, 10, 0};
    // hybrid SSM + attention files: every fullAttentionInterval-th layer is attention (0: all of them)
    bool isAttentionLayer(uint32_t i) const { return fullAttentionInterval == 0 || (i + 1) % fullAttentionInterval == 0; }
};
ModelConfig extractModelConfig(const GGUFFile& gguf);

// Dequantised rows (the q6k_gather / q6k_gather_batched dispatch).
int gatherKQ(GGUFType type, const GPUBuffer& W, uint32_t rowStrideWords, const GPUBuffer& tokens, uint32_t M,
             uint32_t K, const GPUBuffer& out, void* stream = nullptr);

}  // namespace bp
