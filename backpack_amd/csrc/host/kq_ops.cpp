// kq_ops.cpp — see kq_ops.h.  Host-only C++; device work goes through the C ABI.
#include "kq_ops.h"

#include <hip/hip_runtime_api.h>

#include <cstdio>
#include <cstring>

namespace bp {

static KQuantPacked pack(GGUFType type, const void* raw, uint32_t N, uint32_t K)
{
    KQuantPacked r;
    r.N = N; r.K = K; r.type = type;
    if (bpk_kq_layout((int)type, K, &r.nBlocks, &r.rowStrideWords) != BPK_OK) {
        fprintf(stderr, "pack: %s\n", bpk_last_error());
        return r;
    }
    r.data.resize((size_t)N * r.rowStrideWords);
    if (bpk_kq_pack_host((int)type, raw, N, K, r.data.data()) != BPK_OK) fprintf(stderr, "pack: %s\n", bpk_last_error());
    return r;
}

KQuantPacked pack_q4k(const void* raw, uint32_t N, uint32_t K) { return pack(GGUF_TYPE_Q4_K, raw, N, K); }
KQuantPacked pack_q5k(const void* raw, uint32_t N, uint32_t K) { return pack(GGUF_TYPE_Q5_K, raw, N, K); }
KQuantPacked pack_q6k(const void* raw, uint32_t N, uint32_t K) { return pack(GGUF_TYPE_Q6_K, raw, N, K); }

KQuantPacked fuseKQ(const std::vector<const KQuantPacked*>& parts)
{
    KQuantPacked r;
    if (parts.empty()) return r;
    r = *parts[0];
    for (size_t i = 1; i < parts.size(); ++i) {
        const KQuantPacked& p = *parts[i];
        if (p.K != r.K || p.type != r.type || p.rowStrideWords != r.rowStrideWords) {
            fprintf(stderr, "fuseKQ: part %zu has a different K or type\n", i);
            return KQuantPacked{};
        }
        r.data.insert(r.data.end(), p.data.begin(), p.data.end());
        r.N += p.N;
    }
    return r;
}

GPUBuffer createBuffer(const std::string& name, size_t bytes)
{
    GPUBuffer b;
    if (hipMalloc(&b.handle, bytes) != hipSuccess) {
        fprintf(stderr, "createBuffer(%s, %zu) failed\n", name.c_str(), bytes);
        b.handle = nullptr;
        return b;
    }
    b.size = bytes;
    return b;
}

void writeBuffer(const GPUBuffer& b, const void* src, size_t bytes)
{
    if (hipMemcpy(b.ptr(), src, bytes, hipMemcpyHostToDevice) != hipSuccess) fprintf(stderr, "writeBuffer failed\n");
}

void readBuffer(const GPUBuffer& b, void* dst, size_t bytes)
{
    if (hipMemcpy(dst, b.ptr(), bytes, hipMemcpyDeviceToHost) != hipSuccess) fprintf(stderr, "readBuffer failed\n");
}

void releaseBuffer(GPUBuffer& b)
{
    if (b.handle) (void)hipFree(b.handle);
    b = GPUBuffer{};
}

GPUBuffer uploadKQWeight(const std::string& name, const KQuantPacked& w)
{
    // the kernels fetch packed rows in 16-byte pieces: the allocation carries KQ_WEIGHT_TAIL_BYTES readable
    // (zeroed) bytes behind the last row, as bpk_weight_create's does
    const size_t bytes = w.data.size() * sizeof(uint32_t);
    GPUBuffer b = createBuffer(name, bytes + KQ_WEIGHT_TAIL_BYTES);
    if (!b.handle) return b;
    if (bytes) writeBuffer(b, w.data.data(), bytes);
    if (hipMemset((char*)b.handle + bytes, 0, KQ_WEIGHT_TAIL_BYTES) != hipSuccess) fprintf(stderr, "uploadKQWeight(%s): clearing the tail failed\n", name.c_str());
    return b;
}

int checkKQWeightView(GGUFType type, const GPUBuffer& W, uint32_t rows, uint32_t rowStrideWords, const std::string& name)
{
    if (!W.handle) return BPK_OK;   // the library reports the missing pointer
    const size_t need = (size_t)rows * rowStrideWords * sizeof(uint32_t) + (type == GGUF_TYPE_Q6_K ? KQ_WEIGHT_TAIL_BYTES : 0);
    if (W.offset > W.size || W.size - W.offset < need) {
        fprintf(stderr, "[%s] weight view of %zu bytes at offset %zu is smaller than the %zu bytes its %u rows need%s\n",
                name.c_str(), W.size, W.offset, need, rows,
                type == GGUF_TYPE_Q6_K ? " (Q6_K rows are fetched in 16-byte pieces: 16 readable bytes must follow the last row; "
                                         "uploadKQWeight allocates them)" : "");
        return BPK_ERR_SHAPE;
    }
    return BPK_OK;
}

int KQDispatch::run(void* stream) const
{
    if (const int bad = checkKQWeightView(type, W, P.v[1], P.v[3], name)) return bad;
    const int rc = bpk_kq_matmul((int)type, (const float*)X.ptr(), W.ptr(), (const float*)Bias.ptr(), (float*)Y.ptr(), M,
                                 P.v[1], P.v[0], P.v[2], P.v[3], P.v[4], stream);
    if (rc != BPK_OK) fprintf(stderr, "[%s] %s\n", name.c_str(), bpk_last_error());
    return rc;
}

int gatherKQ(GGUFType type, const GPUBuffer& W, uint32_t rowStrideWords, const GPUBuffer& tokens, uint32_t M, uint32_t K,
             const GPUBuffer& out, void* stream)
{
    const int rc = bpk_kq_dequant_rows((int)type, W.ptr(), rowStrideWords, (const int32_t*)tokens.ptr(), M, K,
                                       (float*)out.ptr(), stream);
    if (rc != BPK_OK) fprintf(stderr, "[gatherKQ] %s\n", bpk_last_error());
    return rc;
}

int KQFusedDispatch::run(void* stream) const
{
    const KQDispatch& d = base;
    // with an epilogue W holds gate rows and up rows: twice the outputs
    if (const int bad = checkKQWeightView(d.type, d.W, d.P.v[1] * (epilogue != BPK_EPI_NONE ? 2u : 1u), d.P.v[3], d.name)) return bad;
    bpk_kq_fusion f{prologue, (const float*)NormW.ptr(), eps, (const float*)Residual.ptr(), epilogue};
    const int rc = bpk_kq_matmul_fused((int)d.type, (const float*)d.X.ptr(), d.W.ptr(), (const float*)d.Bias.ptr(),
                                       (float*)d.Y.ptr(), d.M, d.P.v[1], d.P.v[0], d.P.v[2], d.P.v[3], d.P.v[4], &f,
                                       Workspace.ptr(), Workspace.handle ? Workspace.size - Workspace.offset : 0, stream);
    if (rc != BPK_OK) fprintf(stderr, "%s: %s\n", d.name.c_str(), bpk_last_error());
    return rc;
}

KQChain::~KQChain() { bpk_chain_destroy(c_); }

int KQChain::build()
{
    bpk_chain_destroy(c_);
    c_ = nullptr;
    std::vector<bpk_chain_op> ops(ops_.size());
    for (size_t i = 0; i < ops_.size(); ++i) {
        const KQFusedDispatch& f = ops_[i];
        const KQDispatch& d = f.base;
        if (d.M != 1) {
            fprintf(stderr, "%s: a chain takes one token per dispatch\n", d.name.c_str());
            return BPK_ERR_SHAPE;
        }
        if (const int bad = checkKQWeightView(d.type, d.W, d.P.v[1] * (f.epilogue != BPK_EPI_NONE ? 2u : 1u), d.P.v[3], d.name)) return bad;
        ops[i] = bpk_chain_op{(int)d.type, (const float*)d.X.ptr(), d.W.ptr(), (const float*)d.Bias.ptr(), (float*)d.Y.ptr(),
                              d.P.v[1], d.P.v[0], d.P.v[2], d.P.v[3], d.P.v[4],
                              bpk_kq_fusion{f.prologue, (const float*)f.NormW.ptr(), f.eps, (const float*)f.Residual.ptr(),
                                            f.epilogue}};
    }
    const int rc = bpk_chain_create(ops.data(), (uint32_t)ops.size(), &c_);
    if (rc != BPK_OK) fprintf(stderr, "KQChain::build: %s\n", bpk_last_error());
    return rc;
}

int KQChain::run(uint32_t first, uint32_t count, void* stream)
{
    const int rc = c_ ? bpk_chain_run(c_, first, count, stream) : BPK_ERR_NULL;
    if (rc != BPK_OK) fprintf(stderr, "KQChain::run: %s\n", c_ ? bpk_last_error() : "not built");
    return rc;
}

int KQChain::status() { return c_ ? bpk_chain_status(c_) : BPK_ERR_NULL; }
int KQChain::reset() { return c_ ? bpk_chain_reset(c_) : BPK_ERR_NULL; }

GGUFFile::~GGUFFile() { bpk_gguf_close(g_); }

bool GGUFFile::open(const std::string& path)
{
    bpk_gguf_close(g_);
    g_ = nullptr;
    tensors.clear();
    if (bpk_gguf_open(path.c_str(), &g_) != BPK_OK) {
        fprintf(stderr, "GGUFFile::open: %s\n", bpk_last_error());
        return false;
    }
    bpk_gguf_info(g_, &version, &n_tensors, nullptr, &data_offset);
    tensors.resize((size_t)n_tensors);
    for (uint64_t i = 0; i < n_tensors; ++i) {
        bpk_gguf_tensor t;
        bpk_gguf_tensor_at(g_, i, &t);
        GGUFTensorInfo& o = tensors[(size_t)i];
        o.name = t.name;
        o.shape.assign(t.dims, t.dims + t.n_dims);
        o.type = t.type;
        o.offset = t.offset;
        o.data = t.data;
        o.bytes = t.bytes;
    }
    return true;
}

const GGUFTensorInfo* GGUFFile::find(const std::string& name) const
{
    for (const auto& t : tensors)
        if (t.name == name) return &t;
    return nullptr;
}

std::string GGUFFile::getString(const std::string& key, const std::string& def) const
{
    if (!g_ || bpk_gguf_key_type(g_, key.c_str()) != 8) return def;
    size_t n = 0;
    bpk_gguf_get_string(g_, key.c_str(), nullptr, 0, &n);
    std::string s(n, '\0');
    std::vector<char> buf(n + 1);
    bpk_gguf_get_string(g_, key.c_str(), buf.data(), n + 1, nullptr);
    s.assign(buf.data(), n);
    return s;
}

uint32_t GGUFFile::getU32(const std::string& key, uint32_t def) const
{
    uint32_t v = def;
    if (g_) bpk_gguf_get_u32(g_, key.c_str(), def, &v);
    return v;
}

float GGUFFile::getFloat(const std::string& key, float def) const
{
    float v = def;
    if (g_) bpk_gguf_get_f32(g_, key.c_str(), def, &v);
    return v;
}

bool GGUFFile::getBool(const std::string& key, bool def) const
{
    int v = def;
    if (g_) bpk_gguf_get_bool(g_, key.c_str(), def, &v);
    return v != 0;
}

bool GGUFFile::hasKey(const std::string& key) const { return g_ && bpk_gguf_has_key(g_, key.c_str()); }

bool GGUFFile::loadKQWeight(const std::vector<std::string>& names, GPUBuffer& W, KQuantPacked& desc,
                            bpk_weight** owner) const
{
    std::vector<const char*> c;
    for (const auto& n : names) c.push_back(n.c_str());
    if (!g_ || bpk_gguf_weight_create(g_, c.data(), (uint32_t)c.size(), owner) != BPK_OK) {
        fprintf(stderr, "GGUFFile::loadKQWeight: %s\n", g_ ? bpk_last_error() : "file not open");
        return false;
    }
    bpk_weight_desc d;
    bpk_weight_describe(*owner, &d);
    W = GPUBuffer{d.data, d.bytes + KQ_WEIGHT_TAIL_BYTES, 0};   // the library's allocation carries the readable tail
    desc = KQuantPacked{};
    desc.N = d.N; desc.K = d.K; desc.rowStrideWords = d.row_stride_words; desc.nBlocks = d.n_blocks;
    desc.type = (GGUFType)d.type;
    return true;
}

void releaseWeight(bpk_weight* owner) { bpk_weight_destroy(owner); }

ModelConfig extractModelConfig(const GGUFFile& gguf)
{
    ModelConfig cfg;
    bpk_model_config c;
    if (!gguf.handle() || bpk_gguf_model_config(gguf.handle(), &c, nullptr, 0) != BPK_OK) return cfg;
    std::vector<uint8_t> kinds(c.n_layer_attn_types);
    if (!kinds.empty()) bpk_gguf_model_config(gguf.handle(), &c, kinds.data(), (uint32_t)kinds.size());
    cfg.arch = c.arch;
    cfg.nLayer = c.n_layer; cfg.nHead = c.n_head; cfg.nKvHeads = c.n_kv_heads; cfg.nEmbd = c.n_embd;
    cfg.intermediateSize = c.intermediate_size; cfg.nVocab = c.n_vocab; cfg.headDim = c.head_dim; cfg.kvHeadDim = c.kv_head_dim;
    cfg.rmsNormEps = c.rms_norm_eps; cfg.ropeTheta = c.rope_theta;
    cfg.tieWordEmbeddings = c.tie_word_embeddings != 0; cfg.hasQkNorm = c.has_qk_norm != 0;
    cfg.activation = c.activation == BPK_ACT_GELU ? ActivationType::GELU : ActivationType::SiLU;
    cfg.embeddingScale = c.embedding_scale; cfg.logitSoftcap = c.logit_softcap; cfg.slidingWindow = c.sliding_window;
    for (uint8_t k : kinds) cfg.layerAttnTypes.push_back(k ? AttnLayerType::SlidingWindow : AttnLayerType::Global);
    cfg.hasSandwichNorm = c.has_sandwich_norm != 0; cfg.pleSize = c.ple_size; cfg.sharedKvLayers = c.shared_kv_layers;
    cfg.hasMtp = c.has_mtp != 0; cfg.mtpNumLayers = c.mtp_num_layers;
    cfg.numExperts = c.num_experts; cfg.numExpertsPerTok = c.num_experts_per_tok;
    cfg.moeIntermediateSize = c.moe_intermediate_size; cfg.moeSharedIntermediateSize = c.moe_shared_intermediate_size;
    cfg.ssmInnerSize = c.ssm_inner_size; cfg.ssmStateSize = c.ssm_state_size; cfg.ssmConvKernel = c.ssm_conv_kernel;
    cfg.ssmGroupCount = c.ssm_group_count; cfg.ssmTimeStepRank = c.ssm_time_step_rank;
    cfg.fullAttentionInterval = c.full_attention_interval;
    cfg.ropeSections.assign(c.rope_sections, c.rope_sections + 4);
    return cfg;
}

}  // namespace bp
