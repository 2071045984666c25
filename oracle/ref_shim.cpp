// ref_shim.cpp — extern "C" doorway into the reference's own CPU functions.
//
// TEST INFRASTRUCTURE ONLY.  Compiled together with the reference's
// runtime/gguf_loader.cpp, from where that file lies in the reference checkout,
// into oracle/_ref/libbp_ref.so (see the Makefile).  It adds no arithmetic of
// its own: every call forwards to pack_q4k / pack_q6k / dequant_kquant
// (runtime/gguf_loader.h:108-124, :147) so the restatement in kq_oracle.c can
// be compared with the reference as this compiler builds it, and so the
// benchmark can time the reference's real CPU path; the bpref_gguf_* calls
// forward to GGUFFile (runtime/gguf_loader.h:56-86) so the library's container
// reader can be compared with the reference's parser on the same files.
#include "gguf_loader.h"

#include <chrono>
#include <cstring>
#include <vector>

extern "C" {

// Writes N*rowStrideWords words to out (if non-null) and reports the descriptor.
int bpref_pack(int type, const void* raw, uint32_t N, uint32_t K, uint32_t* out,
               uint32_t* n_blocks, uint32_t* row_stride_words)
{
    KQuantPacked p;
    if (type == (int)GGUF_TYPE_Q4_K) p = pack_q4k(raw, N, K);
    else if (type == (int)GGUF_TYPE_Q5_K) p = pack_q5k(raw, N, K);
    else if (type == (int)GGUF_TYPE_Q6_K) p = pack_q6k(raw, N, K);
    else return -1;
    if (n_blocks) *n_blocks = p.nBlocks;
    if (row_stride_words) *row_stride_words = p.rowStrideWords;
    if (out) std::memcpy(out, p.data.data(), p.data.size() * sizeof(uint32_t));
    return 0;
}

int bpref_dequant(int type, const void* raw, float* out, uint32_t N, uint32_t K)
{
    if (type != (int)GGUF_TYPE_Q4_K && type != (int)GGUF_TYPE_Q5_K && type != (int)GGUF_TYPE_Q6_K) return -1;
    dequant_kquant(raw, out, N, K, (GGUFType)type);
    return 0;
}

// The CPU path as the reference's kernel tests run it: dequant_kquant into an
// fp32 matrix, then one sequential fp32 dot per output (kernel_test.cpp:1682).
// Seconds for each leg are returned so the benchmark can report them apart.
int bpref_matmul_timed(int type, const float* X, const void* raw, float* deq,
                       float* Y, uint32_t M, uint32_t N, uint32_t K,
                       double* t_dequant, double* t_dot)
{
    using clk = std::chrono::steady_clock;
    if (type != (int)GGUF_TYPE_Q4_K && type != (int)GGUF_TYPE_Q6_K) return -1;
    auto t0 = clk::now();
    dequant_kquant(raw, deq, N, K, (GGUFType)type);
    auto t1 = clk::now();
    for (uint32_t m = 0; m < M; m++)
        for (uint32_t n = 0; n < N; n++) {
            float a = 0.0f;
            for (uint32_t k = 0; k < K; k++) a += X[(size_t)m * K + k] * deq[(size_t)n * K + k];
            Y[(size_t)m * N + n] = a;
        }
    auto t2 = clk::now();
    if (t_dequant) *t_dequant = std::chrono::duration<double>(t1 - t0).count();
    if (t_dot) *t_dot = std::chrono::duration<double>(t2 - t1).count();
    return 0;
}

// ---- GGUFFile, field by field ------------------------------------------------
void* bpref_gguf_open(const char* path)
{
    GGUFFile* g = new GGUFFile;
    if (!g->open(path)) { delete g; return nullptr; }
    return g;
}

void bpref_gguf_close(void* h) { delete (GGUFFile*)h; }

void bpref_gguf_info(const void* h, uint32_t* version, uint64_t* n_tensors, uint64_t* data_offset)
{
    const GGUFFile* g = (const GGUFFile*)h;
    *version = g->version;
    *n_tensors = g->n_tensors;
    *data_offset = g->data_offset;
}

// name: pointer into the GGUFFile (valid until close); dims: up to 8 entries.
int bpref_gguf_tensor(const void* h, uint64_t i, const char** name, uint32_t* type, uint32_t* n_dims,
                      uint64_t* dims, uint64_t* offset)
{
    const GGUFFile* g = (const GGUFFile*)h;
    if (i >= g->tensors.size()) return -1;
    const GGUFTensorInfo& t = g->tensors[i];
    *name = t.name.c_str();
    *type = (uint32_t)t.type;
    *n_dims = (uint32_t)t.shape.size();
    for (size_t d = 0; d < t.shape.size() && d < 8; d++) dims[d] = t.shape[d];
    *offset = t.offset;
    return 0;
}

int64_t bpref_gguf_find(const void* h, const char* name)
{
    const GGUFFile* g = (const GGUFFile*)h;
    auto it = g->tensor_index.find(name);
    return it == g->tensor_index.end() ? -1 : (int64_t)it->second;
}

int bpref_gguf_has_key(const void* h, const char* key) { return ((const GGUFFile*)h)->hasKey(key) ? 1 : 0; }
uint32_t bpref_gguf_u32(const void* h, const char* key, uint32_t def) { return ((const GGUFFile*)h)->getU32(key, def); }
float bpref_gguf_f32(const void* h, const char* key, float def) { return ((const GGUFFile*)h)->getFloat(key, def); }
int bpref_gguf_bool(const void* h, const char* key, int def) { return ((const GGUFFile*)h)->getBool(key, def != 0) ? 1 : 0; }

// Copies getString(key, def) into buf (cap bytes, terminated); returns its length.
size_t bpref_gguf_string(const void* h, const char* key, const char* def, char* buf, size_t cap)
{
    const std::string s = ((const GGUFFile*)h)->getString(key, def);
    if (cap) {
        const size_t n = s.size() < cap - 1 ? s.size() : cap - 1;
        std::memcpy(buf, s.data(), n);
        buf[n] = 0;
    }
    return s.size();
}

// Element count of a string array (-1 when the key holds none) and one element.
int64_t bpref_gguf_string_array_len(const void* h, const char* key)
{
    auto* a = ((const GGUFFile*)h)->getStringArray(key);
    return a ? (int64_t)a->size() : -1;
}

size_t bpref_gguf_string_array_at(const void* h, const char* key, uint64_t i, char* buf, size_t cap)
{
    auto* a = ((const GGUFFile*)h)->getStringArray(key);
    if (!a || i >= a->size()) return 0;
    const std::string& s = (*a)[i];
    if (cap) {
        const size_t n = s.size() < cap - 1 ? s.size() : cap - 1;
        std::memcpy(buf, s.data(), n);
        buf[n] = 0;
    }
    return s.size();
}

// int32 array: count (-1 when none); copies up to cap elements.
int64_t bpref_gguf_i32_array(const void* h, const char* key, int32_t* out, uint64_t cap)
{
    auto* a = ((const GGUFFile*)h)->getI32Array(key);
    if (!a) return -1;
    for (uint64_t i = 0; i < a->size() && i < cap; i++) out[i] = (*a)[i];
    return (int64_t)a->size();
}

// extractModelConfig(file) as flat arrays: u[28] in the order of the assignments below, f[4], the four rope
// sections, the architecture name and, per layer, 1 for a sliding-window layer (count returned).
uint32_t bpref_model_config(const void* h, uint32_t* u, float* f, int32_t* sections, uint8_t* layer_types, uint32_t cap,
                            char* arch, size_t arch_cap)
{
    const ModelConfig c = extractModelConfig(*(const GGUFFile*)h);
    const uint32_t vals[28] = {c.nLayer, c.nHead, c.nKvHeads, c.nEmbd, c.intermediateSize, c.nVocab, c.headDim, c.kvHeadDim,
                               c.tieWordEmbeddings, c.hasQkNorm, c.activation == ActivationType::GELU, c.slidingWindow,
                               (uint32_t)c.layerAttnTypes.size(), c.hasSandwichNorm, c.pleSize, c.sharedKvLayers, c.hasMtp,
                               c.mtpNumLayers, c.numExperts, c.numExpertsPerTok, c.moeIntermediateSize,
                               c.moeSharedIntermediateSize, c.ssmInnerSize, c.ssmStateSize, c.ssmConvKernel, c.ssmGroupCount,
                               c.ssmTimeStepRank, c.fullAttentionInterval};
    std::memcpy(u, vals, sizeof(vals));
    f[0] = c.rmsNormEps; f[1] = c.ropeTheta; f[2] = c.embeddingScale; f[3] = c.logitSoftcap;
    for (int i = 0; i < 4; i++) sections[i] = i < (int)c.ropeSections.size() ? c.ropeSections[i] : 0;
    for (uint32_t i = 0; i < c.layerAttnTypes.size() && i < cap; i++)
        layer_types[i] = c.layerAttnTypes[i] == AttnLayerType::SlidingWindow;
    if (arch_cap) {
        const size_t n = c.arch.size() < arch_cap - 1 ? c.arch.size() : arch_cap - 1;
        std::memcpy(arch, c.arch.data(), n);
        arch[n] = 0;
    }
    return (uint32_t)c.layerAttnTypes.size();
}

}  // extern "C"
