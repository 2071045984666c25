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
    GPUBuffer b = createBuffer(name, w.data.size() * sizeof(uint32_t));
    if (b.handle) writeBuffer(b, w.data.data(), w.data.size() * sizeof(uint32_t));
    return b;
}

int KQDispatch::run(void* stream) const
{
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

}  // namespace bp
