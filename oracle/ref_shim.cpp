// ref_shim.cpp — extern "C" doorway into the reference's own CPU functions.
//
// TEST INFRASTRUCTURE ONLY.  Compiled together with the reference's
// runtime/gguf_loader.cpp, from where that file lies in the reference checkout,
// into oracle/_ref/libbp_ref.so (see the Makefile).  It adds no arithmetic of
// its own: every call forwards to pack_q4k / pack_q6k / dequant_kquant
// (runtime/gguf_loader.h:108-124, :147) so the restatement in kq_oracle.c can
// be compared with the reference as this compiler builds it, and so the
// benchmark can time the reference's real CPU path.
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
    else if (type == (int)GGUF_TYPE_Q6_K) p = pack_q6k(raw, N, K);
    else return -1;
    if (n_blocks) *n_blocks = p.nBlocks;
    if (row_stride_words) *row_stride_words = p.rowStrideWords;
    if (out) std::memcpy(out, p.data.data(), p.data.size() * sizeof(uint32_t));
    return 0;
}

int bpref_dequant(int type, const void* raw, float* out, uint32_t N, uint32_t K)
{
    if (type != (int)GGUF_TYPE_Q4_K && type != (int)GGUF_TYPE_Q6_K) return -1;
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

}  // extern "C"
