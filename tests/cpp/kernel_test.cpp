// The reference's eleven Q4_K / Q5_K / Q6_K kernel tests (runtime/tests/kernel_test.cpp:1669-1748)
// re-stated against the C++ host layer: same names, same closed-form inputs, same
// tolerances; then the layer's own additions (fused dispatches, GGUF file, chain, model configuration).  Expected values come from the CPU oracle (test infrastructure),
// which plays the part of dequant_kquant + the sequential fp32 dot.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <functional>
#include <string>
#include <vector>

#include "../../backpack_amd/csrc/host/kq_ops.h"
#include "../../oracle/kq_oracle.h"

using namespace bp;

struct CheckResult { bool ok; std::string msg; };
struct TestEntry { const char* name; std::function<CheckResult()> fn; };
static std::vector<TestEntry>& registry() { static std::vector<TestEntry> r; return r; }
#define TEST(name) \
    static CheckResult test_##name(); \
    static struct Reg_##name { Reg_##name() { registry().push_back({#name, test_##name}); } } reg_##name; \
    static CheckResult test_##name()

static std::vector<float> randnVec(uint32_t seed, int n)
{
    kqo_rng r; kqo_rng_seed(&r, seed);
    std::vector<float> v(n); kqo_rng_randn_vec(&r, v.data(), n); return v;
}
static uint16_t f32ToF16(float f) { return kqo_f32_to_f16_trunc(f); }

static CheckResult assertClose(const float* a, const float* e, int n, float atol, float rtol)
{
    float worst = 0;
    int bad = kqo_assert_close(a, e, n, atol, rtol, &worst);
    if (!bad) return {true, ""};
    int at = 0; float ex = -1.0f;
    for (int i = 0; i < n; i++) {
        const float x = std::fabs(a[i] - e[i]) - (atol + rtol * std::fabs(e[i]));
        if (x > ex) { ex = x; at = i; }
    }
    char buf[192];
    snprintf(buf, sizeof buf, "%d elements outside tolerance, worst excess %g (element %d: got %.9g, expected %.9g)", bad, worst,
             at, a[at], e[at]);
    return {false, buf};
}

// raw blocks -> pack -> upload -> dispatch -> readback, expected = oracle
static CheckResult runMatmul(GGUFType type, const std::vector<uint8_t>& raw, int M, int N, int K,
                             const std::vector<float>& x, const std::vector<float>& bias, bool biasFirst)
{
    KQuantPacked pk = type == GGUF_TYPE_Q4_K ? pack_q4k(raw.data(), N, K)
                    : type == GGUF_TYPE_Q5_K ? pack_q5k(raw.data(), N, K) : pack_q6k(raw.data(), N, K);
    std::vector<float> expected(M * N);
    kqo_matmul((int)type, x.data(), pk.data.data(), biasFirst ? bias.data() : nullptr, expected.data(), M, N, K,
               pk.rowStrideWords, 0, 0);
    GPUBuffer bx = createBuffer("X", x.size() * 4), bw = uploadKQWeight("W", pk), bb = createBuffer("B", N * 4),
              by = createBuffer("Y", (size_t)M * N * 4);
    writeBuffer(bx, x.data(), x.size() * 4);
    writeBuffer(bb, bias.data(), N * 4);
    KQDispatch d{type, bx, bw, bb, by, makeKQParams(K, N, pk.nBlocks, pk.rowStrideWords, 0), (uint32_t)M, "kq"};
    if (d.run() != BPK_OK) return {false, bpk_last_error()};
    std::vector<float> got(M * N);
    readBuffer(by, got.data(), got.size() * 4);
    releaseBuffer(bx); releaseBuffer(bw); releaseBuffer(bb); releaseBuffer(by);
    return assertClose(got.data(), expected.data(), M * N, 2e-4f, 2e-4f);
}

static std::vector<uint8_t> q4kRaw(int N, int NB, std::function<float(int, int)> d, std::function<float(int, int)> dm,
                                   std::function<int(int, int, int)> byte)
{
    std::vector<uint8_t> raw((size_t)N * NB * 144);
    for (int n = 0; n < N; n++) for (int b = 0; b < NB; b++) {
        uint8_t* p = raw.data() + ((size_t)n * NB + b) * 144;
        uint16_t hd = f32ToF16(d(n, b)), hm = f32ToF16(dm(n, b));
        memcpy(p, &hd, 2); memcpy(p + 2, &hm, 2);
        for (int i = 4; i < 144; i++) p[i] = (uint8_t)byte(n, b, i);
    }
    return raw;
}
static std::vector<uint8_t> q5kRaw(int N, int NB, std::function<float(int, int)> d, std::function<float(int, int)> dm,
                                   std::function<int(int, int, int)> byte)
{
    std::vector<uint8_t> raw((size_t)N * NB * 176);
    for (int n = 0; n < N; n++) for (int b = 0; b < NB; b++) {
        uint8_t* p = raw.data() + ((size_t)n * NB + b) * 176;
        uint16_t hd = f32ToF16(d(n, b)), hm = f32ToF16(dm(n, b));
        memcpy(p, &hd, 2); memcpy(p + 2, &hm, 2);
        for (int i = 4; i < 176; i++) p[i] = (uint8_t)byte(n, b, i);
    }
    return raw;
}
static std::vector<uint8_t> q6kRaw(int N, int NB, std::function<float(int, int)> d, std::function<int(int, int, int)> byte)
{
    std::vector<uint8_t> raw((size_t)N * NB * 210);
    for (int n = 0; n < N; n++) for (int b = 0; b < NB; b++) {
        uint8_t* p = raw.data() + ((size_t)n * NB + b) * 210;
        for (int i = 0; i < 208; i++) p[i] = (uint8_t)byte(n, b, i);
        uint16_t hd = f32ToF16(d(n, b)); memcpy(p + 208, &hd, 2);
    }
    return raw;
}
static std::vector<float> biasVec(int N, bool on) { std::vector<float> b(N, 0.f); if (on) for (int n = 0; n < N; n++) b[n] = .01f * n; return b; }

TEST(q5k_matmul_reference) {
    const int N = 8, K = 256;
    auto raw = q5kRaw(N, 1, [](int n, int) { return .02f + .001f * n; }, [](int n, int) { return .01f + .0005f * n; },
                      [](int n, int, int i) { return (n * 37 + i * 13 + 7) & 255; });
    return runMatmul(GGUF_TYPE_Q5_K, raw, 1, N, K, randnVec(4242, K), biasVec(N, false), false);
}
TEST(q5k_matmul_batched4_reference) {
    const int M = 5, N = 9, K = 512;
    auto raw = q5kRaw(N, 2, [](int n, int) { return .02f + .001f * n; }, [](int, int b) { return .01f + .0002f * b; },
                      [](int n, int b, int i) { return n * 29 + b * 11 + i * 19; });
    return runMatmul(GGUF_TYPE_Q5_K, raw, M, N, K, randnVec(4949, M * K), biasVec(N, true), true);
}
TEST(q4k_matmul_reference) {
    const int N = 8, K = 256;
    auto raw = q4kRaw(N, 1, [](int n, int) { return .02f + .001f * n; }, [](int n, int) { return .01f + .0005f * n; },
                      [](int n, int, int i) { return (n * 31 + i * 17 + 3) & 255; });
    return runMatmul(GGUF_TYPE_Q4_K, raw, 1, N, K, randnVec(4343, K), biasVec(N, false), false);
}
TEST(q4k_matmul_128_reference) {
    const int N = 7, K = 512;
    auto raw = q4kRaw(N, 2, [](int n, int) { return .02f + .001f * n; }, [](int, int b) { return .01f + .0002f * b; },
                      [](int n, int b, int j) { return n * 31 + b * 13 + j * 17; });
    return runMatmul(GGUF_TYPE_Q4_K, raw, 1, N, K, randnVec(5555, K), biasVec(N, true), true);
}
TEST(q6k_matmul_reference) {
    const int N = 8, K = 768;
    auto raw = q6kRaw(N, 3, [](int n, int q) { return .02f + .001f * n + .0003f * q; },
                      [](int n, int q, int i) { return (n * 29 + q * 23 + i * 19 + 5) & 255; });
    return runMatmul(GGUF_TYPE_Q6_K, raw, 1, N, K, randnVec(4646, K), biasVec(N, false), false);
}
TEST(q6k_matmul_wide_reference) {
    const int N = 19, K = 768;
    auto raw = q6kRaw(N, 3, [](int n, int b) { return .018f + .0007f * n + .0002f * b; },
                      [](int n, int b, int i) { return (n * 37 + b * 17 + i * 13 + 11) & 255; });
    return runMatmul(GGUF_TYPE_Q6_K, raw, 1, N, K, randnVec(4747, K), biasVec(N, true), true);
}
TEST(q4k_matmul_batched4_reference) {
    const int M = 5, N = 9, K = 512;
    auto raw = q4kRaw(N, 2, [](int n, int) { return .02f + .001f * n; }, [](int, int b) { return .01f + .0002f * b; },
                      [](int n, int b, int i) { return n * 31 + b * 13 + i * 17; });
    return runMatmul(GGUF_TYPE_Q4_K, raw, M, N, K, randnVec(4848, M * K), biasVec(N, true), true);
}
TEST(q6k_matmul_batched4_reference) {
    const int M = 5, N = 9, K = 768;
    auto raw = q6kRaw(N, 3, [](int n, int b) { return .018f + .0007f * n + .0002f * b; },
                      [](int n, int b, int i) { return n * 23 + b * 17 + i * 13; });
    return runMatmul(GGUF_TYPE_Q6_K, raw, M, N, K, randnVec(5050, M * K), biasVec(N, true), true);
}
TEST(q4k_matmul_batched8_reference) {
    const int M = 9, N = 9, K = 512;
    auto raw = q4kRaw(N, 2, [](int n, int) { return .02f + .001f * n; }, [](int, int b) { return .01f + .0002f * b; },
                      [](int n, int b, int i) { return n * 31 + b * 13 + i * 17; });
    return runMatmul(GGUF_TYPE_Q4_K, raw, M, N, K, randnVec(5151, M * K), biasVec(N, true), true);
}

static CheckResult runGather(const std::vector<uint8_t>& raw, int N, int K, const std::vector<int32_t>& toks)
{
    KQuantPacked pk = pack_q6k(raw.data(), N, K);
    const int M = (int)toks.size();
    std::vector<float> expected((size_t)M * K), got((size_t)M * K);
    kqo_dequant_rows(KQO_TYPE_Q6_K, pk.data.data(), pk.rowStrideWords, toks.data(), M, K, expected.data());
    GPUBuffer bw = uploadKQWeight("W", pk), bt = createBuffer("T", M * 4), bx = createBuffer("X", got.size() * 4);
    writeBuffer(bt, toks.data(), M * 4);
    if (gatherKQ(GGUF_TYPE_Q6_K, bw, pk.rowStrideWords, bt, M, K, bx) != BPK_OK) return {false, bpk_last_error()};
    readBuffer(bx, got.data(), got.size() * 4);
    releaseBuffer(bw); releaseBuffer(bt); releaseBuffer(bx);
    return assertClose(got.data(), expected.data(), M * K, 1e-6f, 1e-6f);
}
TEST(q6k_gather_reference) {
    auto raw = q6kRaw(3, 3, [](int n, int b) { return .015f + .001f * n + .0002f * b; },
                      [](int n, int b, int i) { return (n * 41 + b * 23 + i * 11 + 9) & 255; });
    return runGather(raw, 3, 768, {2});
}
TEST(q6k_gather_batched_reference) {
    auto raw = q6kRaw(4, 3, [](int n, int) { return .014f + .001f * n; }, [](int n, int b, int i) { return n * 43 + b * 19 + i * 7 + 3; });
    return runGather(raw, 4, 768, {3, 0, 2});
}
TEST(fuse_qkv_rows) {
    // q|k|v fused upload: the fused matvec equals the three separate ones
    const int K = 512, Nq = 9, Nk = 3;
    auto mk = [&](int N, int salt) {
        return q4kRaw(N, 2, [](int n, int) { return .02f + .001f * n; }, [](int, int b) { return .01f + .0002f * b; },
                      [salt](int n, int b, int i) { return n * 31 + b * 13 + i * 17 + salt; });
    };
    auto rq = mk(Nq, 1), rk = mk(Nk, 2), rv = mk(Nk, 3);
    KQuantPacked q = pack_q4k(rq.data(), Nq, K), k = pack_q4k(rk.data(), Nk, K), v = pack_q4k(rv.data(), Nk, K);
    KQuantPacked f = fuseKQ({&q, &k, &v});
    if (f.N != (uint32_t)(Nq + 2 * Nk)) return {false, "fused row count"};
    auto x = randnVec(77, K);
    std::vector<float> expected(f.N), got(f.N), zero(f.N, 0.f);
    kqo_matmul(KQO_TYPE_Q4_K, x.data(), q.data.data(), nullptr, expected.data(), 1, Nq, K, q.rowStrideWords, 0, 0);
    kqo_matmul(KQO_TYPE_Q4_K, x.data(), k.data.data(), nullptr, expected.data() + Nq, 1, Nk, K, k.rowStrideWords, 0, 0);
    kqo_matmul(KQO_TYPE_Q4_K, x.data(), v.data.data(), nullptr, expected.data() + Nq + Nk, 1, Nk, K, v.rowStrideWords, 0, 0);
    GPUBuffer bx = createBuffer("X", K * 4), bw = uploadKQWeight("qkv", f), by = createBuffer("Y", f.N * 4);
    writeBuffer(bx, x.data(), K * 4);
    KQDispatch d{GGUF_TYPE_Q4_K, bx, bw, GPUBuffer{}, by, makeKQParams(K, f.N, f.nBlocks, f.rowStrideWords), 1, "qkv"};
    if (d.run() != BPK_OK) return {false, bpk_last_error()};
    readBuffer(by, got.data(), f.N * 4);
    releaseBuffer(bx); releaseBuffer(bw); releaseBuffer(by);
    return assertClose(got.data(), expected.data(), f.N, 2e-4f, 2e-4f);
}

TEST(fused_down_silu_residual) {
    // act*mul -> kq_down -> add_inplace (runtime/model_runner.cpp:3748-3793) as one dispatch, against the
    // oracle's three steps
    const int N = 24, K = 512;
    auto raw = q6kRaw(N, 2, [](int n, int b) { return .018f + .0007f * n + .0002f * b; },
                      [](int n, int b, int i) { return n * 23 + b * 17 + i * 13; });
    KQuantPacked pk = pack_q6k(raw.data(), N, K);
    auto gu = randnVec(91, 2 * K), res = randnVec(92, N);
    std::vector<float> act(K), expected(N), got(N);
    kqo_prologue(2, gu.data(), nullptr, 0.f, 1, K, act.data());
    kqo_matmul(KQO_TYPE_Q6_K, act.data(), pk.data.data(), nullptr, expected.data(), 1, N, K, pk.rowStrideWords, 0, 0);
    for (int n = 0; n < N; n++) expected[n] += res[n];
    GPUBuffer bx = createBuffer("GateUp", 2 * K * 4), bw = uploadKQWeight("down", pk), by = createBuffer("x", N * 4);
    writeBuffer(bx, gu.data(), 2 * K * 4);
    writeBuffer(by, res.data(), N * 4);
    KQFusedDispatch d;
    d.base = KQDispatch{GGUF_TYPE_Q6_K, bx, bw, GPUBuffer{}, by, makeKQParams(K, N, pk.nBlocks, pk.rowStrideWords), 1, "down"};
    d.prologue = BPK_PRO_SILU_MUL;
    d.Residual = by;   // x += down(...)
    if (d.run() != BPK_OK) return {false, bpk_last_error()};
    readBuffer(by, got.data(), N * 4);
    releaseBuffer(bx); releaseBuffer(bw); releaseBuffer(by);
    return assertClose(got.data(), expected.data(), N, 2e-4f, 2e-4f);
}
TEST(gguf_file_to_fused_weight) {
    // a two-tensor GGUF written here, read through the GGUFFile mirror, gate|up stacked from it
    const int K = 256, N = 6;
    auto rg = q4kRaw(N, 1, [](int n, int) { return .02f + .001f * n; }, [](int, int) { return .01f; },
                     [](int n, int, int i) { return n * 31 + i * 17; });
    auto ru = q4kRaw(N, 1, [](int n, int) { return .03f + .001f * n; }, [](int, int) { return .02f; },
                     [](int n, int, int i) { return n * 7 + i * 5 + 1; });
    std::vector<uint8_t> f;
    auto put = [&](const void* p, size_t n) { f.insert(f.end(), (const uint8_t*)p, (const uint8_t*)p + n); };
    auto u32 = [&](uint32_t v) { put(&v, 4); };
    auto u64 = [&](uint64_t v) { put(&v, 8); };
    auto str = [&](const std::string& s) { u64(s.size()); put(s.data(), s.size()); };
    u32(0x46554747); u32(3); u64(2); u64(2);
    str("general.architecture"); u32(8); str("llama");
    str("llama.block_count"); u32(4); u32(32);
    const size_t bytes = (size_t)N * 144;
    str("blk.0.ffn_gate.weight"); u32(2); u64(K); u64(N); u32(12); u64(0);
    str("blk.0.ffn_up.weight"); u32(2); u64(K); u64(N); u32(12); u64((bytes + 31) / 32 * 32);
    const size_t data_offset = (f.size() + 31) / 32 * 32;
    f.resize(data_offset, 0);
    put(rg.data(), bytes);
    f.resize(data_offset + (bytes + 31) / 32 * 32, 0);
    put(ru.data(), bytes);
    const char* path = "/tmp/bpk_kernel_test.gguf";
    FILE* fp = fopen(path, "wb");
    if (!fp) return {false, "cannot write the temporary file"};
    fwrite(f.data(), 1, f.size(), fp);
    fclose(fp);
    GGUFFile g;
    if (!g.open(path)) return {false, bpk_last_error()};
    if (g.version != 3 || g.n_tensors != 2 || g.data_offset != data_offset) return {false, "header fields"};
    if (g.getString("general.architecture") != "llama" || g.getU32("llama.block_count") != 32 ||
        g.getU32("missing", 7) != 7 || g.hasKey("nope"))
        return {false, "metadata getters"};
    const GGUFTensorInfo* t = g.find("blk.0.ffn_up.weight");
    if (!t || t->shape.size() != 2 || t->shape[0] != (uint64_t)K || memcmp(t->data, ru.data(), bytes)) return {false, "tensor table"};
    GPUBuffer W; KQuantPacked desc; bpk_weight* owner = nullptr;
    if (!g.loadKQWeight({"blk.0.ffn_gate.weight", "blk.0.ffn_up.weight"}, W, desc, &owner)) return {false, bpk_last_error()};
    if (desc.N != 2u * N || desc.K != (uint32_t)K) return {false, "stacked descriptor"};
    KQuantPacked pg = pack_q4k(rg.data(), N, K), pu = pack_q4k(ru.data(), N, K);
    auto x = randnVec(5, K);
    std::vector<float> expected(2 * N), got(2 * N);
    kqo_matmul(KQO_TYPE_Q4_K, x.data(), pg.data.data(), nullptr, expected.data(), 1, N, K, pg.rowStrideWords, 0, 0);
    kqo_matmul(KQO_TYPE_Q4_K, x.data(), pu.data.data(), nullptr, expected.data() + N, 1, N, K, pu.rowStrideWords, 0, 0);
    GPUBuffer bx = createBuffer("X", K * 4), by = createBuffer("Y", 2 * N * 4);
    writeBuffer(bx, x.data(), K * 4);
    KQDispatch d{desc.type, bx, W, GPUBuffer{}, by, makeKQParams(K, desc.N, desc.nBlocks, desc.rowStrideWords), 1, "gate_up"};
    if (d.run() != BPK_OK) return {false, bpk_last_error()};
    readBuffer(by, got.data(), got.size() * 4);
    releaseBuffer(bx); releaseBuffer(by); releaseWeight(owner);
    remove(path);
    return assertClose(got.data(), expected.data(), 2 * N, 2e-4f, 2e-4f);
}

TEST(chain_of_a_decoder_layer_tail) {
    // o + residual -> norm -> gate|up -> silu*up -> down + residual, recorded as three fused dispatches and run as
    // ONE launch; expected = the same composition on the oracle, op after op
    const int H = 512, I = 768, NBH = H / 256, NBI = I / 256;
    auto ro = q4kRaw(H, NBH, [](int n, int) { return .004f + .00001f * n; }, [](int, int b) { return .002f + .0001f * b; },
                     [](int n, int b, int i) { return n * 31 + b * 13 + i * 17; });
    auto rg = q4kRaw(2 * I, NBH, [](int n, int) { return .003f + .000005f * n; }, [](int, int) { return .0015f; },
                     [](int n, int b, int i) { return n * 7 + b * 5 + i * 3 + 1; });
    auto rd = q6kRaw(H, NBI, [](int n, int b) { return .002f + .00001f * n + .0001f * b; },
                     [](int n, int b, int i) { return n * 29 + b * 23 + i * 19 + 5; });
    KQuantPacked po = pack_q4k(ro.data(), H, H), pg = pack_q4k(rg.data(), 2 * I, H), pd = pack_q6k(rd.data(), H, I);
    auto attn = randnVec(11, H), x0 = randnVec(12, H), nw = randnVec(13, H);
    for (auto& v : nw) v = 1.0f + 0.1f * v;
    const float eps = 1e-5f;
    // oracle
    std::vector<float> x = x0, t(H), xn(H), gu(2 * I), act(I), dn(H);
    kqo_matmul(KQO_TYPE_Q4_K, attn.data(), po.data.data(), nullptr, t.data(), 1, H, H, po.rowStrideWords, 0, 0);
    for (int i = 0; i < H; i++) x[i] += t[i];
    kqo_prologue(1, x.data(), nw.data(), eps, 1, H, xn.data());
    kqo_matmul(KQO_TYPE_Q4_K, xn.data(), pg.data.data(), nullptr, gu.data(), 1, 2 * I, H, pg.rowStrideWords, 0, 0);
    kqo_prologue(2, gu.data(), nullptr, 0.0f, 1, I, act.data());
    kqo_matmul(KQO_TYPE_Q6_K, act.data(), pd.data.data(), nullptr, dn.data(), 1, H, I, pd.rowStrideWords, 0, 0);
    std::vector<float> expected = x;
    for (int i = 0; i < H; i++) expected[i] += dn[i];
    // device
    GPUBuffer bAttn = createBuffer("attn", H * 4), bX = createBuffer("x", H * 4), bNw = createBuffer("nw", H * 4),
              bAct = createBuffer("act", I * 4), wo = uploadKQWeight("o", po), wg = uploadKQWeight("gate_up", pg),
              wd = uploadKQWeight("down", pd);
    writeBuffer(bAttn, attn.data(), H * 4); writeBuffer(bX, x0.data(), H * 4); writeBuffer(bNw, nw.data(), H * 4);
    KQChain chain;
    KQFusedDispatch o; o.base = KQDispatch{GGUF_TYPE_Q4_K, bAttn, wo, GPUBuffer{}, bX, makeKQParams(H, H, po.nBlocks, po.rowStrideWords), 1, "o"};
    o.Residual = bX;
    KQFusedDispatch g; g.base = KQDispatch{GGUF_TYPE_Q4_K, bX, wg, GPUBuffer{}, bAct, makeKQParams(H, I, pg.nBlocks, pg.rowStrideWords), 1, "gate_up"};
    g.prologue = BPK_PRO_RMS_NORM; g.NormW = bNw; g.eps = eps; g.epilogue = BPK_EPI_SILU_MUL;
    KQFusedDispatch d; d.base = KQDispatch{GGUF_TYPE_Q6_K, bAct, wd, GPUBuffer{}, bX, makeKQParams(I, H, pd.nBlocks, pd.rowStrideWords), 1, "down"};
    d.Residual = bX;
    chain.add(o); chain.add(g); chain.add(d);
    if (chain.build() != BPK_OK) return {false, bpk_last_error()};
    if (chain.run(0, 3) != BPK_OK || chain.status() != BPK_OK) return {false, bpk_last_error()};
    std::vector<float> got(H);
    readBuffer(bX, got.data(), H * 4);
    // and the same ops as separate fused dispatches give the same residual stream
    writeBuffer(bX, x0.data(), H * 4);
    if (o.run() != BPK_OK || g.run() != BPK_OK || d.run() != BPK_OK) return {false, bpk_last_error()};
    std::vector<float> sep(H);
    readBuffer(bX, sep.data(), H * 4);
    releaseBuffer(bAttn); releaseBuffer(bX); releaseBuffer(bNw); releaseBuffer(bAct); releaseBuffer(wo); releaseBuffer(wg); releaseBuffer(wd);
    CheckResult r = assertClose(got.data(), expected.data(), H, 2e-4f, 2e-4f);
    if (!r.ok) return {false, "chain against the oracle: " + r.msg};
    // (the two forms apply the norm's 1/rms at different places — to the activations in the chain, to the outputs in
    // the fused dispatch — and down's sums cancel heavily with these weights: a rounding's worth of difference in
    // act shows as a few 1e-5 relative in single elements)
    r = assertClose(sep.data(), expected.data(), H, 2e-4f, 2e-4f);
    if (!r.ok) return {false, "separate fused dispatches against the oracle: " + r.msg};
    r = assertClose(sep.data(), got.data(), H, 1e-4f, 1e-4f);
    if (!r.ok) return {false, "separate fused dispatches against the chain: " + r.msg};
    return r;
}
TEST(model_config_from_gguf) {
    // a metadata-only file of a Gemma-3-shaped model, read through the GGUFFile mirror and extractModelConfig
    std::vector<uint8_t> f;
    auto put = [&](const void* p, size_t n) { f.insert(f.end(), (const uint8_t*)p, (const uint8_t*)p + n); };
    auto u32 = [&](uint32_t v) { put(&v, 4); };
    auto u64 = [&](uint64_t v) { put(&v, 8); };
    auto f32 = [&](float v) { put(&v, 4); };
    auto str = [&](const std::string& s) { u64(s.size()); put(s.data(), s.size()); };
    u32(0x46554747); u32(3); u64(2); u64(8);
    str("general.architecture"); u32(8); str("gemma3");
    str("gemma3.block_count"); u32(4); u32(12);
    str("gemma3.embedding_length"); u32(4); u32(2560);
    str("gemma3.attention.head_count"); u32(4); u32(8);
    str("gemma3.attention.head_count_kv"); u32(4); u32(4);
    str("gemma3.attention.key_length"); u32(4); u32(256);
    str("gemma3.attention.sliding_window"); u32(4); u32(1024);
    str("gemma3.feed_forward_length"); u32(9); u32(5); u64(3); u32(6144); u32(10240); u32(1228);   // int32 array: the largest counts
    str("token_embd.weight"); u32(2); u64(8); u64(3); u32(0); u64(0);
    str("blk.0.post_attention_norm.weight"); u32(1); u64(8); u32(0); u64(96);
    const size_t data_offset = (f.size() + 31) / 32 * 32;
    f.resize(data_offset + 96 + 32, 0);
    const char* path = "/tmp/bpk_kernel_test_cfg.gguf";
    FILE* fp = fopen(path, "wb");
    if (!fp) return {false, "cannot write the temporary file"};
    fwrite(f.data(), 1, f.size(), fp);
    fclose(fp);
    (void)f32;
    GGUFFile g;
    if (!g.open(path)) return {false, bpk_last_error()};
    const ModelConfig c = extractModelConfig(g);
    remove(path);
    if (c.arch != "gemma3" || c.nLayer != 12 || c.nEmbd != 2560 || c.nHead != 8 || c.nKvHeads != 4) return {false, "dimensions"};
    if (c.headDim != 256 || c.kvHeadDim != 256 || c.intermediateSize != 10240 || c.nVocab != 3) return {false, "derived dimensions"};
    if (c.rmsNormEps != 1e-6f || c.ropeTheta != 1000000.0f || !c.tieWordEmbeddings) return {false, "defaults"};
    if (c.activation != ActivationType::GELU || c.embeddingScale != sqrtf(2560.0f) || !c.hasSandwichNorm) return {false, "gemma family"};
    if (c.slidingWindow != 1024 || c.layerAttnTypes.size() != 12) return {false, "sliding window"};
    for (uint32_t i = 0; i < 12; i++)
        if (c.layerAttnTypes[i] != ((i + 1) % 6 == 0 ? AttnLayerType::Global : AttnLayerType::SlidingWindow)) return {false, "layer pattern"};
    if (c.numExperts != 0 || c.hasMtp || c.ropeSections != std::vector<int32_t>({11, 11, 10, 0}) || !c.isAttentionLayer(5))
        return {false, "remaining defaults"};
    return {true, ""};
}

// Host-only checks (no device is touched): a Q6_K weight view without the 16 readable bytes behind its last row
// is refused before anything is launched; the same view with them passes the check.
static int hostOnlyChecks()
{
    int failed = 0;
    auto expect = [&](const char* what, bool ok) { printf("%-60s %s\n", what, ok ? "PASS" : "FAIL"); failed += !ok; };
    const uint32_t N = 4096, K = 14336;
    uint32_t nb = 0, rs = 0;
    expect("layout of a Q6_K row", bpk_kq_layout(BPK_TYPE_Q6_K, K, &nb, &rs) == BPK_OK && nb == 56 && rs == 2940);
    const size_t rows = (size_t)N * rs * 4;   // 11760 * 4096 bytes: a whole number of allocation granules
    GPUBuffer exact{(void*)0x1000, rows, 0}, tailed{(void*)0x1000, rows + KQ_WEIGHT_TAIL_BYTES, 0};
    expect("Q6_K view without the tail is refused", checkKQWeightView(GGUF_TYPE_Q6_K, exact, N, rs, "down") == BPK_ERR_SHAPE);
    expect("Q6_K view with the tail passes", checkKQWeightView(GGUF_TYPE_Q6_K, tailed, N, rs, "down") == BPK_OK);
    GPUBuffer sub{(void*)0x1000, rows + KQ_WEIGHT_TAIL_BYTES, rows / 2};
    expect("Q6_K sub-view of the second half of the rows passes", checkKQWeightView(GGUF_TYPE_Q6_K, sub, N / 2, rs, "down") == BPK_OK);
    expect("Q6_K sub-view that runs past the allocation is refused",
           checkKQWeightView(GGUF_TYPE_Q6_K, sub, N / 2 + 1, rs, "down") == BPK_ERR_SHAPE);
    expect("Q4_K needs no tail", checkKQWeightView(GGUF_TYPE_Q4_K, GPUBuffer{(void*)0x1000, (size_t)N * 576 * 4, 0}, N, 576, "o") == BPK_OK);
    // the dispatches run the check before they launch: a refused view returns without a device call
    KQDispatch d{GGUF_TYPE_Q6_K, GPUBuffer{(void*)0x2000, (size_t)K * 4, 0}, exact, GPUBuffer{}, GPUBuffer{(void*)0x3000, (size_t)N * 4, 0},
                 makeKQParams(K, N, nb, rs), 1, "down"};
    expect("KQDispatch::run refuses it", d.run() == BPK_ERR_SHAPE);
    KQFusedDispatch f; f.base = d;
    expect("KQFusedDispatch::run refuses it", f.run() == BPK_ERR_SHAPE);
    KQChain c; c.add(f);
    expect("KQChain::build refuses it", c.build() == BPK_ERR_SHAPE);
    printf("%d host-only checks failed\n", failed);
    return failed ? 1 : 0;
}

int main(int argc, char** argv)
{
    if (argc > 1 && !strcmp(argv[1], "--host-only")) return hostOnlyChecks();
    if (bpk_init(0) != BPK_OK) { fprintf(stderr, "bpk_init: %s\n", bpk_last_error()); return 2; }
    int failed = 0;
    for (auto& t : registry()) {
        CheckResult r = t.fn();
        printf("%-36s %s %s\n", t.name, r.ok ? "PASS" : "FAIL", r.msg.c_str());
        fflush(stdout);
        failed += !r.ok;
    }
    printf("%zu tests, %d failed\n", registry().size(), failed);
    return failed ? 1 : 0;
}
