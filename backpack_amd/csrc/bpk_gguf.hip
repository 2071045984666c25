// bpk_gguf.hip — GGUF container reader on the host side of the C ABI: header, metadata, tensor table and
// the step from named tensors to device weights (host code only; it lives in a .hip file so that it is
// built into the same library).
//
// Replaces, for this path, GGUFFile::open and its accessors (runtime/gguf_loader.cpp:90-182,
// runtime/gguf_loader.h:49-86) and the tensor -> packKQ -> fuseKQ -> uploadKQWeight sequence of the loader
// (runtime/model_runner.cpp:1275-1338).  Differences by design: the file is memory-mapped and every length
// and offset is checked against its size (a truncated or hostile file is refused, not read past its end),
// and `general.alignment` is honoured when present (the reference always aligns the data section to 32,
// which is also the default here).
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <new>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/bpk_kquant.h"

namespace kq {
int api_fail(int code, const char* fmt, va_list ap);   // bpk_api.hip: stores the message of bpk_last_error()
}

namespace {

int fail(int code, const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    const int rc = kq::api_fail(code, fmt, ap);
    va_end(ap);
    return rc;
}

enum MetaType : uint32_t {
    META_UINT8 = 0, META_INT8 = 1, META_UINT16 = 2, META_INT16 = 3, META_UINT32 = 4, META_INT32 = 5,
    META_FLOAT32 = 6, META_BOOL = 7, META_STRING = 8, META_ARRAY = 9, META_UINT64 = 10, META_INT64 = 11,
    META_FLOAT64 = 12,
};

// One metadata value: scalars widened to 64 bits, strings and arrays kept as views into the mapping.
struct MetaValue {
    uint32_t type = 0;        // MetaType of the value (META_ARRAY for arrays)
    uint32_t elem_type = 0;   // arrays: MetaType of the elements
    uint64_t u = 0;           // unsigned scalars, bool
    int64_t i = 0;            // signed scalars
    double f = 0.0;           // float scalars
    const char* str = nullptr;   // strings: bytes (not terminated) ...
    uint64_t len = 0;            // ... and their count; arrays: element count
    const uint8_t* arr = nullptr;   // arrays of fixed-size elements: first element
    std::vector<std::pair<const char*, uint64_t>> strs;   // arrays of strings
};

struct Tensor {
    std::string name;
    uint32_t type = 0, n_dims = 0;
    uint64_t dims[4] = {1, 1, 1, 1};
    uint64_t offset = 0;   // from the start of the data section
    uint64_t bytes = 0;    // 0 when the type's block size is not known here
};

// (elements per block, bytes per block) of the ggml tensor types; {0, 0} = unknown
void type_block(uint32_t type, uint32_t& elems, uint32_t& bytes)
{
    switch (type) {
        case 0: elems = 1; bytes = 4; return;        // F32
        case 1: elems = 1; bytes = 2; return;        // F16
        case 2: elems = 32; bytes = 18; return;      // Q4_0
        case 3: elems = 32; bytes = 20; return;      // Q4_1
        case 6: elems = 32; bytes = 22; return;      // Q5_0
        case 7: elems = 32; bytes = 24; return;      // Q5_1
        case 8: elems = 32; bytes = 34; return;      // Q8_0
        case 9: elems = 32; bytes = 36; return;      // Q8_1
        case 10: elems = 256; bytes = 84; return;    // Q2_K
        case 11: elems = 256; bytes = 110; return;   // Q3_K
        case 12: elems = 256; bytes = 144; return;   // Q4_K
        case 13: elems = 256; bytes = 176; return;   // Q5_K
        case 14: elems = 256; bytes = 210; return;   // Q6_K
        case 20: elems = 32; bytes = 18; return;     // IQ4_NL
        case 23: elems = 256; bytes = 136; return;   // IQ4_XS
        case 24: elems = 1; bytes = 1; return;       // I8
        case 25: elems = 1; bytes = 2; return;       // I16
        case 26: elems = 1; bytes = 4; return;       // I32
        case 27: elems = 1; bytes = 8; return;       // I64
        case 28: elems = 1; bytes = 8; return;       // F64
        case 30: elems = 1; bytes = 2; return;       // BF16
        default: elems = 0; bytes = 0; return;
    }
}

// Bounds-checked cursor over the mapping.
struct Cursor {
    const uint8_t* base;
    uint64_t size, pos = 0;
    bool ok = true;
    bool need(uint64_t n)
    {
        if (!ok || n > size - pos) { ok = false; return false; }
        return true;
    }
    template <typename T>
    T get()
    {
        T v{};
        if (need(sizeof(T))) { memcpy(&v, base + pos, sizeof(T)); pos += sizeof(T); }
        return v;
    }
    bool str(const char*& s, uint64_t& len)
    {
        len = get<uint64_t>();
        if (!need(len)) return false;
        s = (const char*)(base + pos);
        pos += len;
        return true;
    }
};

uint32_t scalar_size(uint32_t t)
{
    switch (t) {
        case META_UINT8: case META_INT8: case META_BOOL: return 1;
        case META_UINT16: case META_INT16: return 2;
        case META_UINT32: case META_INT32: case META_FLOAT32: return 4;
        case META_UINT64: case META_INT64: case META_FLOAT64: return 8;
        default: return 0;
    }
}

bool read_scalar(Cursor& c, uint32_t t, MetaValue& v)
{
    switch (t) {
        case META_UINT8: v.u = c.get<uint8_t>(); v.i = (int64_t)v.u; v.f = (double)v.u; break;
        case META_INT8: v.i = c.get<int8_t>(); v.u = (uint64_t)v.i; v.f = (double)v.i; break;
        case META_UINT16: v.u = c.get<uint16_t>(); v.i = (int64_t)v.u; v.f = (double)v.u; break;
        case META_INT16: v.i = c.get<int16_t>(); v.u = (uint64_t)v.i; v.f = (double)v.i; break;
        case META_UINT32: v.u = c.get<uint32_t>(); v.i = (int64_t)v.u; v.f = (double)v.u; break;
        case META_INT32: v.i = c.get<int32_t>(); v.u = (uint64_t)v.i; v.f = (double)v.i; break;
        case META_UINT64: v.u = c.get<uint64_t>(); v.i = (int64_t)v.u; v.f = (double)v.u; break;
        case META_INT64: v.i = c.get<int64_t>(); v.u = (uint64_t)v.i; v.f = (double)v.i; break;
        case META_FLOAT32: v.f = c.get<float>(); break;
        case META_FLOAT64: v.f = c.get<double>(); break;
        case META_BOOL: v.u = c.get<uint8_t>() != 0; v.i = (int64_t)v.u; break;
        default: return false;
    }
    return c.ok;
}

bool read_value(Cursor& c, uint32_t t, MetaValue& v, int depth)
{
    v.type = t;
    if (t == META_STRING) return c.str(v.str, v.len);
    if (t != META_ARRAY) return read_scalar(c, t, v);
    v.elem_type = c.get<uint32_t>();
    v.len = c.get<uint64_t>();
    if (!c.ok) return false;
    if (v.elem_type == META_STRING) {
        if (v.len > (c.size - c.pos) / 8u) return false;   // each string costs at least its 8-byte length
        v.strs.reserve((size_t)v.len);
        for (uint64_t i = 0; i < v.len; ++i) {
            const char* s; uint64_t n;
            if (!c.str(s, n)) return false;
            v.strs.emplace_back(s, n);
        }
        return true;
    }
    if (v.elem_type == META_ARRAY) {   // nested arrays: walked and dropped
        if (depth > 4) return false;
        for (uint64_t i = 0; i < v.len; ++i) {
            MetaValue inner;
            if (!read_value(c, META_ARRAY, inner, depth + 1)) return false;
        }
        v.len = 0;
        return true;
    }
    const uint32_t es = scalar_size(v.elem_type);
    if (es == 0 || v.len > (c.size - c.pos) / es) return false;
    v.arr = c.base + c.pos;
    c.pos += v.len * es;
    return true;
}

}  // namespace

struct bpk_gguf {
    const uint8_t* map = nullptr;
    uint64_t size = 0;
    uint32_t version = 0;
    uint64_t n_kv = 0, data_offset = 0;
    std::unordered_map<std::string, MetaValue> meta;
    std::vector<Tensor> tensors;
    std::unordered_map<std::string, size_t> index;
};

namespace {

const MetaValue* find_meta(const bpk_gguf* g, const char* key)
{
    auto it = g->meta.find(key);
    return it == g->meta.end() ? nullptr : &it->second;
}

void fill_info(const bpk_gguf* g, const Tensor& t, bpk_gguf_tensor* out)
{
    out->name = t.name.c_str();
    out->type = t.type;
    out->n_dims = t.n_dims;
    for (int d = 0; d < 4; ++d) out->dims[d] = t.dims[d];
    out->offset = t.offset;
    out->bytes = t.bytes;
    out->data = g->map + g->data_offset + t.offset;
}

}  // namespace

extern "C" {

static int gguf_open_body(const char* path, bpk_gguf** out);

// (no exception crosses the C boundary: a file that makes the parser run out of memory is a bad file)
int bpk_gguf_open(const char* path, bpk_gguf** out)
{
    if (!path || !out) return fail(BPK_ERR_NULL, "path and out must be non-null");
    *out = nullptr;
    try {
        return gguf_open_body(path, out);
    } catch (const std::bad_alloc&) {
        return fail(BPK_ERR_FORMAT, "%s: metadata too large to hold in memory", path);
    } catch (...) {
        return fail(BPK_ERR_IO, "%s: unexpected failure while reading", path);
    }
}

static int gguf_open_body(const char* path, bpk_gguf** out)
{
    const int fd = open(path, O_RDONLY | O_CLOEXEC);
    if (fd < 0) return fail(BPK_ERR_IO, "cannot open %s", path);
    struct stat st;
    if (fstat(fd, &st) != 0 || st.st_size < 24) { close(fd); return fail(BPK_ERR_FORMAT, "%s is too short to be a GGUF file", path); }
    void* m = mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
    close(fd);   // the mapping outlives the descriptor
    if (m == MAP_FAILED) return fail(BPK_ERR_IO, "cannot map %s", path);
    bpk_gguf* g = new bpk_gguf;
    g->map = (const uint8_t*)m;
    g->size = (uint64_t)st.st_size;
    // whatever way this function is left other than by success (an error return, an exception from a
    // container), the mapping and the object go with it
    struct Guard {
        bpk_gguf* g;
        ~Guard()
        {
            if (!g) return;
            munmap((void*)g->map, (size_t)g->size);
            delete g;
        }
    } guard{g};
    auto bail = [&](int code, const char* what) { return fail(code, "%s: %s", path, what); };
    Cursor c{g->map, g->size};
    if (c.get<uint32_t>() != 0x46554747u) return bail(BPK_ERR_FORMAT, "not a GGUF file (magic)");
    g->version = c.get<uint32_t>();
    if (g->version < 2 || g->version > 3) return bail(BPK_ERR_FORMAT, "unsupported GGUF version (2 and 3 are read)");
    const uint64_t n_tensors = c.get<uint64_t>();
    g->n_kv = c.get<uint64_t>();
    if (!c.ok || n_tensors > g->size / 24 || g->n_kv > g->size / 12) return bail(BPK_ERR_FORMAT, "counts exceed the file size");
    for (uint64_t i = 0; i < g->n_kv; ++i) {
        const char* k; uint64_t kl;
        if (!c.str(k, kl)) return bail(BPK_ERR_FORMAT, "truncated metadata key");
        const uint32_t vt = c.get<uint32_t>();
        MetaValue v;
        if (!c.ok || !read_value(c, vt, v, 0)) return bail(BPK_ERR_FORMAT, "truncated or malformed metadata value");
        g->meta[std::string(k, (size_t)kl)] = std::move(v);
    }
    g->tensors.resize((size_t)n_tensors);
    for (uint64_t i = 0; i < n_tensors; ++i) {
        Tensor& t = g->tensors[(size_t)i];
        const char* n; uint64_t nl;
        if (!c.str(n, nl)) return bail(BPK_ERR_FORMAT, "truncated tensor name");
        t.name.assign(n, (size_t)nl);
        t.n_dims = c.get<uint32_t>();
        if (!c.ok || t.n_dims > 4) return bail(BPK_ERR_FORMAT, "tensor with more than 4 dimensions");
        for (uint32_t d = 0; d < t.n_dims; ++d) t.dims[d] = c.get<uint64_t>();
        t.type = c.get<uint32_t>();
        t.offset = c.get<uint64_t>();
        if (!c.ok) return bail(BPK_ERR_FORMAT, "truncated tensor table");
        g->index[t.name] = (size_t)i;
    }
    uint64_t align = 32;
    if (const MetaValue* a = find_meta(g, "general.alignment"))
        if (a->type != META_STRING && a->type != META_ARRAY && a->u >= 1 && a->u <= (1u << 20) && (a->u & (a->u - 1)) == 0) align = a->u;
    g->data_offset = (c.pos + align - 1) / align * align;
    if (n_tensors && g->data_offset > g->size) return bail(BPK_ERR_FORMAT, "no data section");
    for (Tensor& t : g->tensors) {
        uint32_t be, bb;
        type_block(t.type, be, bb);
        if (be == 0) {           // size unknown here: the caller gets the pointer only, and it lies inside the file
            if (t.offset > g->size - g->data_offset) return bail(BPK_ERR_FORMAT, "tensor data lies outside the file");
            continue;
        }
        uint64_t n = 1;
        for (uint32_t d = 0; d < t.n_dims; ++d) {
            if (t.dims[d] != 0 && n > UINT64_MAX / t.dims[d]) return bail(BPK_ERR_FORMAT, "tensor element count overflows");
            n *= t.dims[d];
        }
        if (t.n_dims && t.dims[0] % be) return bail(BPK_ERR_FORMAT, "row length is not a multiple of the type's block");
        t.bytes = n / be * bb;
        if (t.offset > g->size - g->data_offset || t.bytes > g->size - g->data_offset - t.offset)
            return bail(BPK_ERR_FORMAT, "tensor data lies outside the file");
    }
    guard.g = nullptr;
    *out = g;
    return BPK_OK;
}

int bpk_gguf_close(bpk_gguf* g)
{
    if (!g) return BPK_OK;
    munmap((void*)g->map, (size_t)g->size);
    delete g;
    return BPK_OK;
}

int bpk_gguf_info(const bpk_gguf* g, uint32_t* version, uint64_t* n_tensors, uint64_t* n_kv, uint64_t* data_offset)
{
    if (!g) return fail(BPK_ERR_NULL, "null file handle");
    if (version) *version = g->version;
    if (n_tensors) *n_tensors = g->tensors.size();
    if (n_kv) *n_kv = g->n_kv;
    if (data_offset) *data_offset = g->data_offset;
    return BPK_OK;
}

int bpk_gguf_tensor_at(const bpk_gguf* g, uint64_t index, bpk_gguf_tensor* out)
{
    if (!g || !out) return fail(BPK_ERR_NULL, "null argument");
    if (index >= g->tensors.size()) return fail(BPK_ERR_SHAPE, "tensor index %llu out of range", (unsigned long long)index);
    fill_info(g, g->tensors[(size_t)index], out);
    return BPK_OK;
}

int bpk_gguf_find_tensor(const bpk_gguf* g, const char* name, bpk_gguf_tensor* out)
{
    if (!g || !name || !out) return fail(BPK_ERR_NULL, "null argument");
    auto it = g->index.find(name);
    if (it == g->index.end()) return fail(BPK_ERR_NOT_FOUND, "no tensor named %s", name);
    fill_info(g, g->tensors[it->second], out);
    return BPK_OK;
}

int bpk_gguf_has_key(const bpk_gguf* g, const char* key) { return g && key && find_meta(g, key) ? 1 : 0; }

int bpk_gguf_key_type(const bpk_gguf* g, const char* key)
{
    const MetaValue* v = g && key ? find_meta(g, key) : nullptr;
    return v ? (int)v->type : -1;
}

// Integers of any width, bool as 0/1; an integer array yields its largest element (the reference sizes
// buffers from per-layer arrays that way, runtime/gguf_loader.cpp:158-166).
int bpk_gguf_get_u32(const bpk_gguf* g, const char* key, uint32_t def, uint32_t* out)
{
    if (!g || !key || !out) return fail(BPK_ERR_NULL, "null argument");
    *out = def;
    const MetaValue* v = find_meta(g, key);
    if (!v) return BPK_OK;
    switch (v->type) {
        case META_UINT8: case META_UINT16: case META_UINT32: case META_UINT64: *out = (uint32_t)v->u; break;
        case META_INT8: case META_INT16: case META_INT32: case META_INT64: *out = (uint32_t)v->i; break;
        case META_ARRAY:
            // (the reference keeps both kinds as int32 and compares them so; elements of a uint32 array are
            // compared as what they are, which differs only from 2^31 on)
            if (v->elem_type == META_INT32 && v->len) {
                int32_t m;
                memcpy(&m, v->arr, 4);
                for (uint64_t i = 1; i < v->len; ++i) {
                    int32_t x;
                    memcpy(&x, v->arr + 4 * i, 4);
                    if (x > m) m = x;
                }
                *out = (uint32_t)m;
            } else if (v->elem_type == META_UINT32 && v->len) {
                uint32_t m;
                memcpy(&m, v->arr, 4);
                for (uint64_t i = 1; i < v->len; ++i) {
                    uint32_t x;
                    memcpy(&x, v->arr + 4 * i, 4);
                    if (x > m) m = x;
                }
                *out = m;
            }
            break;
        default: break;
    }
    return BPK_OK;
}

int bpk_gguf_get_f32(const bpk_gguf* g, const char* key, float def, float* out)
{
    if (!g || !key || !out) return fail(BPK_ERR_NULL, "null argument");
    const MetaValue* v = find_meta(g, key);
    *out = v && (v->type == META_FLOAT32 || v->type == META_FLOAT64) ? (float)v->f : def;
    return BPK_OK;
}

int bpk_gguf_get_bool(const bpk_gguf* g, const char* key, int def, int* out)
{
    if (!g || !key || !out) return fail(BPK_ERR_NULL, "null argument");
    const MetaValue* v = find_meta(g, key);
    *out = v && v->type == META_BOOL ? (int)v->u : def;
    return BPK_OK;
}

// Copies at most cap-1 bytes and terminates; *len receives the full length (0 when the key is absent or
// not a string).
int bpk_gguf_get_string(const bpk_gguf* g, const char* key, char* buf, size_t cap, size_t* len)
{
    if (!g || !key) return fail(BPK_ERR_NULL, "null argument");
    const MetaValue* v = find_meta(g, key);
    const bool is_str = v && v->type == META_STRING;
    if (len) *len = is_str ? (size_t)v->len : 0;
    if (buf && cap) {
        const size_t n = is_str ? (v->len < cap - 1 ? (size_t)v->len : cap - 1) : 0;
        if (n) memcpy(buf, v->str, n);
        buf[n] = 0;
    }
    return BPK_OK;
}

// Element count of an array-valued key (0 when absent or not an array) and, for arrays of strings, one
// element copied like bpk_gguf_get_string.
int bpk_gguf_array_len(const bpk_gguf* g, const char* key, uint64_t* n, uint32_t* elem_type)
{
    if (!g || !key || !n) return fail(BPK_ERR_NULL, "null argument");
    const MetaValue* v = find_meta(g, key);
    const bool is_arr = v && v->type == META_ARRAY;
    *n = is_arr ? (v->elem_type == META_STRING ? v->strs.size() : v->len) : 0;
    if (elem_type) *elem_type = is_arr ? v->elem_type : 0;
    return BPK_OK;
}

int bpk_gguf_array_data(const bpk_gguf* g, const char* key, const void** data, uint64_t* n, uint32_t* elem_type)
{
    if (!g || !key || !data || !n) return fail(BPK_ERR_NULL, "null argument");
    const MetaValue* v = find_meta(g, key);
    if (!v || v->type != META_ARRAY || !v->arr) {
        *data = nullptr;
        *n = 0;
        if (elem_type) *elem_type = 0;
        return BPK_OK;
    }
    *data = v->arr;
    *n = v->len;
    if (elem_type) *elem_type = v->elem_type;
    return BPK_OK;
}

int bpk_gguf_array_string(const bpk_gguf* g, const char* key, uint64_t index, char* buf, size_t cap, size_t* len)
{
    if (!g || !key) return fail(BPK_ERR_NULL, "null argument");
    const MetaValue* v = find_meta(g, key);
    if (!v || v->type != META_ARRAY || v->elem_type != META_STRING || index >= v->strs.size())
        return fail(BPK_ERR_NOT_FOUND, "%s[%llu] is not a string array element", key, (unsigned long long)index);
    const auto& s = v->strs[(size_t)index];
    if (len) *len = (size_t)s.second;
    if (buf && cap) {
        const size_t n = s.second < cap - 1 ? (size_t)s.second : cap - 1;
        if (n) memcpy(buf, s.first, n);
        buf[n] = 0;
    }
    return BPK_OK;
}

// Named Q4_K / Q5_K / Q6_K matrices (GGUF shape {K, N}) -> one device weight, rows stacked in the order given
// (q|k|v, gate|up).  All parts must share the type and K.
static int gguf_weight_create_body(const bpk_gguf* g, const char* const* names, uint32_t n_names, bpk_weight** out);

// Model hyper-parameters from the metadata and the tensor directory (extractModelConfig,
// runtime/gguf_loader.cpp:184-317): the same keys, defaults and probes.
static int model_config_body(const bpk_gguf* g, bpk_model_config* c, uint8_t* layer_types, uint32_t cap)
{
    memset(c, 0, sizeof(*c));
    std::string a = "llama";
    if (const MetaValue* v = find_meta(g, "general.architecture"); v && v->type == META_STRING) a.assign(v->str, (size_t)v->len);
    snprintf(c->arch, sizeof(c->arch), "%s", a.c_str());
    auto u32 = [&](const std::string& key, uint32_t def = 0) {
        uint32_t x = def;
        bpk_gguf_get_u32(g, key.c_str(), def, &x);
        return x;
    };
    auto f32 = [&](const std::string& key, float def) {
        float x = def;
        bpk_gguf_get_f32(g, key.c_str(), def, &x);
        return x;
    };
    auto has_tensor = [&](const std::string& name) { return g->index.count(name) > 0; };
    c->n_layer = u32(a + ".block_count");
    c->n_embd = u32(a + ".embedding_length");
    c->intermediate_size = u32(a + ".feed_forward_length");
    c->n_head = u32(a + ".attention.head_count");
    c->n_kv_heads = u32(a + ".attention.head_count_kv", c->n_head);
    c->rms_norm_eps = f32(a + ".attention.layer_norm_rms_epsilon", 1e-6f);
    c->rope_theta = f32(a + ".rope.freq_base", 1000000.0f);
    c->tie_word_embeddings = find_meta(g, "output.weight") ? 0 : 1;   // (a metadata key of that name, as the reference asks)
    // attention.key_length is the head width where rotary embedding covers only part of it
    const uint32_t dense_head = c->n_head ? c->n_embd / c->n_head : 0;
    c->kv_head_dim = u32(a + ".attention.key_length", dense_head);
    c->head_dim = c->kv_head_dim ? c->kv_head_dim : dense_head;
    if (auto it = g->index.find("token_embd.weight"); it != g->index.end()) {
        const Tensor& t = g->tensors[it->second];
        c->n_vocab = (uint32_t)(t.n_dims >= 2 ? t.dims[1] : t.dims[0]);   // GGUF shapes are (columns, rows)
    }
    c->has_qk_norm = has_tensor("blk.0.attn_q_norm.weight");
    for (uint32_t i = 1; i < c->n_layer && !c->has_qk_norm; ++i)   // hybrids carry it on their attention layers only
        c->has_qk_norm = has_tensor("blk." + std::to_string(i) + ".attn_q_norm.weight");
    const bool gemma = a == "gemma" || a == "gemma2" || a == "gemma3" || a == "gemma4";
    c->activation = gemma ? BPK_ACT_GELU : BPK_ACT_SILU;
    c->embedding_scale = gemma ? sqrtf((float)c->n_embd) : 0.0f;
    c->logit_softcap = f32(a + ".final_logit_softcapping", 0.0f);
    c->sliding_window = u32(a + ".attention.sliding_window");
    // per-layer attention kinds: 0 = global, 1 = sliding window
    c->n_layer_attn_types = c->sliding_window > 0 && c->n_layer > 0 ? c->n_layer : 0;
    if (layer_types && c->n_layer_attn_types) {
        if (cap < c->n_layer) return fail(BPK_ERR_SHAPE, "layer_types holds %u entries, the model has %u layers", cap, c->n_layer);
        const MetaValue* pat = find_meta(g, (a + ".attention.sliding_window_pattern").c_str());
        const bool use_pat = a == "gemma4" && pat && pat->type == META_ARRAY && pat->elem_type == META_BOOL && pat->arr &&
                             pat->len == c->n_layer;
        for (uint32_t i = 0; i < c->n_layer; ++i) {
            uint8_t t = 0;
            if (a == "gemma2") t = i % 2 == 0;                         // even layers slide
            else if (a == "gemma3") t = (i + 1) % 6 != 0;              // five sliding, one global
            else if (a == "gemma4") t = use_pat ? pat->arr[i] != 0 : (i + 1) % 6 != 0;
            layer_types[i] = t;
        }
    }
    c->shared_kv_layers = u32(a + ".attention.shared_kv_layers");
    c->ple_size = u32(a + ".embedding_length_per_layer_input");
    c->has_sandwich_norm = has_tensor("blk.0.post_norm.weight") || has_tensor("blk.0.attn_post_norm.weight") ||
                           has_tensor("blk.0.post_attention_norm.weight");
    c->has_mtp = has_tensor("mtp.0.blk.0.attn_q.weight") || has_tensor("mtp.0.enorm.weight");
    if (!c->has_mtp) {
        const uint32_t nextn = u32(a + ".nextn_predict_layers");
        if (nextn > 0) { c->has_mtp = 1; c->mtp_num_layers = nextn; }
    }
    c->num_experts = u32(a + ".expert_count");
    c->num_experts_per_tok = u32(a + ".expert_used_count");
    c->moe_intermediate_size = u32(a + ".expert_feed_forward_length");
    c->moe_shared_intermediate_size = u32(a + ".expert_shared_feed_forward_length", c->moe_intermediate_size);
    c->ssm_inner_size = u32(a + ".ssm.inner_size");
    c->ssm_state_size = u32(a + ".ssm.state_size");
    c->ssm_conv_kernel = u32(a + ".ssm.conv_kernel");
    c->ssm_group_count = u32(a + ".ssm.group_count");
    c->ssm_time_step_rank = u32(a + ".ssm.time_step_rank");
    c->full_attention_interval = u32(a + ".full_attention_interval");
    const int32_t sections[4] = {11, 11, 10, 0};
    memcpy(c->rope_sections, sections, sizeof(sections));
    const MetaValue* rs = find_meta(g, (a + ".rope.dimension_sections").c_str());
    if (rs && rs->type == META_ARRAY && (rs->elem_type == META_INT32 || rs->elem_type == META_UINT32) && rs->arr && rs->len >= 4)
        memcpy(c->rope_sections, rs->arr, 16);
    return BPK_OK;
}

int bpk_gguf_model_config(const bpk_gguf* g, bpk_model_config* out, uint8_t* layer_types, uint32_t layer_types_cap)
{
    if (!g || !out) return fail(BPK_ERR_NULL, "file and out must be non-null");
    try {
        return model_config_body(g, out, layer_types, layer_types_cap);
    } catch (const std::exception&) {
        return fail(BPK_ERR_IO, "out of memory while reading the model configuration");
    }
}

int bpk_gguf_weight_create(const bpk_gguf* g, const char* const* names, uint32_t n_names, bpk_weight** out)
{
    try {
        return gguf_weight_create_body(g, names, n_names, out);
    } catch (const std::bad_alloc&) {
        return fail(BPK_ERR_IO, "out of host memory while creating a weight");
    } catch (...) {
        return fail(BPK_ERR_IO, "unexpected failure while creating a weight");
    }
}

static int gguf_weight_create_body(const bpk_gguf* g, const char* const* names, uint32_t n_names, bpk_weight** out)
{
    if (!g || !names || !out) return fail(BPK_ERR_NULL, "null argument");
    if (n_names == 0 || n_names > 64) return fail(BPK_ERR_SHAPE, "1..64 tensors per weight");
    const void* parts[64];
    uint32_t rows[64];
    uint32_t type = 0, K = 0;
    for (uint32_t i = 0; i < n_names; ++i) {
        if (!names[i]) return fail(BPK_ERR_NULL, "null tensor name");
        auto it = g->index.find(names[i]);
        if (it == g->index.end()) return fail(BPK_ERR_NOT_FOUND, "no tensor named %s", names[i]);
        const Tensor& t = g->tensors[it->second];
        if (t.type != BPK_TYPE_Q4_K && t.type != BPK_TYPE_Q5_K && t.type != BPK_TYPE_Q6_K)
            return fail(BPK_ERR_TYPE, "%s has GGUF type %u; this path takes Q4_K (12), Q5_K (13) and Q6_K (14)", names[i], t.type);
        if (t.n_dims < 1 || t.n_dims > 2 || t.dims[0] > 0xFFFFFFFFull || t.dims[1] > 0xFFFFFFFFull || t.dims[1] == 0)
            return fail(BPK_ERR_SHAPE, "%s is not a matrix", names[i]);
        if (i == 0) { type = t.type; K = (uint32_t)t.dims[0]; }
        else if (t.type != type || t.dims[0] != K)
            return fail(BPK_ERR_SHAPE, "%s does not match the type and row length of %s", names[i], names[0]);
        parts[i] = g->map + g->data_offset + t.offset;
        rows[i] = (uint32_t)t.dims[1];
    }
    return bpk_weight_create((int)type, K, n_names, parts, rows, out);
}

}  // extern "C"
