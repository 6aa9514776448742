// GGUF container reader and model loader: from a .gguf file on disk to a ready decoder on the GPU.
//
// Stands in for the reference's GGUFReader (torch/io/gguf_loader.h:386-630: header, metadata key/values, tensor
// table, aligned data section) and for GGUFModel's quantised upload (torch/io/gguf_model.h:126-181 config keys,
// :1177-1360 tensor names and verbatim upload of the super-blocks): the file is memory-mapped, every Q4_K / Q6_K
// matrix is copied to HBM byte for byte, norm vectors as fp32, and the decode runtime is created on top.
// Written from the GGUF format description (versions 2 and 3, little endian):
//   u32 magic "GGUF" | u32 version | u64 n_tensors | u64 n_kv
//   n_kv  x { string key | u32 type | value }            string = u64 length + bytes; array = u32 type | u64 n | items
//   n_tensors x { string name | u32 n_dims | u64 dims[n_dims] | u32 ggml_type | u64 offset }
//   padding to general.alignment (default 32) | tensor data (offsets relative to here)
// dims[0] is the contiguous dimension (K, columns), dims[1] the rows (N).
#include "ptm_common.h"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstring>
#include <map>
#include <new>
#include <string>
#include <vector>

namespace ptm {

enum GgufType : uint32_t { G_U8, G_I8, G_U16, G_I16, G_U32, G_I32, G_F32, G_BOOL, G_STR, G_ARR, G_U64, G_I64, G_F64 };

struct GgufValue {
    uint32_t type = 0;
    uint64_t u = 0;      // integers and bool, widened
    double f = 0.0;      // floats, widened
    std::string s;       // strings
    uint32_t arr_type = 0;
    uint64_t arr_n = 0;
    const uint8_t* arr_data = nullptr;      // first element of a numeric or string array, inside the mapping
    std::vector<const uint8_t*> arr_items;  // string arrays: start of each element's u64 length (arrays of arrays: kept as shape only)
};

struct Cursor {
    const uint8_t* p;
    const uint8_t* end;
    bool ok = true;
    template <typename T>
    T get() {
        T v{};
        if (!ok || (size_t)(end - p) < sizeof(T)) { ok = false; return v; }
        memcpy(&v, p, sizeof(T));
        p += sizeof(T);
        return v;
    }
    std::string str() {
        const uint64_t n = get<uint64_t>();
        if (!ok || n > (uint64_t)(end - p) || n > (1u << 20)) { ok = false; return {}; }
        std::string s(reinterpret_cast<const char*>(p), (size_t)n);
        p += n;
        return s;
    }
    void skip(uint64_t n) {
        if (!ok || n > (uint64_t)(end - p)) { ok = false; return; }
        p += n;
    }
};

static int scalar_size(uint32_t t) {
    switch (t) {
        case G_U8: case G_I8: case G_BOOL: return 1;
        case G_U16: case G_I16: return 2;
        case G_U32: case G_I32: case G_F32: return 4;
        case G_U64: case G_I64: case G_F64: return 8;
        default: return 0;
    }
}

static bool read_value(Cursor& c, uint32_t type, GgufValue& v, int depth) {
    v.type = type;
    switch (type) {
        case G_U8: v.u = c.get<uint8_t>(); break;
        case G_I8: v.u = (uint64_t)(int64_t)c.get<int8_t>(); break;
        case G_U16: v.u = c.get<uint16_t>(); break;
        case G_I16: v.u = (uint64_t)(int64_t)c.get<int16_t>(); break;
        case G_U32: v.u = c.get<uint32_t>(); break;
        case G_I32: v.u = (uint64_t)(int64_t)c.get<int32_t>(); break;
        case G_U64: v.u = c.get<uint64_t>(); break;
        case G_I64: v.u = (uint64_t)c.get<int64_t>(); break;
        case G_BOOL: v.u = c.get<uint8_t>() != 0; break;
        case G_F32: v.f = c.get<float>(); break;
        case G_F64: v.f = c.get<double>(); break;
        case G_STR: v.s = c.str(); break;
        case G_ARR: {
            if (depth > 2) return false;
            v.arr_type = c.get<uint32_t>();
            v.arr_n = c.get<uint64_t>();
            if (!c.ok) return false;
            const int sz = scalar_size(v.arr_type);
            if (sz) {
                if (v.arr_n > (uint64_t)(c.end - c.p) / sz) return false;
                v.arr_data = c.p;
                c.skip(v.arr_n * sz);
            } else if (v.arr_type == G_STR) {
                if (v.arr_n > (uint64_t)(c.end - c.p) / 8) return false;  // every element has at least its length field
                v.arr_data = c.p;
                if (depth == 0) v.arr_items.reserve((size_t)v.arr_n);
                for (uint64_t i = 0; i < v.arr_n && c.ok; ++i) {
                    if (depth == 0) v.arr_items.push_back(c.p);
                    const uint64_t n = c.get<uint64_t>();
                    c.skip(n);
                }
            } else if (v.arr_type == G_ARR) {
                GgufValue inner;
                for (uint64_t i = 0; i < v.arr_n && c.ok; ++i)
                    if (!read_value(c, G_ARR, inner, depth + 1)) return false;
            } else {
                return false;
            }
            break;
        }
        default: return false;
    }
    return c.ok;
}

static int64_t tensor_bytes(uint32_t ggml_type, uint64_t n_elems) {
    switch (ggml_type) {
        case 0: return (int64_t)n_elems * 4;                               // F32
        case 1: return (int64_t)n_elems * 2;                               // F16
        case PTM_TYPE_Q4_K: return n_elems % 256 ? -1 : (int64_t)(n_elems / 256) * 144;
        case PTM_TYPE_Q6_K: return n_elems % 256 ? -1 : (int64_t)(n_elems / 256) * 210;
        case PTM_TYPE_Q5_K: return n_elems % 256 ? -1 : (int64_t)(n_elems / 256) * 176;
        case PTM_TYPE_Q8_0: return n_elems % 32 ? -1 : (int64_t)(n_elems / 32) * 34;
        case PTM_TYPE_Q5_0: return n_elems % 32 ? -1 : (int64_t)(n_elems / 32) * 22;
        default: return -1;  // a type this reader does not size; the tensor stays listed with nbytes = -1
    }
}

}  // namespace ptm

using namespace ptm;

struct ptm_gguf {
    int fd = -1;
    const uint8_t* map = nullptr;
    size_t map_size = 0;
    uint32_t version = 0;
    uint64_t alignment = 32;
    const uint8_t* data = nullptr;  // start of the tensor data section
    std::map<std::string, GgufValue> kv;
    std::vector<std::string> names;
    std::vector<ptm_gguf_tensor> tensors;
    std::map<std::string, size_t> index;
};

struct ptm_model {
    ptm_gguf* file = nullptr;
    std::vector<void*> device_allocs;
    std::vector<ptm_layer> layers;
    ptm_decode_config cfg{};
    ptm_decoder* dec = nullptr;
};

extern "C" {

void ptm_gguf_close(ptm_gguf* g) {
    if (!g) return;
    if (g->map) munmap(const_cast<uint8_t*>(g->map), g->map_size);
    if (g->fd >= 0) close(g->fd);
    delete g;
}

int ptm_gguf_open(const char* path, ptm_gguf** out) {
    if (!path || !out) return PTM_E_NULL;
    *out = nullptr;
    ptm_gguf* g = new (std::nothrow) ptm_gguf();
    if (!g) return PTM_E_STATE;
    g->fd = open(path, O_RDONLY);
    struct stat st{};
    if (g->fd < 0 || fstat(g->fd, &st) != 0 || st.st_size < 24) { ptm_gguf_close(g); return PTM_E_IO; }
    g->map_size = (size_t)st.st_size;
    void* m = mmap(nullptr, g->map_size, PROT_READ, MAP_PRIVATE, g->fd, 0);
    if (m == MAP_FAILED) { g->map = nullptr; ptm_gguf_close(g); return PTM_E_IO; }
    g->map = static_cast<const uint8_t*>(m);
    Cursor c{g->map, g->map + g->map_size};
    if (c.get<uint32_t>() != 0x46554747u) { ptm_gguf_close(g); return PTM_E_FORMAT; }
    g->version = c.get<uint32_t>();
    if (g->version < 2 || g->version > 3) { ptm_gguf_close(g); return PTM_E_UNSUPPORTED; }
    const uint64_t n_tensors = c.get<uint64_t>(), n_kv = c.get<uint64_t>();
    if (!c.ok || n_tensors > (1u << 20) || n_kv > (1u << 20)) { ptm_gguf_close(g); return PTM_E_FORMAT; }
    for (uint64_t i = 0; i < n_kv; ++i) {
        std::string key = c.str();
        const uint32_t type = c.get<uint32_t>();
        GgufValue v;
        if (!c.ok || !read_value(c, type, v, 0)) { ptm_gguf_close(g); return PTM_E_FORMAT; }
        g->kv.emplace(std::move(key), std::move(v));
    }
    auto al = g->kv.find("general.alignment");
    if (al != g->kv.end() && al->second.type != G_STR && al->second.type != G_ARR && al->second.u > 0) g->alignment = al->second.u;
    if (g->alignment > (1u << 20) || (g->alignment & (g->alignment - 1))) { ptm_gguf_close(g); return PTM_E_FORMAT; }
    std::vector<uint64_t> offsets;
    g->names.reserve(n_tensors);
    for (uint64_t i = 0; i < n_tensors; ++i) {
        g->names.push_back(c.str());
        ptm_gguf_tensor t{};
        t.n_dims = (int32_t)c.get<uint32_t>();
        if (!c.ok || t.n_dims < 1 || t.n_dims > 4) { ptm_gguf_close(g); return PTM_E_FORMAT; }
        uint64_t n = 1;
        for (int d = 0; d < 4; ++d) t.dims[d] = 1;
        for (int d = 0; d < t.n_dims; ++d) {
            const uint64_t dim = c.get<uint64_t>();
            if (!c.ok || dim == 0 || dim > (1ull << 40) || n > (1ull << 50) / dim) { ptm_gguf_close(g); return PTM_E_FORMAT; }
            t.dims[d] = (int64_t)dim;
            n *= dim;
        }
        t.ggml_type = c.get<uint32_t>();
        offsets.push_back(c.get<uint64_t>());
        if (!c.ok) { ptm_gguf_close(g); return PTM_E_FORMAT; }
        t.nbytes = tensor_bytes(t.ggml_type, n);
        g->tensors.push_back(t);
    }
    const uint64_t pos = (uint64_t)(c.p - g->map);
    const uint64_t data_off = (pos + g->alignment - 1) / g->alignment * g->alignment;
    if (data_off > g->map_size) { ptm_gguf_close(g); return PTM_E_FORMAT; }
    g->data = g->map + data_off;
    const uint64_t data_size = g->map_size - data_off;
    for (size_t i = 0; i < g->tensors.size(); ++i) {
        ptm_gguf_tensor& t = g->tensors[i];
        t.name = g->names[i].c_str();
        if (offsets[i] % g->alignment) { ptm_gguf_close(g); return PTM_E_FORMAT; }
        if (offsets[i] > data_size || (t.nbytes >= 0 && (uint64_t)t.nbytes > data_size - offsets[i])) { ptm_gguf_close(g); return PTM_E_FORMAT; }
        t.data = g->data + offsets[i];
        g->index[g->names[i]] = i;
    }
    *out = g;
    return PTM_OK;
}

int ptm_gguf_version(const ptm_gguf* g) { return g ? (int)g->version : 0; }
int64_t ptm_gguf_alignment(const ptm_gguf* g) { return g ? (int64_t)g->alignment : 0; }
int64_t ptm_gguf_n_tensors(const ptm_gguf* g) { return g ? (int64_t)g->tensors.size() : 0; }

int ptm_gguf_tensor_at(const ptm_gguf* g, int64_t i, ptm_gguf_tensor* out) {
    if (!g || !out) return PTM_E_NULL;
    if (i < 0 || (size_t)i >= g->tensors.size()) return PTM_E_RANGE;
    *out = g->tensors[(size_t)i];
    return PTM_OK;
}

int ptm_gguf_find_tensor(const ptm_gguf* g, const char* name, ptm_gguf_tensor* out) {
    if (!g || !name || !out) return PTM_E_NULL;
    auto it = g->index.find(name);
    if (it == g->index.end()) return PTM_E_NOT_FOUND;
    *out = g->tensors[it->second];
    return PTM_OK;
}

int ptm_gguf_get_int(const ptm_gguf* g, const char* key, int64_t* out) {
    if (!g || !key || !out) return PTM_E_NULL;
    auto it = g->kv.find(key);
    if (it == g->kv.end()) return PTM_E_NOT_FOUND;
    const GgufValue& v = it->second;
    if (v.type == G_STR || v.type == G_ARR || v.type == G_F32 || v.type == G_F64) return PTM_E_FORMAT;
    *out = (int64_t)v.u;
    return PTM_OK;
}

int ptm_gguf_get_float(const ptm_gguf* g, const char* key, double* out) {
    if (!g || !key || !out) return PTM_E_NULL;
    auto it = g->kv.find(key);
    if (it == g->kv.end()) return PTM_E_NOT_FOUND;
    const GgufValue& v = it->second;
    if (v.type == G_F32 || v.type == G_F64) *out = v.f;
    else if (v.type == G_STR || v.type == G_ARR) return PTM_E_FORMAT;
    else *out = (double)(int64_t)v.u;
    return PTM_OK;
}

const char* ptm_gguf_get_string(const ptm_gguf* g, const char* key) {
    if (!g || !key) return nullptr;
    auto it = g->kv.find(key);
    return (it == g->kv.end() || it->second.type != G_STR) ? nullptr : it->second.s.c_str();
}

int ptm_gguf_get_array(const ptm_gguf* g, const char* key, uint32_t* elem_type, int64_t* count) {
    if (!g || !key) return PTM_E_NULL;
    auto it = g->kv.find(key);
    if (it == g->kv.end()) return PTM_E_NOT_FOUND;
    if (it->second.type != G_ARR) return PTM_E_FORMAT;
    if (elem_type) *elem_type = it->second.arr_type;
    if (count) *count = (int64_t)it->second.arr_n;
    return PTM_OK;
}

int ptm_gguf_array_string(const ptm_gguf* g, const char* key, int64_t i, const char** data, int64_t* len) {
    if (!g || !key || !data || !len) return PTM_E_NULL;
    auto it = g->kv.find(key);
    if (it == g->kv.end()) return PTM_E_NOT_FOUND;
    const GgufValue& v = it->second;
    if (v.type != G_ARR || v.arr_type != G_STR) return PTM_E_FORMAT;
    if (i < 0 || (uint64_t)i >= v.arr_items.size()) return PTM_E_RANGE;
    uint64_t n;
    memcpy(&n, v.arr_items[(size_t)i], 8);  // bounds were checked when the file was parsed
    *data = reinterpret_cast<const char*>(v.arr_items[(size_t)i] + 8);
    *len = (int64_t)n;
    return PTM_OK;
}

const void* ptm_gguf_array_data(const ptm_gguf* g, const char* key) {
    if (!g || !key) return nullptr;
    auto it = g->kv.find(key);
    if (it == g->kv.end() || it->second.type != G_ARR || !scalar_size(it->second.arr_type)) return nullptr;
    return it->second.arr_data;
}

// ---------------------------------------------------------------------------------------------------------------
// model loader
// ---------------------------------------------------------------------------------------------------------------
void ptm_model_free(ptm_model* m) {
    if (!m) return;
    if (m->dec) ptm_decode_destroy(m->dec);
    for (void* p : m->device_allocs) (void)hipFree(p);
    if (m->file) ptm_gguf_close(m->file);
    delete m;
}

static int upload(ptm_model* m, const void* src, size_t bytes, void** dev) {
    void* d = nullptr;
    int rc = hip_status(hipMalloc(&d, bytes));
    if (rc != PTM_OK) return rc;
    m->device_allocs.push_back(d);
    if (src) rc = hip_status(hipMemcpy(d, src, bytes, hipMemcpyHostToDevice));
    else rc = hip_status(hipMemset(d, 0, bytes));
    *dev = d;
    return rc;
}

// a [rows x cols] Q4_K / Q6_K matrix: uploaded verbatim
static int load_matrix(ptm_model* m, const std::string& name, int64_t rows, int64_t cols, ptm_qweight* w) {
    ptm_gguf_tensor t{};
    int rc = ptm_gguf_find_tensor(m->file, name.c_str(), &t);
    if (rc != PTM_OK) return rc;
    int blk_bytes = 0, blk_vals = 0;
    switch (t.ggml_type) {  // the GEMV dispatcher's formats (gguf_dequant.h:29-58)
        case PTM_TYPE_Q4_K: blk_bytes = 144; blk_vals = 256; break;
        case PTM_TYPE_Q6_K: blk_bytes = 210; blk_vals = 256; break;
        case PTM_TYPE_Q5_K: blk_bytes = 176; blk_vals = 256; break;
        case PTM_TYPE_Q8_0: blk_bytes = 34; blk_vals = 32; break;
        case PTM_TYPE_Q5_0: blk_bytes = 22; blk_vals = 32; break;
        default: return PTM_E_UNSUPPORTED;
    }
    if (t.n_dims != 2 || t.dims[0] != cols || t.dims[1] != rows || t.nbytes <= 0 || cols % blk_vals != 0) return PTM_E_SHAPE;
    void* d = nullptr;
    if ((rc = upload(m, t.data, (size_t)t.nbytes, &d)) != PTM_OK) return rc;
    w->data = d;
    w->ggml_type = t.ggml_type;
    w->rows = (int32_t)rows;
    w->cols = (int32_t)cols;
    w->row_stride_bytes = cols / blk_vals * blk_bytes;
    return PTM_OK;
}

static int load_vector(ptm_model* m, const std::string& name, int64_t n, const float** out) {
    ptm_gguf_tensor t{};
    int rc = ptm_gguf_find_tensor(m->file, name.c_str(), &t);
    if (rc != PTM_OK) return rc;
    if (t.ggml_type != 0) return PTM_E_UNSUPPORTED;  // norm weights are stored as F32
    if (t.n_dims != 1 || t.dims[0] != n) return PTM_E_SHAPE;
    void* d = nullptr;
    if ((rc = upload(m, t.data, (size_t)n * 4, &d)) != PTM_OK) return rc;
    *out = static_cast<const float*>(d);
    return PTM_OK;
}

int ptm_model_load_gguf(const char* path, int max_seq, int kv_fp16, int use_graph, ptm_model** out) {
    if (!path || !out) return PTM_E_NULL;
    *out = nullptr;
    if (max_seq <= 0) return PTM_E_SHAPE;
    ptm_model* m = new (std::nothrow) ptm_model();
    if (!m) return PTM_E_STATE;
    int rc = ptm_gguf_open(path, &m->file);
    if (rc != PTM_OK) { ptm_model_free(m); return rc; }
#define PTM_L(x) do { rc = (x); if (rc != PTM_OK) { ptm_model_free(m); return rc; } } while (0)
    const char* arch_c = ptm_gguf_get_string(m->file, "general.architecture");
    if (!arch_c) { ptm_model_free(m); return PTM_E_FORMAT; }
    const std::string arch = arch_c;
    // three decode steps are built here, all RMSNorm + SwiGLU: qwen3 (per-head QK-norm, rotation pairs half a head
    // apart), qwen2 (no QK-norm, the same pairs, bias vectors on q / k / v) and llama, which mistral files also carry
    // (no QK-norm, interleaved pairs (2d, 2d+1)); gguf_model.h:194-217 makes the same split by architecture name
    // gemma3 (gguf_model.h:157-197): QK-norm, NeoX pairs, embedding rows times sqrt(hidden), tanh-GELU gate, post-norm
    // vectors, sliding-window layers (every sliding_window_pattern-th layer global, 6 when the key is missing) with
    // their own rotation base
    const bool is_llama = arch == "llama";
    const bool is_gemma3 = arch == "gemma3";
    const bool has_qk_norm = arch == "qwen3" || is_gemma3;
    if (arch != "qwen3" && arch != "qwen2" && !is_llama && !is_gemma3) { ptm_model_free(m); return PTM_E_UNSUPPORTED; }
    auto geti = [&](const char* key, int64_t def, bool required) -> int64_t {
        int64_t v = def;
        const int r = ptm_gguf_get_int(m->file, (arch + "." + key).c_str(), &v);
        if (r != PTM_OK && required) rc = r == PTM_E_NOT_FOUND ? PTM_E_FORMAT : r;
        return v;
    };
    rc = PTM_OK;
    ptm_decode_config& c = m->cfg;
    c.hidden = (int32_t)geti("embedding_length", 0, true);
    c.n_layers = (int32_t)geti("block_count", 0, true);
    c.n_heads = (int32_t)geti("attention.head_count", 0, true);
    c.n_kv_heads = (int32_t)geti("attention.head_count_kv", c.n_heads, false);
    c.inter = (int32_t)geti("feed_forward_length", 0, true);
    if (rc != PTM_OK) { ptm_model_free(m); return rc; }
    if (c.hidden <= 0 || c.n_layers <= 0 || c.n_heads <= 0 || c.n_kv_heads <= 0 || c.inter <= 0 || c.n_layers > 4096) { ptm_model_free(m); return PTM_E_FORMAT; }
    const int64_t key_len = geti("attention.key_length", 0, false);
    c.head_dim = (int32_t)(key_len > 0 ? key_len : c.hidden / c.n_heads);  // gguf_model.h:179-181
    double fv = 10000.0;
    (void)ptm_gguf_get_float(m->file, (arch + ".rope.freq_base").c_str(), &fv);
    c.rope_freq_base = (float)fv;
    {   // linear position scaling: rope.scaling.type == "linear" with a factor above 1, else the older
        // rope.scale_linear key (gguf_model.h:136-156); other scaling types leave the positions as they are
        c.rope_scale = 1.0f;
        const char* st = ptm_gguf_get_string(m->file, (arch + ".rope.scaling.type").c_str());
        double f = 0.0;
        if (st && std::string(st) == "linear" &&
            ptm_gguf_get_float(m->file, (arch + ".rope.scaling.factor").c_str(), &f) == PTM_OK && (float)f > 1.0f)
            c.rope_scale = (float)f;
        if (c.rope_scale == 1.0f && ptm_gguf_get_float(m->file, (arch + ".rope.scale_linear").c_str(), &f) == PTM_OK &&
            (float)f > 1.0f)
            c.rope_scale = (float)f;
    }
    fv = 1e-6;
    (void)ptm_gguf_get_float(m->file, (arch + ".attention.layer_norm_rms_epsilon").c_str(), &fv);
    c.rms_eps = (float)fv;
    c.max_seq = max_seq;
    c.kv_fp16 = kv_fp16 ? 1 : 0;
    c.use_graph = use_graph ? 1 : 0;
    c.rope_interleaved = is_llama ? 1 : 0;
    if (is_gemma3) {
        c.scale_embeddings = 1;
        c.ffn_gelu = 1;
        c.swa_window = (int32_t)geti("attention.sliding_window", 0, false);
        c.swa_pattern = (int32_t)geti("attention.sliding_window_pattern", 0, false);
        if (c.swa_window > 0 && c.swa_pattern == 0) c.swa_pattern = 6;  // gguf_model.h:166-170
        double fb = 10000.0;
        (void)ptm_gguf_get_float(m->file, (arch + ".rope.freq_base_swa").c_str(), &fb);
        c.rope_swa_freq_base = (float)fb;
    }
    // vocabulary size from the embedding table [hidden x vocab]
    ptm_gguf_tensor emb{};
    PTM_L(ptm_gguf_find_tensor(m->file, "token_embd.weight", &emb));
    if (emb.n_dims != 2 || emb.dims[0] != c.hidden) { ptm_model_free(m); return PTM_E_SHAPE; }
    c.vocab = (int32_t)emb.dims[1];
    const int64_t qd = (int64_t)c.n_heads * c.head_dim, kvd = (int64_t)c.n_kv_heads * c.head_dim;

    // output projection: output.weight, or the embedding table when the model ties them
    ptm_gguf_tensor outw{};
    const bool tied = ptm_gguf_find_tensor(m->file, "output.weight", &outw) != PTM_OK;
    PTM_L(load_matrix(m, tied ? "token_embd.weight" : "output.weight", c.vocab, c.hidden, &c.lm_head));
    if (tied && c.lm_head.ggml_type == PTM_TYPE_Q6_K) {
        c.embedding_f32 = nullptr;  // embedding rows are dequantised from the shared Q6_K table on the fly
    } else {
        // separate (or Q4_K) embedding table: dequantise it once to fp32 on the device (gguf_model.h:6774)
        ptm_qweight ew{};
        if (tied) ew = c.lm_head;
        else PTM_L(load_matrix(m, "token_embd.weight", c.vocab, c.hidden, &ew));
        void* table = nullptr;
        const int64_t n = (int64_t)c.vocab * c.hidden;
        PTM_L(upload(m, nullptr, (size_t)n * 4, &table));
        switch (ew.ggml_type) {
            case PTM_TYPE_Q4_K: PTM_L(ptm_dequant_q4k(ew.data, static_cast<float*>(table), n, nullptr)); break;
            case PTM_TYPE_Q6_K: PTM_L(ptm_dequant_q6k(ew.data, static_cast<float*>(table), n, nullptr)); break;
            case PTM_TYPE_Q5_K: PTM_L(ptm_dequant_q5k(ew.data, static_cast<float*>(table), n, nullptr)); break;
            case PTM_TYPE_Q8_0: PTM_L(ptm_dequant_q8_0(ew.data, static_cast<float*>(table), n, nullptr)); break;
            default: ptm_model_free(m); return PTM_E_UNSUPPORTED;  // the reference has no Q5_0 dequantiser either
        }
        PTM_L(hip_status(hipDeviceSynchronize()));
        c.embedding_f32 = static_cast<const float*>(table);
    }
    PTM_L(load_vector(m, "output_norm.weight", c.hidden, &c.out_norm));

    m->layers.resize((size_t)c.n_layers);
    const size_t kv_bytes = (size_t)max_seq * (size_t)kvd * (kv_fp16 ? 2 : 4);
    for (int i = 0; i < c.n_layers; ++i) {
        ptm_layer& L = m->layers[(size_t)i];
        const std::string p = "blk." + std::to_string(i) + ".";
        ptm_gguf_tensor bias{};
        if (ptm_gguf_find_tensor(m->file, (p + "attn_q.bias").c_str(), &bias) == PTM_OK) {  // gguf_model.h:6750-6754
            PTM_L(load_vector(m, p + "attn_q.bias", qd, &L.q_bias));
            PTM_L(load_vector(m, p + "attn_k.bias", kvd, &L.k_bias));
            PTM_L(load_vector(m, p + "attn_v.bias", kvd, &L.v_bias));
        }
        PTM_L(load_vector(m, p + "attn_norm.weight", c.hidden, &L.attn_norm));
        PTM_L(load_matrix(m, p + "attn_q.weight", qd, c.hidden, &L.q));
        PTM_L(load_matrix(m, p + "attn_k.weight", kvd, c.hidden, &L.k));
        PTM_L(load_matrix(m, p + "attn_v.weight", kvd, c.hidden, &L.v));
        PTM_L(load_matrix(m, p + "attn_output.weight", c.hidden, qd, &L.o));
        if (!has_qk_norm) {
            L.q_norm = nullptr;
            L.k_norm = nullptr;
        } else {
            PTM_L(load_vector(m, p + "attn_q_norm.weight", c.head_dim, &L.q_norm));
            PTM_L(load_vector(m, p + "attn_k_norm.weight", c.head_dim, &L.k_norm));
        }
        if (is_gemma3) {  // LayerWeights::post_attention_norm / post_ffw_norm
            PTM_L(load_vector(m, p + "post_attention_norm.weight", c.hidden, &L.post_attn_norm));
            PTM_L(load_vector(m, p + "post_ffw_norm.weight", c.hidden, &L.post_ffn_norm));
        }
        PTM_L(load_vector(m, p + "ffn_norm.weight", c.hidden, &L.ffn_norm));
        PTM_L(load_matrix(m, p + "ffn_gate.weight", c.inter, c.hidden, &L.gate));
        PTM_L(load_matrix(m, p + "ffn_up.weight", c.inter, c.hidden, &L.up));
        PTM_L(load_matrix(m, p + "ffn_down.weight", c.hidden, c.inter, &L.down));
        PTM_L(upload(m, nullptr, kv_bytes, &L.k_cache));
        PTM_L(upload(m, nullptr, kv_bytes, &L.v_cache));
    }
    c.layers = m->layers.data();
    PTM_L(ptm_decode_create(&c, &m->dec));
#undef PTM_L
    *out = m;
    return PTM_OK;
}

ptm_decoder* ptm_model_decoder(ptm_model* m) { return m ? m->dec : nullptr; }

int ptm_model_config(const ptm_model* m, ptm_decode_config* out) {
    if (!m || !out) return PTM_E_NULL;
    *out = m->cfg;
    return PTM_OK;
}

int ptm_model_layer(const ptm_model* m, int i, ptm_layer* out) {
    if (!m || !out) return PTM_E_NULL;
    if (i < 0 || (size_t)i >= m->layers.size()) return PTM_E_RANGE;
    *out = m->layers[(size_t)i];
    return PTM_OK;
}

}  // extern "C"
