// TEST INFRASTRUCTURE ONLY — thin extern "C" harness around the *reference's own*
// CPU implementation of the GGUF k-quant decode path.  It contains no arithmetic of
// its own: every function forwards to a symbol defined in the reference's headers,
// which are compiled from where they lie (the reference checkout passed as REF=...
// to oracle/Makefile).  The resulting library (oracle/_ref/libptm_ref.so) is used to
// (1) validate oracle/ptm_oracle.c, (2) write the golden fixtures under tests/golden/,
// and (3) optionally serve as the "reference" CPU baseline.  Nothing in the product
// path links or loads it.
#include <cstdint>
#include <cstring>
#include <vector>
#include <memory>

#include "torch/io/gguf_dequant.h"
#include "torch/io/cpu_quant_gemv.h"
#include "torch/io/gguf_model.h"

using torch::io::GGUFModel;
namespace q = torch::io::cpu_quant;
namespace g = torch::io::gguf;

extern "C" {

// torch/io/gguf_dequant.h:73
float ref_fp16_to_fp32(uint16_t h) { return g::fp16_to_fp32(h); }
// torch/io/gguf_dequant.h:289
void ref_get_scale_min_k4(int j, const uint8_t* s, uint8_t* d, uint8_t* m) { g::get_scale_min_k4(j, s, d, m); }
// torch/io/gguf_dequant.h:304
void ref_dequantize_q4_k(const void* src, float* dst, int64_t n) { g::dequantize_q4_k(src, dst, n); }
// torch/io/gguf_dequant.h:395
void ref_dequantize_q6_k(const void* src, float* dst, int64_t n) { g::dequantize_q6_k(src, dst, n); }
// torch/io/gguf_dequant.h:237, :348
void ref_dequantize_q8_0(const void* src, float* dst, int64_t n) { g::dequantize_q8_0(src, dst, n); }
void ref_dequantize_q5_k(const void* src, float* dst, int64_t n) { g::dequantize_q5_k(src, dst, n); }

// torch/io/cpu_quant_gemv.h:147 — the Q8Block struct is alignas(32) (64 B); unpack to flat arrays.
void ref_quantize_x_q8(const float* x, int64_t K, float* d_out, float* sum_out, int8_t* qs_out) {
    const int64_t nb = K / 32;
    std::vector<q::Q8Block> blk(nb);
    q::quantize_x_q8(x, blk.data(), K);
    for (int64_t i = 0; i < nb; ++i) {
        d_out[i] = blk[i].d; sum_out[i] = blk[i].sum;
        std::memcpy(qs_out + i * 32, blk[i].qs, 32);
    }
}
// torch/io/cpu_quant_gemv.h:1635
void ref_cpu_quant_gemv(uint32_t type, const void* W, const float* x, float* y,
                        int64_t K, int64_t N, int64_t stride) {
    q::cpu_quant_gemv(type, W, x, y, K, N, stride, nullptr);
}
// torch/io/cpu_quant_gemv.h:689 / :1024 / :62 — fp32-activation cross-check variants
void ref_q4k_gemv_scalar(const void* W, const float* x, float* y, int64_t K, int64_t N, int64_t stride) {
    q::q4k_gemv_scalar(W, x, y, K, N, stride, nullptr);
}
void ref_q6k_gemv_scalar(const void* W, const float* x, float* y, int64_t K, int64_t N, int64_t stride) {
    q::q6k_gemv_scalar(W, x, y, K, N, stride, nullptr);
}
// torch/io/cpu_quant_gemv.h:2423
void ref_fused_rmsnorm_gate_up(const float* x, const float* gamma, float eps, int add_one,
                               uint32_t tg, const void* wg, uint32_t tu, const void* wu,
                               float* yg, float* yu, int64_t H, int64_t Ng, int64_t Nu,
                               int64_t sg, int64_t su) {
    q::cpu_fused_rmsnorm_gate_up_gemv(x, gamma, eps, add_one != 0, tg, wg, tu, wu, yg, yu, H, Ng, Nu, sg, su);
}
// torch/io/cpu_quant_gemv.h:2567
void ref_rmsnorm_inplace(float* x, const float* gamma, float eps, int add_one, int64_t H) {
    q::cpu_rmsnorm_inplace(x, gamma, eps, add_one != 0, H);
}
// aten/src/ATen/native/cpu/hot_loops.cpp:1853
void ref_rope_precompute(float* c, float* s, int64_t pos, int64_t head_dim, float base) {
    at::native::hot::rope_precompute(c, s, pos, head_dim, base, 1.0f, nullptr, 1.0f);
}
// aten/src/ATen/native/cpu/hot_loops.cpp:2035
void ref_rope_apply_neox(float* qv, float* kv, const float* c, const float* s,
                         int64_t nh, int64_t nkv, int64_t hd) {
    at::native::hot::rope_apply_fused_neox(qv, kv, c, s, nh, nkv, hd);
}
// aten/src/ATen/native/cpu/VectorizedOps.h:56
void ref_exp256(const float* in, float* out, int64_t n8) {
    for (int64_t i = 0; i < n8; ++i)
        _mm256_storeu_ps(out + 8 * i, at::native::vec::exp256_ps(_mm256_loadu_ps(in + 8 * i)));
}
void ref_rope_apply_norm(float* qv, float* kv, const float* c, const float* s,
                         int64_t n_heads, int64_t n_kv_heads, int64_t head_dim) {
    at::native::hot::rope_apply_fused(qv, kv, c, s, n_heads, n_kv_heads, head_dim);
}
int ref_num_threads() { return c10::get_thread_pool().num_threads(); }

// ---------------------------------------------------------------------------------
// Whole-model decode: a GGUFModel populated directly from caller-owned host buffers
// (no .gguf file), stepped with the reference's forward_decode_cpu
// (torch/io/gguf_model.h:3222) and its greedy argmax (:4864-4901).
// ---------------------------------------------------------------------------------
struct RefModel { GGUFModel m; };

void* ref_model_create(int64_t vocab, int64_t hidden, int64_t n_layers, int64_t n_heads,
                       int64_t n_kv_heads, int64_t head_dim, int64_t inter,
                       float rope_base, float eps, int64_t max_seq) {
    auto* r = new RefModel();
    auto& c = r->m.config;
    c.architecture = "qwen3";
    c.vocab_size = vocab; c.hidden_size = hidden; c.num_layers = n_layers;
    c.num_heads = n_heads; c.num_kv_heads = n_kv_heads; c.head_dim = head_dim;
    c.intermediate_size = inter; c.context_length = max_seq;
    c.rope_freq_base = rope_base; c.rms_norm_eps = eps;
    c.has_qk_norm = true; c.rope_neox = true; c.tie_word_embeddings = true;
    r->m.layers.resize(n_layers);
    r->m.use_quant_gemv_ = true;
    r->m.use_cuda_ = false;
    r->m.kv_cache.allocate(n_layers, max_seq, n_kv_heads * head_dim, false);
    return r;
}
// llama-style models: no per-head QK-norm (the norm tensors stay undefined: never call ref_model_set_norm with which 2, 3)
// and interleaved rotation pairs (config.rope_neox, gguf_model.h:98)
void ref_model_set_arch(void* h, int has_qk_norm, int rope_neox) {
    auto& c = static_cast<RefModel*>(h)->m.config;
    c.has_qk_norm = has_qk_norm != 0;
    c.rope_neox = rope_neox != 0;
}
// gemma-family switches of ModelConfig (gguf_model.h:74-88, :184-197): embedding scaling, tanh-GELU gate, post-norms,
// alternating sliding-window layers with their own rotation base
void ref_model_set_gemma(void* h, int scale_embeddings, int ffn_gelu, int has_post_norm, int64_t swa_window,
                         int64_t swa_pattern, float rope_swa_base) {
    auto& c = static_cast<RefModel*>(h)->m.config;
    c.scale_embeddings = scale_embeddings != 0;
    c.ffn_gelu = ffn_gelu != 0;
    c.has_post_norm = has_post_norm != 0;
    c.swa_window = swa_window; c.swa_pattern = swa_pattern;
    c.rope_swa_freq_base = rope_swa_base; c.rope_swa_scale = 1.0f;
}
// linear rotary position scaling (ModelConfig::rope_scale, gguf_model.h:71, read from rope.scaling.* at :136-156)
void ref_model_set_rope_scale(void* h, float scale) { static_cast<RefModel*>(h)->m.config.rope_scale = scale; }
void ref_rope_precompute_scaled(float* c, float* s, int64_t pos, int64_t head_dim, float base, float scale) {
    at::native::hot::rope_precompute(c, s, pos, head_dim, base, scale, nullptr, 1.0f);
}
// phi3 LongRoPE fields of ModelConfig (gguf_model.h:89-96): per-frequency factor sets, the context length up to which the
// short set applies, and the factor cos / sin are scaled by
void ref_model_set_rope_factors(void* h, const float* fshort, int64_t n_short, const float* flong, int64_t n_long,
                                int64_t orig_ctx, float attn_factor) {
    auto& c = static_cast<RefModel*>(h)->m.config;
    c.rope_factors_short.assign(fshort, fshort + n_short);
    c.rope_factors_long.assign(flong, flong + n_long);
    c.rope_orig_ctx = orig_ctx;
    c.rope_attn_factor = attn_factor;
}
void ref_rope_precompute_factors(float* c, float* s, int64_t pos, int64_t head_dim, float base, float scale,
                                 const float* factors, float attn_factor) {
    at::native::hot::rope_precompute(c, s, pos, head_dim, base, scale, factors, attn_factor);
}
void ref_model_destroy(void* h) {
    auto* r = static_cast<RefModel*>(h);
    // weights are caller-owned: detach before QuantizedWeight could free them
    for (auto& L : r->m.layers) {
        for (auto* w : {&L.q_attn_q, &L.q_attn_k, &L.q_attn_v, &L.q_attn_output,
                        &L.q_ffn_gate, &L.q_ffn_up, &L.q_ffn_down}) w->cpu_data = nullptr;
    }
    r->m.q_output_weight.cpu_data = nullptr;
    delete r;
}
static at::Tensor vec_tensor(const float* src, int64_t n) {
    at::Tensor t = at::empty({n});
    std::memcpy(t.mutable_data_ptr<float>(), src, n * sizeof(float));
    return t;
}
static void set_qw(torch::io::QuantizedWeight& w, const void* data, uint32_t type, int64_t rows, int64_t cols) {
    w.cpu_data = const_cast<void*>(data);
    w.rows = rows; w.cols = cols; w.quant_type = type;
    // block sizes of the dispatcher's formats (torch/io/gguf_dequant.h:29-58)
    const int64_t blk_bytes = type == 12 ? 144 : type == 14 ? 210 : type == 13 ? 176 : type == 8 ? 34 : 22;
    w.row_stride_bytes = cols / (type == 8 || type == 6 ? 32 : 256) * blk_bytes;
    w.total_bytes = rows * w.row_stride_bytes;
    w.valid = true; w.mmap_owned = true; w.owns_cpu_data = false;
}
// which: 0 q,1 k,2 v,3 o,4 gate,5 up,6 down
void ref_model_set_weight(void* h, int64_t layer, int which, const void* data, uint32_t type,
                          int64_t rows, int64_t cols) {
    auto& L = static_cast<RefModel*>(h)->m.layers[layer];
    torch::io::QuantizedWeight* w[] = {&L.q_attn_q, &L.q_attn_k, &L.q_attn_v, &L.q_attn_output,
                                        &L.q_ffn_gate, &L.q_ffn_up, &L.q_ffn_down};
    set_qw(*w[which], data, type, rows, cols);
}
// which: 0 attn_norm, 1 ffn_norm, 2 q_norm, 3 k_norm, 4 / 5 / 6 attn_q / attn_k / attn_v bias (gguf_model.h:410-412),
// 7 post_attention_norm, 8 post_ffw_norm
void ref_model_set_norm(void* h, int64_t layer, int which, const float* gamma, int64_t n) {
    auto& L = static_cast<RefModel*>(h)->m.layers[layer];
    at::Tensor t = vec_tensor(gamma, n);
    if (which == 0) L.attn_norm = t; else if (which == 1) L.ffn_norm = t;
    else if (which == 2) L.attn_q_norm = t; else if (which == 3) L.attn_k_norm = t;
    else if (which == 4) L.attn_q_bias = t; else if (which == 5) L.attn_k_bias = t; else if (which == 6) L.attn_v_bias = t;
    else if (which == 7) L.post_attention_norm = t; else L.post_ffw_norm = t;
}
void ref_model_set_output(void* h, const float* out_norm, const void* lm_head, uint32_t type) {
    auto& m = static_cast<RefModel*>(h)->m;
    m.output_norm = vec_tensor(out_norm, m.config.hidden_size);
    set_qw(m.q_output_weight, lm_head, type, m.config.vocab_size, m.config.hidden_size);
}
// fp32 token-embedding table [vocab, hidden]; copied into a reference Tensor.
void ref_model_set_embedding(void* h, const float* table) {
    auto& m = static_cast<RefModel*>(h)->m;
    m.token_embedding = at::empty({m.config.vocab_size, m.config.hidden_size});
    std::memcpy(m.token_embedding.mutable_data_ptr<float>(), table,
                sizeof(float) * m.config.vocab_size * m.config.hidden_size);
}
// Fill positions [0, n_pos) of layer's fp32 K/V cache and set seq_len = n_pos.
void ref_model_set_kv(void* h, int64_t layer, const float* k, const float* v, int64_t n_pos) {
    auto& m = static_cast<RefModel*>(h)->m;
    const int64_t kv_dim = m.config.num_kv_heads * m.config.head_dim;
    std::memcpy(m.kv_cache.key_cache[layer].mutable_data_ptr<float>(), k, sizeof(float) * n_pos * kv_dim);
    std::memcpy(m.kv_cache.value_cache[layer].mutable_data_ptr<float>(), v, sizeof(float) * n_pos * kv_dim);
    m.kv_cache.seq_len = n_pos;
}
// Copy out the rows appended at position pos (to let a caller round them to fp16).
void ref_model_get_kv_row(void* h, int64_t layer, int64_t pos, float* k, float* v) {
    auto& m = static_cast<RefModel*>(h)->m;
    const int64_t kv_dim = m.config.num_kv_heads * m.config.head_dim;
    std::memcpy(k, m.kv_cache.key_cache[layer].data_ptr<float>() + pos * kv_dim, sizeof(float) * kv_dim);
    std::memcpy(v, m.kv_cache.value_cache[layer].data_ptr<float>() + pos * kv_dim, sizeof(float) * kv_dim);
}
void ref_model_put_kv_row(void* h, int64_t layer, int64_t pos, const float* k, const float* v) {
    auto& m = static_cast<RefModel*>(h)->m;
    const int64_t kv_dim = m.config.num_kv_heads * m.config.head_dim;
    std::memcpy(m.kv_cache.key_cache[layer].mutable_data_ptr<float>() + pos * kv_dim, k, sizeof(float) * kv_dim);
    std::memcpy(m.kv_cache.value_cache[layer].mutable_data_ptr<float>() + pos * kv_dim, v, sizeof(float) * kv_dim);
}
int64_t ref_model_seq_len(void* h) { return static_cast<RefModel*>(h)->m.kv_cache.seq_len; }
// One forward_decode_cpu step; writes logits[vocab]; returns greedy argmax (strict '>', first max).
int64_t ref_model_decode(void* h, int64_t token, float* logits_out) {
    auto& m = static_cast<RefModel*>(h)->m;
    at::Tensor lg = m.forward_decode_cpu(token);
    const float* p = lg.data_ptr<float>();
    const int64_t V = m.config.vocab_size;
    if (logits_out) std::memcpy(logits_out, p, sizeof(float) * V);
    int64_t best = 0; float bv = p[0];
    for (int64_t j = 1; j < V; ++j) if (p[j] > bv) { bv = p[j]; best = j; }
    return best;
}
// GGUFModel::sample_token (torch/io/gguf_model.h:7658-7751).  Its generator is a function-local
// `static std::mt19937 rng(42)`: the n-th sampling call of a process (temperature >= 1e-6) uses the n-th draw.
int32_t ref_sample_token(void* h, const float* logits, int64_t vocab, float temperature, int top_k, float top_p) {
    return static_cast<RefModel*>(h)->m.sample_token(vec_tensor(logits, vocab), temperature, top_k, top_p);
}

// ---------------------------------------------------------------------------------
// GGUFTokenizer (torch/io/tokenizer.h) loaded by the reference's own GGUFReader (torch/io/gguf_loader.h) from a
// .gguf file, and GGUFModel::apply_chat_template (torch/io/gguf_model.h:4178-4236).
// ---------------------------------------------------------------------------------
void* ref_tokenizer_load(const char* gguf_path) {
    g::GGUFReader reader;
    reader.open(gguf_path);
    auto* t = new torch::io::GGUFTokenizer();
    t->load(reader);
    return t;
}
void ref_tokenizer_free(void* h) { delete static_cast<torch::io::GGUFTokenizer*>(h); }
int64_t ref_tokenizer_encode(void* h, const char* text, int64_t len, int use_bos, int32_t* out, int64_t cap) {
    const auto ids = static_cast<torch::io::GGUFTokenizer*>(h)->encode(std::string(text, (size_t)len), use_bos != 0);
    for (size_t i = 0; i < ids.size() && (int64_t)i < cap; ++i) out[i] = ids[i];
    return (int64_t)ids.size();
}
int64_t ref_tokenizer_decode(void* h, const int32_t* ids, int64_t n, int skip_special, char* out, int64_t cap) {
    const std::string s = static_cast<torch::io::GGUFTokenizer*>(h)->decode(std::vector<int32_t>(ids, ids + n), skip_special != 0);
    memcpy(out, s.data(), (size_t)std::min<int64_t>(cap, (int64_t)s.size()));
    return (int64_t)s.size();
}
int64_t ref_tokenizer_token(void* h, int32_t id, char* out, int64_t cap) {
    const std::string s = static_cast<torch::io::GGUFTokenizer*>(h)->decode_token(id);
    memcpy(out, s.data(), (size_t)std::min<int64_t>(cap, (int64_t)s.size()));
    return (int64_t)s.size();
}
// architecture / model name as the reference keeps them in its config; the system prompt and the no-think switch
// are read from the environment by the reference itself (PT_SYSTEM_PROMPT, PT_NO_THINK)
int64_t ref_chat_template(const char* architecture, const char* model_name, const char* prompt, char* out, int64_t cap) {
    GGUFModel m;
    m.config.architecture = architecture;
    m.config.model_name = model_name;
    const std::string s = m.apply_chat_template(prompt);
    memcpy(out, s.data(), (size_t)std::min<int64_t>(cap, (int64_t)s.size()));
    return (int64_t)s.size();
}
// ---------------------------------------------------------------------------------
// The reference's own loader: GGUFModel::load (torch/io/gguf_model.h:2038-2089: ModelConfig::parse :122-263, tokenizer,
// load_weights :6770-6886, load_quantized_mmap :1747-1975) on a .gguf file, then forward_decode_cpu on what it loaded.
// The handle is stepped with ref_model_decode and released with ref_model_free_loaded (the weights belong to the
// reference's mapping here, not to the caller).
// ---------------------------------------------------------------------------------
void* ref_model_load_gguf(const char* gguf_path, int64_t max_seq) {
    auto* r = new RefModel();
    try {
        r->m.load(gguf_path);
    } catch (...) {
        delete r;
        return nullptr;
    }
    r->m.use_cuda_ = false;
    r->m.kv_cache.allocate(r->m.config.num_layers, max_seq, r->m.config.num_kv_heads * r->m.config.head_dim, false);
    return r;
}
void ref_model_free_loaded(void* h) { delete static_cast<RefModel*>(h); }
// What the reference's parser made of the file's metadata and tensors.  ints[16]: vocab, hidden, layers, heads, kv heads,
// head_dim, intermediate, tie_word_embeddings, has_qk_norm, rope_neox, scale_embeddings, ffn_gelu, has_post_norm, swa_window,
// swa_pattern, use_quant_gemv_; floats[5]: rope_freq_base, rms_norm_eps, rope_scale, rope_swa_freq_base, rope_swa_scale;
// types[7 * layers + 1]: ggml type of q, k, v, o, gate, up, down per layer as load_quantized_mmap registered them, then of
// the output matrix (0xffffffff: not registered as a quantised weight)
void ref_model_describe(void* h, int64_t* ints, float* floats, uint32_t* types) {
    auto& m = static_cast<RefModel*>(h)->m;
    const auto& c = m.config;
    const int64_t iv[16] = {c.vocab_size, c.hidden_size, c.num_layers, c.num_heads, c.num_kv_heads, c.head_dim,
                            c.intermediate_size, c.tie_word_embeddings, c.has_qk_norm, c.rope_neox, c.scale_embeddings,
                            c.ffn_gelu, c.has_post_norm, c.swa_window, c.swa_pattern, m.use_quant_gemv_};
    std::memcpy(ints, iv, sizeof iv);
    const float fv[5] = {c.rope_freq_base, c.rms_norm_eps, c.rope_scale, c.rope_swa_freq_base, c.rope_swa_scale};
    std::memcpy(floats, fv, sizeof fv);
    size_t k = 0;
    for (auto& L : m.layers)
        for (auto* w : {&L.q_attn_q, &L.q_attn_k, &L.q_attn_v, &L.q_attn_output, &L.q_ffn_gate, &L.q_ffn_up, &L.q_ffn_down})
            types[k++] = w->valid ? w->quant_type : 0xffffffffu;
    types[k] = m.q_output_weight.valid ? m.q_output_weight.quant_type : 0xffffffffu;
}

// what the reference's reader sees of a file: tensor count, and name / type / dims / first bytes of tensor i
int64_t ref_gguf_n_tensors(const char* gguf_path) {
    g::GGUFReader reader;
    reader.open(gguf_path);
    return (int64_t)reader.tensors.size();
}

}  // extern "C"
