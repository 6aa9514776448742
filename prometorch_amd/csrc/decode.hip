// Batch-1 greedy decode runtime: the MI355X counterpart of GGUFModel::forward_decode
// (reference: torch/io/gguf_model.h:2575-3113) and of the greedy argmax that follows it
// (:4850-4859).  One HIP stream, scratch allocated once, the whole token step captured in a
// hipGraph; the position and the current token live in device memory, and the last kernel of a
// step feeds the argmax back as the next token, so consecutive tokens need no host round trip.
//
// Per layer (Q4_K_M mix: q/k/o/gate/up Q4_K, v/down Q6_K):
//   RMSNorm + {q,k (Q4_K), v (Q6_K)} in one mixed launch (the norm is recomputed per workgroup; quant
//   type is dispatched per tensor, as gemv_scratch does; other mixes fall back to one launch per type)
//   QK-norm + NeoX RoPE + K/V append + split-KV attention in one launch, then the split merge
//   o-proj GEMV accumulating into the residual
//   rmsnorm + gate + up + SiLU*up in one launch
//   down-proj GEMV accumulating into the residual
#include "ptm_common.h"

#include <cstring>
#include <new>
#include <utility>
#include <vector>

// flash_decode.hip: ptm_attn_decode_fused that also leaves the output as Q8 activation blocks (not part of the C ABI)
extern "C" int ptm_attn_decode_fused_bias(const float* Q, const float* K, const float* V, const float* q_bias,
                                          const float* k_bias, const float* v_bias, const float* q_norm_w,
                                          const float* k_norm_w, void* K_cache, void* V_cache, float* O, void* o_q8,
                                          float* partial_O, float* partial_lse, float* partial_max, const float* rope_table,
                                          int n_heads, int n_kv_heads, int head_dim, const int64_t* d_past_len, int max_seq,
                                          float scale, float eps, int add_one, int kv_fp16, int rope_interleaved, int window,
                                          ptm_stream_t stream);
extern "C" int ptm_attn_decode_folds_bias(int head_dim, int kv_fp16);
extern "C" int ptm_attn_decode_fused_q8(const float* Q, const float* K, const float* V, const float* q_norm_w,
                                        const float* k_norm_w, void* K_cache, void* V_cache, float* O, void* o_q8,
                                        float* partial_O, float* partial_lse, float* partial_max, const float* rope_table,
                                        int n_heads, int n_kv_heads, int head_dim, const int64_t* d_past_len, int max_seq,
                                        float scale, float eps, int add_one, int kv_fp16, int rope_interleaved,
                                        ptm_stream_t stream);

namespace ptm {
int q4k_gemv_multi(int n_mat, const void* const* W, float* const* y, const int* N, const void* x, bool x_is_q8,
                   const float* gamma, float eps, int add_one, int K, int64_t stride, bool accumulate, hipStream_t s);
int q4k_gate_up_silu(const void* wg, const void* wu, const void* x, bool x_is_q8, const float* gamma, float eps,
                     int add_one, float* act, int K, int N, int64_t stride, hipStream_t s, bool gelu);
int q6k_gemv_impl(const void* W, const float* x, float* y, int K, int N, int64_t stride, bool accumulate,
                  const float* gamma, float eps, int add_one, hipStream_t s);
void q6k_init_attributes();
int q6k_gemv_argmax_impl(const void* W, const float* x, const float* gamma, float eps, int add_one, float* xn_out,
                         float* logits, int K, int N, int64_t stride, int64_t* out_index, void* workspace,
                         const ArgmaxAdvance adv, hipStream_t s);
int qgemm_f16_impl(uint32_t ggml_type, const void* W, const void* X, bool x_is_f32, float* Y, int M, int K, int N,
                   int64_t stride, void* workspace, bool accumulate, float* split_ws, size_t split_ws_bytes, bool reuse_rows,
                   hipStream_t s, int* deferred_splits);
int qgemm_f16_reduce_norm_prepare(const float* P, int splits, float* X, bool accumulate, const float* gamma, float eps,
                                  int add_one, void* ws_round, void* ws_plain, int M, int K, hipStream_t s);
int qgemm_f16_splits(int N, int K, int M);
size_t qgemm_f16_multi_split_bytes(int n, const int* N, const uint32_t* types, int K, int M);
void qgemm_f16_multi_plan(int n, const int* N, const uint32_t* types, int K, int M, int* splits);
int qgemm_f16_multi(int n, const uint32_t* types, const void* const* W, const int64_t* strides, const int* N, float* const* Y,
                    int M, int K, void* ws_round, void* ws_plain, float* split_ws, size_t split_ws_bytes, hipStream_t s,
                    const float** deferred_P, int* deferred_splits);
int qknorm_rope_kv_rows_from_parts(const float* const* P, const int* splits, const float* const* bias, float* Q,
                                   const float* q_norm_w, const float* k_norm_w, void* K_cache, void* V_cache,
                                   const float* rope_table, int rows, int n_heads, int n_kv_heads, int head_dim, int64_t pos0,
                                   int max_seq, float eps, int add_one, int kv_fp16, int rope_interleaved, hipStream_t s);
int qgemm_f16_prepare_fused(int pre, const float* X, const float* X2, float eps, int add_one, void* ws_round, void* ws_plain,
                            int M, int K, hipStream_t s);
int sampler_launch_key(const ptm_sampling& host_params, int vocab);
int sampler_enqueue(const float* logits, int vocab, const int32_t* counts, const ptm_sampling& host_params,
                    const ptm_sampling* d_params, const float* d_uniforms, const int* d_step, void* workspace,
                    int64_t* out_token, int32_t* counts_rw, ArgmaxAdvance adv, bool ws_kept_clean, hipStream_t s);
__global__ void fill_i32_kernel(int32_t* p, int64_t n, int32_t v) {
    for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = v;
}
int rmsnorm_mixed_gemv(int n4, const void* const* W4, float* const* y4, const int* N4, int64_t stride4,
                       const void* W6, float* y6, int N6, int64_t stride6, const float* x, const float* gamma,
                       float eps, int add_one, int K, hipStream_t s, const float* pre_h, const float* pre_w, float* pre_out);

__global__ void set_scalars_kernel(int* d_token, int token, int64_t* d_past, int64_t past, int* d_step) {
    *d_token = token;
    *d_past = past;
    *d_step = 0;
}
// end of a step: publish the chosen token, feed it back, advance the position
__global__ void advance_kernel(const int64_t* d_next, int* d_token, int64_t* d_past, int* d_step,
                               int64_t* tokens_out, int cap) {
    const int64_t nx = *d_next;
    const int st = *d_step;
    if (st < cap) tokens_out[st] = nx;
    *d_token = (int)nx;
    *d_past = *d_past + 1;
    *d_step = st + 1;
}
}  // namespace ptm

using namespace ptm;

struct ptm_decoder {
    ptm_decode_config cfg{};
    std::vector<ptm_layer> layers;
    hipStream_t stream = nullptr;
    hipGraph_t graph = nullptr;       // one greedy step
    hipGraphExec_t exec = nullptr;
    bool captured = false;
    hipGraph_t graph_s = nullptr;     // one sampled step
    hipGraphExec_t exec_s = nullptr;
    bool captured_s = false;
    bool eager_fallback = false, eager_fallback_s = false;  // capture or instantiation failed once: plain launches from then on
    bool debug_fail_capture = false;  // test seam: the next capture attempt reports failure on the host, nothing is launched for it
    int sampled_key = -1;             // launch sequence (sampler_launch_key) the sampled-step graph was captured with
    // sampling state: parameters (host + device copy), occurrence counts of generated tokens, uniform draws
    ptm_sampling sampling{0.0f, 1, 1.0f, 1.0f};
    bool sampling_set = false;
    ptm_sampling* d_sampling = nullptr;
    int32_t* d_counts = nullptr;
    float* d_uniforms = nullptr;
    void* sampler_ws = nullptr;
    void* slab = nullptr;
    float *x = nullptr, *xn = nullptr, *q = nullptr, *k = nullptr, *v = nullptr, *attn = nullptr, *act = nullptr,
          *gate = nullptr, *up = nullptr, *logits = nullptr, *pO = nullptr, *pL = nullptr, *pM = nullptr,
          *rope = nullptr;
    float* hb = nullptr;        // [hidden] a branch's output in front of its post-norm
    float* x2 = nullptr;        // [hidden] second residual buffer: a kernel that applies a deferred post-norm reads one, writes the other
    float* rope_swa = nullptr;  // rotation table of the sliding-window layers (their own base, no position scaling)
    uint8_t* xq8 = nullptr;
    void* amax_ws = nullptr;
    int* d_token = nullptr;
    int* d_step = nullptr;
    int64_t* d_past = nullptr;
    int64_t* d_next = nullptr;
    int64_t* d_tokens = nullptr;  // the device's view of h_pinned: the step's last kernel stores the token id straight to the host
    // Greedy steps resume where the device stands: when the caller feeds back the token the last greedy run produced (what a
    // generate loop does), the device already holds it, the position and the step index, and no scalar-setting launch
    // is needed.  out_base = index in h_pinned of the last run's first token.
    bool dev_synced = false;
    int64_t dev_token = -1;
    int chain_base = 0, out_base = 0;
    bool untuned_types = false;   // some matrix is Q5_K / Q8_0 / Q5_0: no row-batched GEMM for it, prompts go token by token
    int64_t* h_pinned = nullptr;  // [max_seq] pinned host memory the token ids are written to by the device
    float* h_uniforms = nullptr;  // [max_seq] pinned host staging for the sampler's draws (an "async" copy from the
                                  // caller's pageable memory would be staged by the runtime synchronously)
    int64_t past_len = 0;
    int status = PTM_OK;
    // prefill scratch for up to pf_rows prompt rows at a time (allocated on the first prefill)
    void* pf_slab = nullptr;
    int pf_rows = 0;
    float *pf_x = nullptr, *pf_q = nullptr, *pf_k = nullptr, *pf_v = nullptr, *pf_attn = nullptr,
          *pf_gate = nullptr, *pf_up = nullptr, *pf_h = nullptr;
    void* pf_ws = nullptr;   // fp16 rows for Q4_K matrices (Q8-rounded)
    void* pf_ws2 = nullptr;  // fp16 rows for Q6_K matrices (plain)
    float* pf_split = nullptr;  // K-split partial sums of the GEMMs
    size_t pf_split_bytes = 0;
    int* pf_tokens = nullptr;
};

static bool tuned_type(uint32_t t) { return t == PTM_TYPE_Q4_K || t == PTM_TYPE_Q6_K; }

// Every type of the GEMV dispatcher is accepted.  Q4_K and Q6_K take the fused kernels of the decode path; Q5_K, Q8_0 and
// Q5_0 matrices go through a separate RMSNorm and the dispatcher's plain kernels, and a model that holds any of them
// is prefilled token by token (as the reference prefills every model: matmul_q is a loop of GEMVs, gguf_model.h:7029-7036).
static int qw_check(const ptm_qweight& w, int rows, int cols) {
    if (!w.data) return PTM_E_NULL;
    if (w.rows != rows || w.cols != cols) return PTM_E_SHAPE;
    if (!ptm_quant_gemv_supported(w.ggml_type)) return PTM_E_UNSUPPORTED;
    // the row stride is the descriptor's own (rows may be padded); it must hold a row and keep the rows aligned
    if (w.ggml_type == PTM_TYPE_Q4_K && (w.row_stride_bytes < (int64_t)(cols / 256) * 144 || (w.row_stride_bytes & 15))) return PTM_E_SHAPE;
    if (w.ggml_type == PTM_TYPE_Q6_K && (w.row_stride_bytes < (int64_t)(cols / 256) * 210 || (w.row_stride_bytes & 1))) return PTM_E_SHAPE;
    return PTM_OK;
}

static int gemv_any(const ptm_qweight& w, const float* x_f32, float* y, bool acc, hipStream_t s) {
    if (w.ggml_type == PTM_TYPE_Q4_K) {
        const void* W = w.data;
        const int N = w.rows;
        return q4k_gemv_multi(1, &W, &y, &N, x_f32, false, nullptr, 0.f, 0, w.cols, w.row_stride_bytes, acc, s);
    }
    if (w.ggml_type == PTM_TYPE_Q6_K)
        return q6k_gemv_impl(w.data, x_f32, y, w.cols, w.rows, w.row_stride_bytes, acc, nullptr, 0.f, 0, s);
    return ptm_quant_gemv(w.ggml_type, w.data, x_f32, y, w.cols, w.rows, w.row_stride_bytes, acc ? 1 : 0, s);
}

// gemma3's alternating layers: li is local (sliding window, own rotation base) unless (li + 1) % swa_pattern == 0
// (ModelConfig::layer_is_global, gguf_model.h:265-281)
static inline bool layer_is_local(const ptm_decode_config& c, int li) {
    return c.swa_window > 0 && c.swa_pattern > 0 && ((li + 1) % c.swa_pattern) != 0;
}

// Enqueue one token step on d->stream. Everything it reads that changes per token is in device memory.
// trace (optional, device [n_layers][2][hidden]): the residual stream after each layer's attention branch and after its
// feed-forward branch, copied out between the launches (never part of a captured graph)
static int enqueue_step(ptm_decoder* d, bool sample = false, float* trace = nullptr) {
    const ptm_decode_config& c = d->cfg;
    hipStream_t s = d->stream;
    const int H = c.hidden, hd = c.head_dim;
    int rc;
#define PTM_TRY(call) do { rc = (call); if (rc != PTM_OK) return rc; } while (0)
    if (c.embedding_f32) PTM_TRY(ptm_embedding_row(c.embedding_f32, d->x, d->d_token, H, s));
    else PTM_TRY(ptm_embedding_row_q6k(c.lm_head.data, d->x, d->d_token, H, c.lm_head.row_stride_bytes, s));
    if (c.scale_embeddings) PTM_TRY(ptm_scale(d->x, sqrtf((float)H), H, s));

    // The residual stream is in xc.  The post-norm of a feed-forward branch (gemma: x += RMSNorm(h) * w) is not a launch of its
    // own where the next layer's q / k / v launch can apply it in its prologue (the mixed Q4_K / Q6_K launch; vectors of up to
    // 4096 values): that launch reads xc, h and w, and its first workgroup writes the updated residual to the other buffer,
    // xo.  pend_h / pend_w: the post-norm waiting for the next layer.  A traced step applies every post-norm at once.
    // (The same in front of the fused gate / up launch for the post-norm of the attention branch gains nothing: the two extra
    // vectors in the prologue of its 1280 workgroups cost what the launch saves.)
    float *xc = d->x, *xo = d->x2;
    const float *pend_h = nullptr, *pend_w = nullptr;
    auto qkv_is_mixed = [&](const ptm_layer& L) {
        if (!tuned_type(L.q.ggml_type) || !tuned_type(L.k.ggml_type) || !tuned_type(L.v.ggml_type)) return false;
        const int n6 = (L.q.ggml_type != PTM_TYPE_Q4_K) + (L.k.ggml_type != PTM_TYPE_Q4_K) + (L.v.ggml_type != PTM_TYPE_Q4_K);
        return n6 == 1 && H <= 16384;
    };
    auto gate_up_is_fused = [&](const ptm_layer& L) {
        return L.gate.ggml_type == PTM_TYPE_Q4_K && L.up.ggml_type == PTM_TYPE_Q4_K &&
               L.gate.row_stride_bytes == L.up.row_stride_bytes && L.gate.rows == L.up.rows;
    };
    const bool may_defer = !trace && H <= 4096;
    for (int li = 0; li < c.n_layers; ++li) {
        const ptm_layer& L = d->layers[li];
        const bool local = layer_is_local(c, li);  // sliding-window layer: own rotation table, attention window
        // attention RMSNorm is recomputed inside each projection kernel (no separate launch):
        // the Q4_K projections share one launch, Q6_K ones get their own
        {
            const ptm_qweight* w[3] = {&L.q, &L.k, &L.v};
            float* y[3] = {d->q, d->k, d->v};
            const void* W4[3]; float* y4[3]; int N4[3]; int n4 = 0;
            int i6 = -1, n6 = 0;
            for (int i = 0; i < 3; ++i) {
                if (w[i]->ggml_type == PTM_TYPE_Q4_K) { W4[n4] = w[i]->data; y4[n4] = y[i]; N4[n4] = w[i]->rows; ++n4; }
                else { i6 = i; ++n6; }
            }
            int64_t s4 = 0;  // the Q4_K projections of one launch share a row stride (checked at create)
            for (int i = 0; i < 3; ++i) if (w[i]->ggml_type == PTM_TYPE_Q4_K) { s4 = w[i]->row_stride_bytes; break; }
            if (!tuned_type(L.q.ggml_type) || !tuned_type(L.k.ggml_type) || !tuned_type(L.v.ggml_type)) {
                PTM_TRY(ptm_rms_norm(xc, L.attn_norm, d->xn, 1, H, c.rms_eps, 0, nullptr, s));
                for (int i = 0; i < 3; ++i) PTM_TRY(gemv_any(*w[i], d->xn, y[i], false, s));
            } else if (n6 == 1 && n4 >= 1 && H <= 16384) {
                // the Q4_K_M mix (q, k in Q4_K; v in Q6_K): all three projections in one launch
                PTM_TRY(rmsnorm_mixed_gemv(n4, W4, y4, N4, s4, w[i6]->data, y[i6], w[i6]->rows, w[i6]->row_stride_bytes,
                                           xc, L.attn_norm, c.rms_eps, 0, H, s, pend_h, pend_w, pend_h ? xo : nullptr));
                if (pend_h) {
                    std::swap(xc, xo);
                    pend_h = pend_w = nullptr;
                }
            } else {
                for (int i = 0; i < 3; ++i)
                    if (w[i]->ggml_type != PTM_TYPE_Q4_K)
                        PTM_TRY(q6k_gemv_impl(w[i]->data, xc, y[i], H, w[i]->rows, w[i]->row_stride_bytes, false,
                                              L.attn_norm, c.rms_eps, 0, s));
                if (n4 > 0) PTM_TRY(q4k_gemv_multi(n4, W4, y4, N4, xc, false, L.attn_norm, c.rms_eps, 0, H, s4, false, s));
            }
        }
        // projection biases (qwen2): added by the attention launch where it can, else by a launch of their own
        const bool fold_bias = L.q_bias && ptm_attn_decode_folds_bias(hd, c.kv_fp16);
        if (L.q_bias && !fold_bias)
            PTM_TRY(ptm_add_qkv_bias(d->q, d->k, d->v, L.q_bias, L.k_bias, L.v_bias, 1, c.n_heads * hd, c.n_kv_heads * hd, s));
        // QK-norm + RoPE + K/V append + split-KV attention in one launch, plus the small merge launch
        // a Q4_K output projection takes the attention output as the Q8 blocks the merge kernel leaves beside the fp32
        // vector: its prologue then copies 1.25 bytes per value instead of fetching and quantising 4
        const bool o_q8 = L.o.ggml_type == PTM_TYPE_Q4_K;
        PTM_TRY(ptm_attn_decode_fused_bias(d->q, d->k, d->v, fold_bias ? L.q_bias : nullptr, fold_bias ? L.k_bias : nullptr,
                                           fold_bias ? L.v_bias : nullptr, L.q_norm, L.k_norm, L.k_cache, L.v_cache, d->attn,
                                           o_q8 ? d->xq8 : nullptr, d->pO, d->pL, d->pM, local ? d->rope_swa : d->rope,
                                           c.n_heads, c.n_kv_heads, hd, d->d_past, c.max_seq, 1.0f / sqrtf((float)hd),
                                           c.rms_eps, 0, c.kv_fp16, c.rope_interleaved, local ? c.swa_window : 0, s));
        // x += Wo . attn, or with a post-norm: h = Wo . attn, x += RMSNorm(h) * w
        float* o_dst = L.post_attn_norm ? d->hb : xc;
        const bool o_acc = !L.post_attn_norm;
        if (o_q8) {
            const void* W = L.o.data;
            const int N = L.o.rows;
            PTM_TRY(q4k_gemv_multi(1, &W, &o_dst, &N, d->xq8, true, nullptr, 0.f, 0, L.o.cols, L.o.row_stride_bytes, o_acc, s));
        } else {
            PTM_TRY(gemv_any(L.o, d->attn, o_dst, o_acc, s));
        }
        if (L.post_attn_norm) PTM_TRY(ptm_rms_norm_add(d->hb, L.post_attn_norm, xc, 1, H, c.rms_eps, 0, s));
        if (trace) PTM_TRY(ptm_copy(xc, trace + (size_t)(2 * li) * H, H, s));
        if (gate_up_is_fused(L)) {
            PTM_TRY(q4k_gate_up_silu(L.gate.data, L.up.data, xc, false, L.ffn_norm, c.rms_eps, 0, d->act, H,
                                     L.gate.rows, L.gate.row_stride_bytes, s, c.ffn_gelu != 0));
        } else {
            PTM_TRY(ptm_rms_norm(xc, L.ffn_norm, d->xn, 1, H, c.rms_eps, 0, nullptr, s));
            PTM_TRY(gemv_any(L.gate, d->xn, d->gate, false, s));
            PTM_TRY(gemv_any(L.up, d->xn, d->up, false, s));
            if (c.ffn_gelu) PTM_TRY(ptm_gelu_mul(d->gate, d->up, d->act, c.inter, s));
            else PTM_TRY(ptm_silu_mul(d->gate, d->up, d->act, c.inter, s));
        }
        if (L.post_ffn_norm) {
            PTM_TRY(gemv_any(L.down, d->act, d->hb, false, s));
            if (may_defer && li + 1 < c.n_layers && qkv_is_mixed(d->layers[li + 1])) {
                pend_h = d->hb;  // applied by the next layer's q / k / v launch
                pend_w = L.post_ffn_norm;
            } else {
                PTM_TRY(ptm_rms_norm_add(d->hb, L.post_ffn_norm, xc, 1, H, c.rms_eps, 0, s));
            }
        } else {
            PTM_TRY(gemv_any(L.down, d->act, xc, true, s));  // x += Wdown . act
        }
        if (trace) PTM_TRY(ptm_copy(xc, trace + (size_t)(2 * li + 1) * H, H, s));
    }
    if (sample) {
        // logits (final RMSNorm in the lm_head prologue), then the sampler, whose last kernel does the step bookkeeping
        if (c.lm_head.ggml_type == PTM_TYPE_Q6_K) {
            PTM_TRY(q6k_gemv_impl(c.lm_head.data, xc, d->logits, H, c.vocab, c.lm_head.row_stride_bytes, false, c.out_norm,
                                  c.rms_eps, 0, s));
        } else {
            PTM_TRY(ptm_rms_norm(xc, c.out_norm, d->xn, 1, H, c.rms_eps, 0, nullptr, s));
            PTM_TRY(gemv_any(c.lm_head, d->xn, d->logits, false, s));
        }
        return sampler_enqueue(d->logits, c.vocab, d->d_counts, d->sampling, d->d_sampling, d->d_uniforms, d->d_step,
                               d->sampler_ws, d->d_next, d->d_counts,
                               ArgmaxAdvance{d->d_token, d->d_past, d->d_step, d->d_tokens, c.max_seq}, true, s);
    }
    if (c.lm_head.ggml_type == PTM_TYPE_Q6_K) {
        // final RMSNorm in the lm_head prologue, step bookkeeping in the argmax tail: two launches for the whole tail
        return q6k_gemv_argmax_impl(c.lm_head.data, xc, c.out_norm, c.rms_eps, 0, d->xn, d->logits, H, c.vocab,
                                    c.lm_head.row_stride_bytes, d->d_next, d->amax_ws,
                                    ArgmaxAdvance{d->d_token, d->d_past, d->d_step, d->d_tokens, c.max_seq}, s);
    }
    PTM_TRY(ptm_rms_norm(xc, c.out_norm, d->xn, 1, H, c.rms_eps, 0, nullptr, s));
    PTM_TRY(gemv_any(c.lm_head, d->xn, d->logits, false, s));
    PTM_TRY(ptm_argmax(d->logits, d->d_next, c.vocab, s));
    hipLaunchKernelGGL(advance_kernel, dim3(1), dim3(1), 0, s, d->d_next, d->d_token, d->d_past, d->d_step,
                       d->d_tokens, c.max_seq);
    return launch_status();
#undef PTM_TRY
}

// ---- prefill: M prompt rows through the layers at once (reference: GGUFModel::forward with use_cache,
// torch/io/gguf_model.h:2510-2571 and transformer_layer :7300-7460) -------------------------------------------
static int prefill_alloc(ptm_decoder* d, int rows) {
    if (d->pf_rows >= rows) return PTM_OK;
    if (d->pf_slab) { (void)hipFree(d->pf_slab); d->pf_slab = nullptr; d->pf_rows = 0; }
    const ptm_decode_config& c = d->cfg;
    const size_t H = c.hidden, qd = (size_t)c.n_heads * c.head_dim, kvd = (size_t)c.n_kv_heads * c.head_dim, I = c.inter;
    const size_t kmax = H > I ? (H > qd ? H : qd) : (I > qd ? I : qd);
    auto up = [](size_t b) { return (b + 255) & ~(size_t)255; };
    size_t off = 0;
    auto take = [&](size_t bytes) { const size_t o = off; off += up(bytes); return o; };
    const size_t R = (size_t)rows;
    const size_t o_h = take(4 * R * H);
    const size_t o_x = take(4 * R * H), o_q = take(4 * R * qd), o_k = take(4 * R * kvd),
                 o_v = take(4 * R * kvd), o_attn = take(4 * R * qd), o_gate = take(4 * R * I), o_up = take(4 * R * I),
                 o_ws = take((size_t)ptm_qgemm_f16_workspace_bytes(rows, (int)kmax)),
                 o_ws2 = take((size_t)ptm_qgemm_f16_workspace_bytes(rows, (int)kmax)), o_tok = take(4 * R);
    size_t split_elems = 0;  // widest splits x N over the layer's matrices (all layers have the same shapes)
    for (const ptm_qweight* w : {&d->layers[0].q, &d->layers[0].k, &d->layers[0].v, &d->layers[0].o, &d->layers[0].gate,
                                 &d->layers[0].up, &d->layers[0].down}) {
        for (const int m : {128, 256, 1024, rows}) {  // the split count depends on the row class: size for the widest use
            const int mm = m < rows ? m : rows;
            const size_t e = (size_t)qgemm_f16_splits(w->rows, w->cols, mm) * w->rows * (size_t)mm;
            split_elems = e > split_elems ? e : split_elems;
        }
    }
    d->pf_split_bytes = 4 * split_elems;
    for (int li = 0; li < c.n_layers; ++li) {  // q, k, v share one launch whose splits depend on the types, which vary by layer
        const ptm_layer& L = d->layers[li];
        const int N3[3] = {L.q.rows, L.k.rows, L.v.rows};
        const uint32_t t3[3] = {L.q.ggml_type, L.k.ggml_type, L.v.ggml_type};
        const int N2[2] = {L.gate.rows, L.up.rows};  // so may gate and up
        const uint32_t t2[2] = {L.gate.ggml_type, L.up.ggml_type};
        for (const int m : {128, 256, 1024, rows}) {
            const size_t b = qgemm_f16_multi_split_bytes(3, N3, t3, (int)H, m < rows ? m : rows);
            d->pf_split_bytes = b > d->pf_split_bytes ? b : d->pf_split_bytes;
            const size_t b2 = qgemm_f16_multi_split_bytes(2, N2, t2, (int)H, m < rows ? m : rows);
            d->pf_split_bytes = b2 > d->pf_split_bytes ? b2 : d->pf_split_bytes;
        }
    }
    const size_t o_split = take(d->pf_split_bytes);
    const int rc = hip_status(hipMalloc(&d->pf_slab, off));
    if (rc != PTM_OK) return rc;
    uint8_t* b = static_cast<uint8_t*>(d->pf_slab);
    d->pf_h = (float*)(b + o_h);
    d->pf_x = (float*)(b + o_x); d->pf_q = (float*)(b + o_q); d->pf_k = (float*)(b + o_k);
    d->pf_v = (float*)(b + o_v); d->pf_attn = (float*)(b + o_attn); d->pf_gate = (float*)(b + o_gate);
    d->pf_up = (float*)(b + o_up); d->pf_ws = b + o_ws; d->pf_ws2 = b + o_ws2; d->pf_tokens = (int*)(b + o_tok);
    d->pf_split = (float*)(b + o_split);
    d->pf_rows = rows;
    return PTM_OK;
}

// rows [0, M) of one chunk at positions pos0 .. pos0 + M - 1; leaves the residual rows in pf_x
static int prefill_chunk(ptm_decoder* d, const int* tokens_host, int M, int64_t pos0) {
    const ptm_decode_config& c = d->cfg;
    hipStream_t s = d->stream;
    const int H = c.hidden, hd = c.head_dim, qd = c.n_heads * hd, kvd = c.n_kv_heads * hd, I = c.inter;
    int rc;
#define PTM_TRY(call) do { rc = (call); if (rc != PTM_OK) return rc; } while (0)
    PTM_TRY(hip_status(hipMemcpyAsync(d->pf_tokens, tokens_host, 4 * (size_t)M, hipMemcpyHostToDevice, s)));
    PTM_TRY(ptm_embedding_rows(c.embedding_f32, c.embedding_f32 ? nullptr : c.lm_head.data, c.lm_head.row_stride_bytes,
                               d->pf_tokens, M, H, c.vocab, d->pf_x, s));
    if (c.scale_embeddings) PTM_TRY(ptm_scale(d->pf_x, sqrtf((float)H), (int64_t)M * H, s));
    // Q4_K matrices take their rows from pf_ws (Q8-rounded fp16), Q6_K ones from pf_ws2 (plain fp16).  RMSNorm and
    // SiLU.up are fused into the conversion (one launch fills both forms); a product whose rows are already in its
    // workspace skips the conversion.
    auto ws_of = [&](const ptm_qweight& w) { return w.ggml_type == PTM_TYPE_Q4_K ? d->pf_ws : d->pf_ws2; };
    auto gemm = [&](const ptm_qweight& w, const float* X, float* Y, bool acc, bool rows_ready, int* deferred = nullptr) {
        return qgemm_f16_impl(w.ggml_type, w.data, X, true, Y, M, w.cols, w.rows, w.row_stride_bytes, ws_of(w), acc,
                              d->pf_split, d->pf_split_bytes, rows_ready, s, deferred);
    };
    // RMSNorm of the residual rows into the row workspaces; `pending` > 0: the projection before it left that many K-split
    // partial sums in pf_split, which the same launch first adds to the residual rows
    auto norm_rows = [&](int pending, const float* gamma, bool need4, bool need6) {
        void* w4 = need4 ? d->pf_ws : nullptr;
        void* w6 = need6 ? d->pf_ws2 : nullptr;
        if (pending > 0)
            return qgemm_f16_reduce_norm_prepare(d->pf_split, pending, d->pf_x, true, gamma, c.rms_eps, 0, w4, w6, M, H, s);
        return qgemm_f16_prepare_fused(1, d->pf_x, gamma, c.rms_eps, 0, w4, w6, M, H, s);
    };
    int pending = 0;  // K-split partial sums of the last projection into pf_x that are still to be added
    auto uses = [](uint32_t type, std::initializer_list<const ptm_qweight*> ws) {
        for (const ptm_qweight* w : ws) if (w->ggml_type == type) return true;
        return false;
    };
    for (int li = 0; li < c.n_layers; ++li) {
        const ptm_layer& L = d->layers[li];
        const bool local = layer_is_local(c, li);
        PTM_TRY(norm_rows(pending, L.attn_norm, uses(PTM_TYPE_Q4_K, {&L.q, &L.k, &L.v}), uses(PTM_TYPE_Q6_K, {&L.q, &L.k, &L.v})));
        pending = 0;
        {  // q, k, v in one launch
            const uint32_t t3[3] = {L.q.ggml_type, L.k.ggml_type, L.v.ggml_type};
            const void* W3[3] = {L.q.data, L.k.data, L.v.data};
            const int64_t s3[3] = {L.q.row_stride_bytes, L.k.row_stride_bytes, L.v.row_stride_bytes};
            const int N3[3] = {L.q.rows, L.k.rows, L.v.rows};
            float* Y3[3] = {d->pf_q, d->pf_k, d->pf_v};
            // the sum of the K splits (and the biases) is left to the next launch, which reads q, k, v once anyway
            const float* P3[3];
            int sp3[3];
            PTM_TRY(qgemm_f16_multi(3, t3, W3, s3, N3, Y3, M, H, d->pf_ws, d->pf_ws2, d->pf_split, d->pf_split_bytes, s, P3, sp3));
            const float* b3[3] = {L.q_bias, L.k_bias, L.v_bias};
            PTM_TRY(qknorm_rope_kv_rows_from_parts(P3, sp3, L.q_bias ? b3 : nullptr, d->pf_q, L.q_norm, L.k_norm, L.k_cache,
                                                   L.v_cache, local ? d->rope_swa : d->rope, M, c.n_heads, c.n_kv_heads, hd,
                                                   pos0, c.max_seq, c.rms_eps, 0, c.kv_fp16, c.rope_interleaved, s));
        }
        PTM_TRY(ptm_prefill_attention_window(d->pf_q, L.k_cache, L.v_cache, d->pf_attn, M, c.n_heads, c.n_kv_heads, hd, pos0,
                                             c.max_seq, 1.0f / sqrtf((float)hd), c.kv_fp16, local ? c.swa_window : 0, s));
        if (L.post_attn_norm) {
            PTM_TRY(gemm(L.o, d->pf_attn, d->pf_h, false, false));
            PTM_TRY(ptm_rms_norm_add(d->pf_h, L.post_attn_norm, d->pf_x, M, H, c.rms_eps, 0, s));
        } else {
            PTM_TRY(gemm(L.o, d->pf_attn, d->pf_x, true, false, H <= 12288 ? &pending : nullptr));  // x += attn . Wo^T
        }
        PTM_TRY(norm_rows(pending, L.ffn_norm, uses(PTM_TYPE_Q4_K, {&L.gate, &L.up}), uses(PTM_TYPE_Q6_K, {&L.gate, &L.up})));
        pending = 0;
        {
            // Gate and up share one launch when that fills the chip better.  The eight-wave tile runs one workgroup per CU, so
            // a launch costs ceil(tiles / 256) workgroup times: 2048 rows are 38 x 16 = 608 tiles per matrix, 3 + 3 rounds
            // apart and 5 together; 512 rows, 152 tiles each, gain nothing (1 + 1 against 2).  Up to 256 rows (the two
            // short row classes) always together: one launch less, and the launch is the cost there.  Beyond, only when both
            // ways use the same K splits, so that the choice changes no result.
            const uint32_t t2[2] = {L.gate.ggml_type, L.up.ggml_type};
            const int N2[2] = {L.gate.rows, L.up.rows};
            bool together = M <= 256;
            if (!together) {
                int sp2[2];
                qgemm_f16_multi_plan(2, N2, t2, (int)H, M, sp2);
                const int row_tiles = (M + 127) / 128;
                const int tg = (N2[0] + 255) / 256 * row_tiles * sp2[0], tu = (N2[1] + 255) / 256 * row_tiles * sp2[1];
                together = sp2[0] == qgemm_f16_splits(N2[0], (int)H, M) && sp2[1] == qgemm_f16_splits(N2[1], (int)H, M) &&
                           (tg + tu + 255) / 256 < (tg + 255) / 256 + (tu + 255) / 256;
            }
            if (together) {
                const void* W2[2] = {L.gate.data, L.up.data};
                const int64_t s2[2] = {L.gate.row_stride_bytes, L.up.row_stride_bytes};
                float* Y2[2] = {d->pf_gate, d->pf_up};
                PTM_TRY(qgemm_f16_multi(2, t2, W2, s2, N2, Y2, M, H, d->pf_ws, d->pf_ws2, d->pf_split, d->pf_split_bytes, s, nullptr, nullptr));
            } else {
                PTM_TRY(gemm(L.gate, d->pf_x, d->pf_gate, false, true));
                PTM_TRY(gemm(L.up, d->pf_x, d->pf_up, false, true));
            }
        }
        const bool act_ready = true;
        // SiLU.up (or, flagged through the add_one slot, GELU.up) fused into the conversion for the down projection
        PTM_TRY(qgemm_f16_prepare_fused(2, d->pf_gate, d->pf_up, 0.0f, c.ffn_gelu ? 1 : 0,
                                        L.down.ggml_type == PTM_TYPE_Q4_K ? d->pf_ws : nullptr,
                                        L.down.ggml_type == PTM_TYPE_Q6_K ? d->pf_ws2 : nullptr, M, I, s));
        if (L.post_ffn_norm) {
            PTM_TRY(gemm(L.down, d->pf_gate, d->pf_h, false, act_ready));
            PTM_TRY(ptm_rms_norm_add(d->pf_h, L.post_ffn_norm, d->pf_x, M, H, c.rms_eps, 0, s));
        } else {
            // x += act . Wdown^T; before another layer the sum of the K splits is left to that layer's first launch
            PTM_TRY(gemm(L.down, d->pf_gate, d->pf_x, true, act_ready, (li + 1 < c.n_layers && H <= 12288) ? &pending : nullptr));
        }
    }
    (void)qd; (void)kvd;
    return PTM_OK;
#undef PTM_TRY
}

extern "C" {

int ptm_decode_create(const ptm_decode_config* cfg, ptm_decoder** out) {
    if (!cfg || !out || !cfg->layers || !cfg->out_norm) return PTM_E_NULL;
    *out = nullptr;
    const ptm_decode_config& c = *cfg;
    if (c.vocab <= 0 || c.hidden <= 0 || c.n_layers <= 0 || c.n_heads <= 0 || c.n_kv_heads <= 0 || c.inter <= 0 ||
        c.max_seq <= 0 || (c.hidden % 256) || (c.inter % 256) || ((c.n_heads * c.head_dim) % 256) ||
        (c.n_heads % c.n_kv_heads))
        return PTM_E_SHAPE;
    if (c.head_dim != 64 && c.head_dim != 128 && c.head_dim != 256) return PTM_E_UNSUPPORTED;
    if (c.swa_window < 0 || c.swa_pattern < 0 || (c.swa_window > 0 && !(c.rope_swa_freq_base > 0.0f))) return PTM_E_SHAPE;
    const int H = c.hidden, qd = c.n_heads * c.head_dim, kvd = c.n_kv_heads * c.head_dim;
    int rc = qw_check(c.lm_head, c.vocab, H);
    if (rc != PTM_OK) return rc;
    if (!c.embedding_f32 && c.lm_head.ggml_type != PTM_TYPE_Q6_K) return PTM_E_UNSUPPORTED;
    for (int i = 0; i < c.n_layers; ++i) {
        const ptm_layer& L = c.layers[i];
        if (!L.attn_norm || !L.ffn_norm || !L.k_cache || !L.v_cache) return PTM_E_NULL;
        if ((L.q_norm == nullptr) != (L.k_norm == nullptr)) return PTM_E_NULL;  // QK-norm: both or neither
        if ((L.q_bias == nullptr) != (L.k_bias == nullptr) || (L.q_bias == nullptr) != (L.v_bias == nullptr)) return PTM_E_NULL;
        if ((rc = qw_check(L.q, qd, H)) || (rc = qw_check(L.k, kvd, H)) || (rc = qw_check(L.v, kvd, H)) ||
            (rc = qw_check(L.o, H, qd)) || (rc = qw_check(L.gate, c.inter, H)) || (rc = qw_check(L.up, c.inter, H)) ||
            (rc = qw_check(L.down, H, c.inter)))
            return rc;
        // q / k / v in Q4_K go through one launch with one row stride
        int64_t s4 = -1;
        for (const ptm_qweight* w : {&L.q, &L.k, &L.v}) {
            if (w->ggml_type != PTM_TYPE_Q4_K) continue;
            if (s4 >= 0 && w->row_stride_bytes != s4) return PTM_E_SHAPE;
            s4 = w->row_stride_bytes;
        }
    }
    ptm_decoder* d = new (std::nothrow) ptm_decoder();
    if (!d) return PTM_E_STATE;
    d->cfg = c;
    d->layers.assign(c.layers, c.layers + c.n_layers);
    d->cfg.layers = d->layers.data();
    d->cfg.rope_factors_short = d->cfg.rope_factors_long = nullptr;  // host arrays of the caller: read below, not kept
    for (const ptm_layer& L : d->layers)
        for (const ptm_qweight* w : {&L.q, &L.k, &L.v, &L.o, &L.gate, &L.up, &L.down})
            if (!tuned_type(w->ggml_type)) d->untuned_types = true;

    const int S = ptm_flash_decode_num_splits(c.max_seq);
    auto up16 = [](size_t b) { return (b + 255) & ~(size_t)255; };
    size_t off = 0;
    auto take = [&](size_t bytes) { const size_t o = off; off += up16(bytes); return o; };
    const size_t o_x = take(4 * (size_t)H), o_xn = take(4 * (size_t)H), o_q = take(4 * (size_t)qd),
                 o_k = take(4 * (size_t)kvd), o_v = take(4 * (size_t)kvd), o_attn = take(4 * (size_t)qd),
                 o_act = take(4 * (size_t)c.inter), o_gate = take(4 * (size_t)c.inter),
                 o_up = take(4 * (size_t)c.inter), o_logits = take(4 * (size_t)c.vocab),
                 o_pO = take(4 * (size_t)S * c.n_heads * c.head_dim), o_pL = take(4 * (size_t)S * c.n_heads),
                 o_pM = take(4 * (size_t)S * c.n_heads), o_rope = take(4 * (size_t)c.max_seq * c.head_dim),
                 o_hb = take(4 * (size_t)H), o_x2 = take(4 * (size_t)H), o_rope_swa = take(c.swa_window > 0 ? 4 * (size_t)c.max_seq * c.head_dim : 0),
                 o_xq8 = take((size_t)ptm_q8_bytes(qd > (H > c.inter ? H : c.inter) ? qd : (H > c.inter ? H : c.inter))),
                 o_ws = take((size_t)ptm_argmax_workspace_bytes(c.vocab)), o_tok = take(256), o_past = take(256),
                 o_next = take(256), o_step = take(256),
                 o_samp = take(256), o_counts = take(4 * (size_t)c.vocab), o_unif = take(4 * (size_t)c.max_seq),
                 o_sws = take((size_t)ptm_sampler_workspace_bytes());
    if ((rc = hip_status(hipMalloc(&d->slab, off))) != PTM_OK) { delete d; return rc; }
    uint8_t* base = static_cast<uint8_t*>(d->slab);
    d->x = (float*)(base + o_x); d->xn = (float*)(base + o_xn); d->q = (float*)(base + o_q);
    d->k = (float*)(base + o_k); d->v = (float*)(base + o_v); d->attn = (float*)(base + o_attn);
    d->act = (float*)(base + o_act); d->gate = (float*)(base + o_gate); d->up = (float*)(base + o_up);
    d->logits = (float*)(base + o_logits); d->pO = (float*)(base + o_pO); d->pL = (float*)(base + o_pL);
    d->pM = (float*)(base + o_pM); d->rope = (float*)(base + o_rope); d->xq8 = base + o_xq8;
    d->hb = (float*)(base + o_hb); d->x2 = (float*)(base + o_x2); d->rope_swa = c.swa_window > 0 ? (float*)(base + o_rope_swa) : d->rope;
    d->amax_ws = base + o_ws; d->d_token = (int*)(base + o_tok); d->d_past = (int64_t*)(base + o_past);
    d->d_next = (int64_t*)(base + o_next); d->d_step = (int*)(base + o_step);
    d->d_sampling = (ptm_sampling*)(base + o_samp); d->d_counts = (int32_t*)(base + o_counts);
    d->d_uniforms = (float*)(base + o_unif); d->sampler_ws = base + o_sws;
    if ((rc = hip_status(hipMemset(d->sampler_ws, 0, (size_t)ptm_sampler_workspace_bytes()))) != PTM_OK) { ptm_decode_destroy(d); return rc; }
    q6k_init_attributes();  // one-time kernel attributes, before anything can be captured

    if ((rc = hip_status(hipStreamCreateWithFlags(&d->stream, hipStreamNonBlocking))) != PTM_OK) { ptm_decode_destroy(d); return rc; }
    if ((rc = hip_status(hipHostMalloc((void**)&d->h_pinned, 8 * (size_t)c.max_seq, hipHostMallocDefault))) != PTM_OK) { ptm_decode_destroy(d); return rc; }
    // token ids go from the step's last kernel straight to pinned host memory (an 8-byte store per token): no copy launch
    // between the step and the host's read
    if ((rc = hip_status(hipHostGetDevicePointer((void**)&d->d_tokens, d->h_pinned, 0))) != PTM_OK) { ptm_decode_destroy(d); return rc; }
    if ((rc = hip_status(hipHostMalloc((void**)&d->h_uniforms, 4 * (size_t)c.max_seq, hipHostMallocDefault))) != PTM_OK) { ptm_decode_destroy(d); return rc; }
    {
        std::vector<float> tab((size_t)c.max_seq * c.head_dim);
        ptm_rope_table_host_factors(tab.data(), c.max_seq, c.head_dim, c.rope_freq_base, c.rope_scale, c.rope_factors_short,
                                    c.rope_factors_long, c.rope_orig_ctx, c.rope_attn_factor);
        if ((rc = hip_status(hipMemcpy(d->rope, tab.data(), tab.size() * 4, hipMemcpyHostToDevice))) != PTM_OK) { ptm_decode_destroy(d); return rc; }
        if (c.swa_window > 0) {  // ModelConfig::layer_rope_freq_base / layer_rope_scale, gguf_model.h:297-302
            ptm_rope_table_host_factors(tab.data(), c.max_seq, c.head_dim, c.rope_swa_freq_base, 1.0f, c.rope_factors_short,
                                        c.rope_factors_long, c.rope_orig_ctx, c.rope_attn_factor);
            if ((rc = hip_status(hipMemcpy(d->rope_swa, tab.data(), tab.size() * 4, hipMemcpyHostToDevice))) != PTM_OK) { ptm_decode_destroy(d); return rc; }
        }
    }
    hipLaunchKernelGGL(set_scalars_kernel, dim3(1), dim3(1), 0, d->stream, d->d_token, 0, d->d_past, (int64_t)0, d->d_step);
    if ((rc = hip_status(hipStreamSynchronize(d->stream))) != PTM_OK) { ptm_decode_destroy(d); return rc; }
    *out = d;
    return PTM_OK;
}

void ptm_decode_destroy(ptm_decoder* d) {
    if (!d) return;
    if (d->stream) (void)hipStreamSynchronize(d->stream);
    if (d->exec) (void)hipGraphExecDestroy(d->exec);
    if (d->graph) (void)hipGraphDestroy(d->graph);
    if (d->exec_s) (void)hipGraphExecDestroy(d->exec_s);
    if (d->graph_s) (void)hipGraphDestroy(d->graph_s);
    if (d->h_pinned) (void)hipHostFree(d->h_pinned);
    if (d->h_uniforms) (void)hipHostFree(d->h_uniforms);
    if (d->pf_slab) (void)hipFree(d->pf_slab);
    if (d->slab) (void)hipFree(d->slab);
    if (d->stream) (void)hipStreamDestroy(d->stream);
    delete d;
}

int ptm_decode_set_past_len(ptm_decoder* d, int64_t past_len) {
    if (!d) return PTM_E_NULL;
    if (past_len < 0 || past_len >= d->cfg.max_seq) return PTM_E_RANGE;
    d->past_len = past_len;
    d->dev_synced = false;
    return PTM_OK;
}

// Run n chained steps starting from `token` (greedy, or sampled with the stored parameters and the uniforms already
// on the device); token ids land in h_pinned[out_base .. out_base + n).
static int run_steps(ptm_decoder* d, int token, int n, bool sample = false) {
    if (d->status != PTM_OK) return PTM_E_STATE;
    if (n <= 0) return PTM_E_SHAPE;
    if (token < 0 || token >= d->cfg.vocab) return PTM_E_RANGE;
    if (d->past_len + n > d->cfg.max_seq) return PTM_E_RANGE;  // KV cache would overflow
    hipStream_t s = d->stream;
    int rc = PTM_OK;
    // sampled steps index their uniform draws by the step counter: they always start from 0
    const bool resume = !sample && d->dev_synced && (int64_t)token == d->dev_token && d->chain_base + n <= d->cfg.max_seq;
    d->dev_synced = false;
    if (!resume) {
        hipLaunchKernelGGL(set_scalars_kernel, dim3(1), dim3(1), 0, s, d->d_token, token, d->d_past, d->past_len, d->d_step);
        if ((rc = launch_status()) != PTM_OK) return rc;
        d->chain_base = 0;
    }
    d->out_base = d->chain_base;
    bool& captured = sample ? d->captured_s : d->captured;
    hipGraph_t& graph = sample ? d->graph_s : d->graph;
    hipGraphExec_t& exec = sample ? d->exec_s : d->exec;
    int done = 0;
    bool& fell_back = sample ? d->eager_fallback_s : d->eager_fallback;
    if (d->cfg.use_graph && !captured && !fell_back) {
        // first step eagerly (sets one-time kernel attributes outside capture), then capture
        if ((rc = enqueue_step(d, sample)) != PTM_OK) return d->status = rc;
        done = 1;
        // A failed capture or instantiation is not an error of the decoder: the step runs as plain launches from then on,
        // as the reference falls back to eager execution (gguf_model.h:2660-2665, :3093-3104).
        hipGraph_t g = nullptr;
        hipGraphExec_t ge = nullptr;
        bool ok = !d->debug_fail_capture;
        d->debug_fail_capture = false;
        if (ok) ok = hip_status(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal)) == PTM_OK;
        if (ok) {
            const int rc_enq = enqueue_step(d, sample);
            const int rc_end = hip_status(hipStreamEndCapture(s, &g));  // always ends the capture, also after a failed launch
            ok = rc_enq == PTM_OK && rc_end == PTM_OK && g != nullptr;
            if (ok) ok = hip_status(hipGraphInstantiate(&ge, g, nullptr, nullptr, 0)) == PTM_OK;
        }
        if (ok) {
            graph = g;
            exec = ge;
            captured = true;
            if (sample) d->sampled_key = sampler_launch_key(d->sampling, d->cfg.vocab);
        } else {
            if (g) (void)hipGraphDestroy(g);
            (void)hipGetLastError();  // the failure has been handled: do not let it surface at the next launch check
            fell_back = true;
        }
    }
    for (; done < n; ++done) {
        if (captured) rc = hip_status(hipGraphLaunch(exec, s));
        else rc = enqueue_step(d, sample);
        if (rc != PTM_OK) return d->status = rc;
    }
    if ((rc = hip_status(hipStreamSynchronize(s))) != PTM_OK) return d->status = rc;
    d->past_len += n;
    d->chain_base += n;
    d->dev_token = d->h_pinned[d->out_base + n - 1];
    d->dev_synced = !sample;
    return PTM_OK;
}

int ptm_decode_sampling_begin(ptm_decoder* d, const ptm_sampling* params) {
    if (!d || !params) return PTM_E_NULL;
    if (d->status != PTM_OK) return PTM_E_STATE;
    const bool greedy = !(params->temperature >= 1e-6f);
    if (!greedy) {
        if (!(params->top_p > 0.0f)) return PTM_E_SHAPE;
    }
    hipStream_t s = d->stream;
    int rc = hip_status(hipMemcpyAsync(d->d_sampling, params, sizeof(ptm_sampling), hipMemcpyHostToDevice, s));
    if (rc != PTM_OK) return rc;
    hipLaunchKernelGGL(fill_i32_kernel, dim3(64), dim3(256), 0, s, d->d_counts, (int64_t)d->cfg.vocab, 0);
    if ((rc = launch_status()) != PTM_OK) return rc;
    if ((rc = hip_status(hipStreamSynchronize(s))) != PTM_OK) return rc;  // params may be a temporary of the caller
    d->sampling = *params;
    d->sampling_set = true;
    // The sampler's launch sequence is chosen on the host from the parameters (candidate list or whole-vocabulary passes,
    // with or without the top-k select and the nucleus walk): a captured sampled step only serves parameters of the same
    // class.  A request of another class drops that graph; the next sampled step captures the new sequence.
    if (d->captured_s && sampler_launch_key(*params, d->cfg.vocab) != d->sampled_key) {
        (void)hipGraphExecDestroy(d->exec_s);
        (void)hipGraphDestroy(d->graph_s);
        d->exec_s = nullptr;
        d->graph_s = nullptr;
        d->captured_s = false;
        d->sampled_key = -1;
    }
    return PTM_OK;
}

// Test seam for the capture fallback: the decoder's next capture attempt reports failure on the host before anything is
// recorded, so the step goes on as plain launches exactly as after a real capture or instantiation failure.
int ptm_decode_debug_fail_next_capture(ptm_decoder* d) {
    if (!d) return PTM_E_NULL;
    d->debug_fail_capture = true;
    return PTM_OK;
}

int ptm_decode_sample(ptm_decoder* d, int token_id, int n, const float* uniforms_host, int64_t* out_tokens) {
    if (!d || !uniforms_host || !out_tokens) return PTM_E_NULL;
    if (!d->sampling_set) return PTM_E_STATE;
    if (n <= 0 || n > d->cfg.max_seq) return PTM_E_SHAPE;
    memcpy(d->h_uniforms, uniforms_host, 4 * (size_t)n);  // the previous call's copy has completed: every call ends synchronised
    int rc = hip_status(hipMemcpyAsync(d->d_uniforms, d->h_uniforms, 4 * (size_t)n, hipMemcpyHostToDevice, d->stream));
    if (rc != PTM_OK) return rc;
    if ((rc = run_steps(d, token_id, n, true)) != PTM_OK) return rc;
    for (int i = 0; i < n; ++i) out_tokens[i] = d->h_pinned[d->out_base + i];
    return PTM_OK;
}

int ptm_decode_prefill(ptm_decoder* d, const int32_t* tokens, int n, int chunk_rows, int64_t* next_token);

// The serving loop (promeserve/api_handlers.h:848-923) in one call: prompt, then sample / check for a stop token /
// feed back until max_new tokens or a stop token (which is not part of the output).  Tokens are generated in chained
// runs of 16 steps; when a stop token turns up inside a run the steps after it are dropped (the cache rows they wrote
// lie beyond past_len and are overwritten by whatever comes next).
int ptm_decode_generate(ptm_decoder* d, const int32_t* prompt, int n_prompt, const ptm_sampling* params,
                        const float* uniforms_host, int max_new, const int32_t* stop_ids, int n_stop, int64_t* out_tokens,
                        int* n_out) {
    if (!d || !prompt || !params || !uniforms_host || !out_tokens || !n_out || (n_stop > 0 && !stop_ids)) return PTM_E_NULL;
    if (n_prompt <= 0 || max_new <= 0 || n_stop < 0) return PTM_E_SHAPE;
    if (d->status != PTM_OK) return PTM_E_STATE;
    if (d->past_len + n_prompt - 1 + max_new > d->cfg.max_seq) return PTM_E_RANGE;
    *n_out = 0;
    int rc;
    if (n_prompt > 1) {
        int64_t unused;
        if ((rc = ptm_decode_prefill(d, prompt, n_prompt - 1, 0, &unused)) != PTM_OK) return rc;
    } else if (prompt[0] < 0 || prompt[0] >= d->cfg.vocab) {
        return PTM_E_RANGE;
    }
    if ((rc = ptm_decode_sampling_begin(d, params)) != PTM_OK) return rc;
    int token = prompt[n_prompt - 1], produced = 0;
    while (produced < max_new) {
        const int run = max_new - produced < 16 ? max_new - produced : 16;
        if ((rc = ptm_decode_sample(d, token, run, uniforms_host + produced, out_tokens + produced)) != PTM_OK) return rc;
        for (int i = 0; i < run; ++i) {
            const int64_t t = out_tokens[produced + i];
            for (int k = 0; k < n_stop; ++k)
                if (t == stop_ids[k]) {
                    d->past_len -= run - (i + 1);  // steps i+1.. of the run fed the stop token and what followed it
                    *n_out = produced + i;
                    return PTM_OK;
                }
        }
        produced += run;
        token = (int)out_tokens[produced - 1];
    }
    *n_out = produced;
    return PTM_OK;
}

int ptm_decode_reserve_prefill(ptm_decoder* d, int rows) {
    if (!d) return PTM_E_NULL;
    if (d->status != PTM_OK) return PTM_E_STATE;
    if (rows <= 0) return PTM_E_SHAPE;
    if (d->untuned_types) return PTM_OK;  // such models are prefilled token by token: no row scratch
    if (rows > 2048) rows = 2048;
    const int rc = hip_status(hipStreamSynchronize(d->stream));  // the slab may be replaced: nothing may still use it
    if (rc != PTM_OK) return rc;
    return prefill_alloc(d, rows);
}

int ptm_decode_prefill(ptm_decoder* d, const int32_t* tokens, int n, int chunk_rows, int64_t* next_token) {
    if (!d || !tokens || !next_token) return PTM_E_NULL;
    if (d->status != PTM_OK) return PTM_E_STATE;
    if (n <= 0) return PTM_E_SHAPE;
    if (d->past_len + n > d->cfg.max_seq) return PTM_E_RANGE;  // KV cache would overflow
    for (int i = 0; i < n; ++i)
        if (tokens[i] < 0 || tokens[i] >= d->cfg.vocab) return PTM_E_RANGE;
    const ptm_decode_config& c = d->cfg;
    if (d->untuned_types) {
        // no row-batched GEMM for these types: the prompt is stepped, each step a full decode step whose token is dropped
        int rc = PTM_OK;
        for (int i = 0; i < n && rc == PTM_OK; ++i) rc = run_steps(d, tokens[i], 1);
        if (rc == PTM_OK) *next_token = d->h_pinned[d->out_base];
        return rc;
    }
    d->dev_synced = false;
    if (chunk_rows <= 0) chunk_rows = 2048;  // measured: 2048-row chunks run a 4096-token prompt 1.4x faster than 512-row ones
    if (chunk_rows > 2048) chunk_rows = 2048;  // bounds the row scratch (and the launch grids) whatever the prompt length
    if (chunk_rows > n) chunk_rows = n;
    int rc = prefill_alloc(d, chunk_rows);
    if (rc != PTM_OK) return rc;
    hipStream_t s = d->stream;
    int last_rows = 0;
    for (int done = 0; done < n; done += last_rows) {
        last_rows = n - done < chunk_rows ? n - done : chunk_rows;
        if ((rc = prefill_chunk(d, tokens + done, last_rows, d->past_len + done)) != PTM_OK) return d->status = rc;
    }
    // only the last row is projected to logits (gguf_model.h:2551-2559): hand it to the decode tail, with the device-side
    // position set so that the tail's bookkeeping leaves it at past_len + n
    if ((rc = hip_status(hipMemcpyAsync(d->x, d->pf_x + (size_t)(last_rows - 1) * c.hidden, 4 * (size_t)c.hidden,
                                        hipMemcpyDeviceToDevice, s))) != PTM_OK) return d->status = rc;
    hipLaunchKernelGGL(set_scalars_kernel, dim3(1), dim3(1), 0, s, d->d_token, (int)tokens[n - 1], d->d_past,
                       d->past_len + n - 1, d->d_step);
    if ((rc = launch_status()) != PTM_OK) return d->status = rc;
    if (c.lm_head.ggml_type == PTM_TYPE_Q6_K) {
        rc = q6k_gemv_argmax_impl(c.lm_head.data, d->x, c.out_norm, c.rms_eps, 0, d->xn, d->logits, c.hidden, c.vocab,
                                  c.lm_head.row_stride_bytes, d->d_next, d->amax_ws,
                                  ArgmaxAdvance{d->d_token, d->d_past, d->d_step, d->d_tokens, c.max_seq}, s);
    } else {
        rc = ptm_rms_norm(d->x, c.out_norm, d->xn, 1, c.hidden, c.rms_eps, 0, nullptr, s);
        if (rc == PTM_OK) rc = gemv_any(c.lm_head, d->xn, d->logits, false, s);
        if (rc == PTM_OK) rc = ptm_argmax(d->logits, d->d_next, c.vocab, s);
        if (rc == PTM_OK) {
            hipLaunchKernelGGL(advance_kernel, dim3(1), dim3(1), 0, s, d->d_next, d->d_token, d->d_past, d->d_step,
                               d->d_tokens, c.max_seq);
            rc = launch_status();
        }
    }
    if (rc != PTM_OK) return d->status = rc;
    if ((rc = hip_status(hipStreamSynchronize(s))) != PTM_OK) return d->status = rc;
    d->past_len += n;
    *next_token = d->h_pinned[0];
    return PTM_OK;
}

int ptm_decode_step(ptm_decoder* d, int token_id, int64_t* next_token) {
    if (!d || !next_token) return PTM_E_NULL;
    const int rc = run_steps(d, token_id, 1);
    if (rc == PTM_OK) *next_token = d->h_pinned[d->out_base];
    return rc;
}

int ptm_decode_step_trace(ptm_decoder* d, int token_id, int64_t* next_token, float* trace_device) {
    if (!d || !next_token || !trace_device) return PTM_E_NULL;
    if (d->status != PTM_OK) return PTM_E_STATE;
    if (token_id < 0 || token_id >= d->cfg.vocab) return PTM_E_RANGE;
    if (d->past_len + 1 > d->cfg.max_seq) return PTM_E_RANGE;
    hipStream_t s = d->stream;
    d->dev_synced = false;
    hipLaunchKernelGGL(set_scalars_kernel, dim3(1), dim3(1), 0, s, d->d_token, token_id, d->d_past, d->past_len, d->d_step);
    int rc = launch_status();
    if (rc != PTM_OK) return rc;
    if ((rc = enqueue_step(d, false, trace_device)) != PTM_OK) return d->status = rc;
    if ((rc = hip_status(hipStreamSynchronize(s))) != PTM_OK) return d->status = rc;
    d->past_len += 1;
    *next_token = d->h_pinned[0];
    return PTM_OK;
}

int ptm_decode_greedy(ptm_decoder* d, int first_token, int n, int64_t* tokens_out) {
    if (!d || !tokens_out) return PTM_E_NULL;
    const int rc = run_steps(d, first_token, n);
    if (rc == PTM_OK) for (int i = 0; i < n; ++i) tokens_out[i] = d->h_pinned[d->out_base + i];
    return rc;
}

int ptm_decode_graph_state(const ptm_decoder* d, int sampled) {
    if (!d) return PTM_E_NULL;
    if (sampled ? d->captured_s : d->captured) return 1;
    if (sampled ? d->eager_fallback_s : d->eager_fallback) return 2;
    return 0;
}

const float* ptm_decode_logits(ptm_decoder* d) { return d ? d->logits : nullptr; }
const float* ptm_decode_hidden(ptm_decoder* d) { return d ? d->xn : nullptr; }
void* ptm_decode_stream(ptm_decoder* d) { return d ? d->stream : nullptr; }

}  // extern "C"
