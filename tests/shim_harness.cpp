// Test harness (not part of the library): one batch-1 decode step written purely against the reference's launcher
// names, `at::cuda::launch_*`, as include/ptm_at_cuda_shim.h provides them.  It issues the launches in the order
// GGUFModel::forward_decode does for a Q4_K_M model (torch/io/gguf_model.h:2670-3087: embedding lookup, separate attention
// norm + per-type GEMVs because q/k and v differ in type, fused QK-norm + RoPE + KV write, flash-decode, output projection
// accumulated into a copy of the residual, fused norm + gate/up, SiLU, down projection + add, final norm, logits) and the
// argmax of generate() (:4855).  Host C++ only; built by __graft_entry__.build() into tests/libshim_harness.so and driven
// through ctypes by tests/test_gpu_shim.py.
#include <cmath>

#include "ptm_at_cuda_shim.h"

extern "C" {

struct ShimQW {
    void* gpu_data;
    int32_t type;  // ggml type id
    int32_t rows, cols;
    int64_t row_stride_bytes;
};

struct ShimLayer {
    ShimQW q, k, v, o, gate, up, down;
    float *attn_norm, *ffn_norm, *q_norm, *k_norm;
    float *key_cache, *value_cache;  // fp32 [max_seq][kv_dim], as the reference's decode keeps them
};

struct ShimModel {
    int32_t n_layers, H, n_heads, n_kv_heads, head_dim, inter, vocab, max_seq;
    float rope_freq_base, eps;
    int32_t rope_neox;
    const float* rope_table;  // device, optional
    const float* emb;         // device fp32 [vocab][H]
    ShimLayer* layers;        // host array
    float* output_norm;
    ShimQW lm_head;
    // scratch (InferenceScratchPool, gguf_model.h:554-631)
    float *buf_x[2], *buf_normed, *buf_q, *buf_k, *buf_v, *buf_attn, *buf_h, *buf_gate, *buf_up, *buf_silu, *buf_down,
        *buf_logits, *fd_partial_O, *fd_partial_lse, *fd_partial_max;
    int* d_token_id;
    int64_t* d_past_len;
    int64_t* d_argmax_idx;
};

static void gemv_scratch(const ShimQW& qw, const float* x, float* y, cudaStream_t s) {
    const int K = qw.cols, Nr = qw.rows;
    if (qw.type == 12) at::cuda::launch_q4km_persistent_gemv(qw.gpu_data, x, y, K, Nr, qw.row_stride_bytes, s);
    else if (qw.type == 14) at::cuda::launch_q6k_gemv(qw.gpu_data, x, y, K, Nr, qw.row_stride_bytes, s);
    else if (qw.type == 13) at::cuda::launch_q5k_gemv(qw.gpu_data, x, y, K, Nr, qw.row_stride_bytes, s);
}

// graph_style != 0: the position is read from *d_past_len by the `_graph` launchers; 0: it is the host argument past_len.
// Returns the number of launcher calls made, or a negative value for a model this harness does not cover.
int shim_forward_decode(ShimModel* m, int graph_style, int64_t past_len, cudaStream_t s) {
    if (!m) return -1;
    const int H = m->H, n_heads = m->n_heads, n_kv_heads = m->n_kv_heads, head_dim = m->head_dim, inter = m->inter;
    const int q_dim = n_heads * head_dim, kv_dim = n_kv_heads * head_dim;
    const float eps = m->eps;
    const bool add_one = false;
    int calls = 0;
    at::cuda::ptm_shim_set_context(m->max_seq, m->rope_neox, m->rope_table);
    at::cuda::launch_embedding_lookup(m->emb, m->buf_x[0], m->d_token_id, H, s); ++calls;
    int cur = 0;
    for (int i = 0; i < m->n_layers; ++i) {
        ShimLayer& layer = m->layers[i];
        float* x_ptr = m->buf_x[cur];
        at::cuda::launch_rms_norm(x_ptr, layer.attn_norm, m->buf_normed, 1, H, eps, add_one, s); ++calls;
        gemv_scratch(layer.q, m->buf_normed, m->buf_q, s);
        gemv_scratch(layer.k, m->buf_normed, m->buf_k, s);
        gemv_scratch(layer.v, m->buf_normed, m->buf_v, s);
        calls += 3;
        const float scale = 1.0f / std::sqrt(static_cast<float>(head_dim));
        if (graph_style) {
            at::cuda::launch_fused_qknorm_rope_kvwrite_graph(m->buf_q, m->buf_k, m->buf_v, layer.q_norm, layer.k_norm,
                                                             layer.key_cache, layer.value_cache, n_heads, n_kv_heads,
                                                             head_dim, m->d_past_len, m->rope_freq_base, eps, add_one, s);
            at::cuda::launch_flash_decode_graph(m->buf_q, layer.key_cache, layer.value_cache, m->buf_attn, m->fd_partial_O,
                                                m->fd_partial_lse, m->fd_partial_max, n_heads, n_kv_heads, head_dim,
                                                m->d_past_len, m->max_seq, scale, s);
        } else {
            at::cuda::launch_fused_qknorm_rope_kvwrite(m->buf_q, m->buf_k, m->buf_v, layer.q_norm, layer.k_norm,
                                                       layer.key_cache, layer.value_cache, n_heads, n_kv_heads, head_dim,
                                                       static_cast<int>(past_len), m->rope_freq_base, eps, add_one, past_len, s);
            at::cuda::launch_flash_decode(m->buf_q, layer.key_cache, layer.value_cache, m->buf_attn, m->fd_partial_O,
                                          m->fd_partial_lse, m->fd_partial_max, n_heads, n_kv_heads, head_dim,
                                          static_cast<int>(past_len + 1), scale, s);
        }
        calls += 2;
        if (layer.o.type == 12) {  // residual copied, projection accumulated on top
            at::cuda::launch_copy(x_ptr, m->buf_h, H, s);
            at::cuda::launch_q4km_persistent_gemv_accumulate(layer.o.gpu_data, m->buf_attn, m->buf_h, layer.o.cols,
                                                             layer.o.rows, layer.o.row_stride_bytes, s);
            calls += 2;
        } else {
            gemv_scratch(layer.o, m->buf_attn, m->buf_down, s);
            at::cuda::launch_add(x_ptr, m->buf_down, m->buf_h, H, s);
            calls += 2;
        }
        if (layer.gate.type == 12 && layer.up.type == 12) {
            at::cuda::launch_q4km_fused_rmsnorm_gate_up_gemv(m->buf_h, layer.ffn_norm, layer.gate.gpu_data, layer.up.gpu_data,
                                                             m->buf_gate, m->buf_up, H, layer.gate.rows, layer.up.rows,
                                                             layer.gate.row_stride_bytes, eps, add_one, s);
            ++calls;
        } else {
            at::cuda::launch_rms_norm(m->buf_h, layer.ffn_norm, m->buf_normed, 1, H, eps, add_one, s);
            gemv_scratch(layer.gate, m->buf_normed, m->buf_gate, s);
            gemv_scratch(layer.up, m->buf_normed, m->buf_up, s);
            calls += 3;
        }
        at::cuda::launch_silu_mul(m->buf_gate, m->buf_up, m->buf_silu, inter, s); ++calls;
        const int next = 1 - cur;
        gemv_scratch(layer.down, m->buf_silu, m->buf_down, s);
        at::cuda::launch_add(m->buf_h, m->buf_down, m->buf_x[next], H, s);
        calls += 2;
        cur = next;
    }
    at::cuda::launch_rms_norm(m->buf_x[cur], m->output_norm, m->buf_normed, 1, H, eps, add_one, s); ++calls;
    gemv_scratch(m->lm_head, m->buf_normed, m->buf_logits, s); ++calls;
    at::cuda::launch_argmax(m->buf_logits, m->d_argmax_idx, m->vocab, s); ++calls;
    (void)q_dim; (void)kv_dim;
    return calls;
}

}  // extern "C"
