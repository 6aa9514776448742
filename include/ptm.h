/*
 * ptm.h — C ABI of libptm_hip.so: MI355X (gfx950) kernels for the GGUF Q4_K / Q6_K
 * batch-1 decode path of PromeTorch.
 *
 * Every entry point is the flat-C counterpart of one operator the reference declares in
 * aten/src/ATen/cuda/CUDAOps.h (C++ `at::cuda::launch_*`, cited per function below);
 * include/ptm_at_cuda_shim.h re-exposes them under the reference's own names.
 *
 * Conventions (reference: CUDAOps.h, gguf_model.h:3117-3140):
 *   - all pointers are DEVICE pointers unless a parameter says "host";
 *   - weights are raw GGUF super-blocks exactly as stored in the file, row-major
 *     [N][K/256] blocks, row_stride_bytes = K/256 * {144 (Q4_K), 210 (Q6_K)};
 *   - activations and outputs are fp32; K % 256 == 0; x and y 16-byte aligned;
 *   - launches are asynchronous on `stream` (a hipStream_t, NULL = default stream),
 *     allocate nothing, and are legal inside hipStreamBeginCapture/EndCapture;
 *   - unlike the reference's void launchers, each call returns PTM_OK or a negative
 *     PTM_E_* after validating its arguments on the host; nothing throws.
 */
#ifndef PTM_H
#define PTM_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* ptm_stream_t; /* hipStream_t */

enum {
    PTM_OK = 0,
    PTM_E_NULL = -1,        /* required pointer is NULL */
    PTM_E_SHAPE = -2,       /* K not a multiple of 256, non-positive size, stride too small ... */
    PTM_E_ALIGN = -3,       /* pointer/stride alignment precondition violated */
    PTM_E_UNSUPPORTED = -4, /* quant type / head_dim / size outside what the kernels implement */
    PTM_E_HIP = -5,         /* a HIP runtime call failed (ptm_last_hip_error() has the code) */
    PTM_E_RANGE = -6,       /* position / token beyond the allocated cache or table */
    PTM_E_STATE = -7,       /* object used before initialisation or after an error */
    PTM_E_IO = -8,          /* file cannot be opened / mapped */
    PTM_E_FORMAT = -9,      /* file is not well-formed GGUF, or a required key is missing or of the wrong kind */
    PTM_E_NOT_FOUND = -10   /* no tensor / metadata key of that name */
};

enum { PTM_TYPE_Q5_0 = 6, PTM_TYPE_Q8_0 = 8, PTM_TYPE_Q4_K = 12, PTM_TYPE_Q5_K = 13, PTM_TYPE_Q6_K = 14 }; /* ggml type ids, gguf_dequant.h:29-58 */

const char* ptm_strerror(int code);
int ptm_last_hip_error(void);
int ptm_version(void);
/* Number of compute units of the current device (used to size grids). */
int ptm_device_cus(void);

/* ---- dequantisation -------------------------------------------------------------- */
/* Q4_K / Q6_K super-blocks -> fp32, bit-exact with dequantize_q4_k / dequantize_q6_k
 * (gguf_dequant.h:304-341, :395-430). n_elems % 256 == 0. */
int ptm_dequant_q4k(const void* blocks, float* out, int64_t n_elems, ptm_stream_t stream);
int ptm_dequant_q6k(const void* blocks, float* out, int64_t n_elems, ptm_stream_t stream);
/* Q4_K -> fp16, COLUMN-major out[k*N + n]; replaces launch_dequant_q4k_to_fp16 (CUDAOps.h:477-480). */
int ptm_dequant_q4k_to_fp16(const void* W, void* out_fp16, int K, int N, int64_t row_stride_bytes,
                            ptm_stream_t stream);

/* ---- Q8 activation blocks -------------------------------------------------------- */
/* Quantise x[K] the way the reference CPU GEMV does (cpu_quant_gemv.h:147-198): per 32
 * values d = amax/127, q = clamp(rne(x/d), -127, 127), sum = d * sum(q).
 * Device layout of q8: int8 qs[K], then float d[K/32], then float sum[K/32]
 * (ptm_q8_bytes(K) = K + K/4 bytes, 16-byte aligned).  Plays the role of
 * launch_quantize_q8_1 (CUDAOps.h:462-464) with the CPU path's block format. */
int64_t ptm_q8_bytes(int K);
int ptm_quantize_q8(const float* x, void* q8, int K, ptm_stream_t stream);

/* ---- dequant-fused GEMV: y[N] (+)= W[N,K] . x[K] --------------------------------- */
/* Q4_K with the reference CPU semantics (Q8 activations, exact int32 sub-block dots, fp32
 * combine; cpu_quant_gemv.h:505-685).  Replaces launch_q4km_gemv / launch_q4km_persistent_gemv
 * / _v2 (CUDAOps.h:427-448) and, with accumulate != 0, launch_q4km_persistent_gemv_accumulate
 * (CUDAOps.h:613-616). x is quantised inside the kernel. */
int ptm_q4k_gemv(const void* W, const float* x, float* y, int K, int N, int64_t row_stride_bytes,
                 int accumulate, ptm_stream_t stream);
/* Same with x already quantised by ptm_quantize_q8 (replaces launch_q4km_q8_gemv, CUDAOps.h:467-470). */
int ptm_q4k_gemv_q8(const void* W, const void* x_q8, float* y, int K, int N, int64_t row_stride_bytes,
                    int accumulate, ptm_stream_t stream);
/* Q4_K with fp32 activations, no Q8 rounding: y (+)= sum_k fma(d*sc, q, -(dmin*m)) * x_k, the arithmetic of the reference's
 * scalar kernel (q4k_gemv_scalar, cpu_quant_gemv.h:689-767; its AVX2 twin q4k_gemv_avx2_float :62-134), which a host with
 * AVX2 never dispatches to.  The exact-math cross-check of ptm_q4k_gemv; a plain row-per-wave kernel, not tuned. */
int ptm_q4k_gemv_f32act(const void* W, const float* x, float* y, int K, int N, int64_t row_stride_bytes, int accumulate,
                        ptm_stream_t stream);
/* Q6_K with fp32 activations (cpu_quant_gemv.h:883-1020). Replaces launch_q6k_gemv (CUDAOps.h:498-501). */
int ptm_q6k_gemv(const void* W, const float* x, float* y, int K, int N, int64_t row_stride_bytes,
                 int accumulate, ptm_stream_t stream);
/* Q6_K GEMV with a fused greedy argmax (strict '>', lowest index on ties):
 * writes *out_index (int64, device) and, if logits != NULL, logits[N].
 * workspace: ptm_argmax_workspace_bytes(N) bytes of device scratch.
 * Fuses launch_q6k_gemv + launch_argmax (CUDAOps.h:498-501, :145). */
int64_t ptm_argmax_workspace_bytes(int N);
int ptm_q6k_gemv_argmax(const void* W, const float* x, float* logits, int K, int N,
                        int64_t row_stride_bytes, int64_t* out_index, void* workspace,
                        ptm_stream_t stream);
/* The same for callers that cannot allocate device memory (code under hipGraph capture, tight serving loops,
 * harnesses that forbid hipMalloc): no workspace argument, the per-workgroup partials live in a device array inside the
 * library (512 KiB per GPU, held until the process ends).  No counterpart in the reference.  N above
 * ptm_q6k_gemv_argmax_noalloc_max_rows() (262144) returns PTM_E_RANGE.  Calls no hipMalloc / hipFree.  All calls on one
 * GPU share that GPU's array: calls that overlap in time on one GPU (different streams) race; calls ordered on one
 * stream do not.  Same results as ptm_q6k_gemv_argmax.
 * The first call on a device looks the array's address up and raises the kernels' LDS cap; neither may happen while a
 * stream is capturing.  A caller that captures calls ptm_q6k_gemv_argmax_noalloc_init() once per device beforehand, with
 * that device current (it allocates nothing either); after it every call is capture-legal. */
int ptm_q6k_gemv_argmax_noalloc_init(void);
int ptm_q6k_gemv_argmax_noalloc_max_rows(void);
int ptm_q6k_gemv_argmax_noalloc(const void* W, const float* x, float* logits, int K, int N, int64_t row_stride_bytes,
                                int64_t* out_index, ptm_stream_t stream);
/* Type dispatcher mirroring cpu_quant_gemv (cpu_quant_gemv.h:1635-1688) and gemv_scratch
 * (gguf_model.h:3117-3140): 12 -> Q4_K, 14 -> Q6_K, 13 -> Q5_K, 8 -> Q8_0, 6 -> Q5_0; anything else returns
 * PTM_E_UNSUPPORTED and launches nothing (the reference silently no-ops).  ptm_quant_gemv_supported mirrors
 * cpu_quant_gemv_supported (cpu_quant_gemv.h:1691-1694). */
int ptm_quant_gemv(uint32_t ggml_type, const void* W, const float* x, float* y, int K, int N,
                   int64_t row_stride_bytes, int accumulate, ptm_stream_t stream);
int ptm_quant_gemv_supported(uint32_t ggml_type);

/* The dispatcher's other formats, fp32 activations, y (+)= W.x (q8_0_gemv_avx2 cpu_quant_gemv.h:784-826, q5k_gemv_avx2
 * :1091-1185, q5_0_gemv_scalar :1572-1630).  K a multiple of 32 (Q8_0: 34-byte blocks; Q5_0: 22-byte blocks; W and the
 * row stride 2-byte aligned) or of 256 (Q5_K: 176-byte super-blocks, 4-byte aligned); x 16-byte aligned.  No file of
 * the decode path's models holds these types: the kernels are plain row-per-wave ones, not tuned. */
int ptm_q8_0_gemv(const void* W, const float* x, float* y, int K, int N, int64_t row_stride_bytes, int accumulate,
                  ptm_stream_t stream);
int ptm_q5k_gemv(const void* W, const float* x, float* y, int K, int N, int64_t row_stride_bytes, int accumulate,
                 ptm_stream_t stream);
int ptm_q5_0_gemv(const void* W, const float* x, float* y, int K, int N, int64_t row_stride_bytes, int accumulate,
                  ptm_stream_t stream);
/* dequantize_q8_0 / dequantize_q5_k (gguf_dequant.h:237-255, :348-388), bit-exact. */
int ptm_dequant_q8_0(const void* blocks, float* out, int64_t n_elems, ptm_stream_t stream);
int ptm_dequant_q5k(const void* blocks, float* out, int64_t n_elems, ptm_stream_t stream);

/* Two / three Q4_K projections of the same x in one launch.
 * Replace launch_q4km_fused_gate_up_gemv (CUDAOps.h:453-458) and
 * launch_q4km_fused_qkv_gemv (CUDAOps.h:578-583). */
int ptm_q4k_fused_gate_up_gemv(const void* w_gate, const void* w_up, const float* x, float* y_gate,
                               float* y_up, int K, int N_gate, int N_up, int64_t row_stride_bytes,
                               ptm_stream_t stream);
int ptm_q4k_fused_qkv_gemv(const void* w_q, const void* w_k, const void* w_v, const float* x,
                           float* out_q, float* out_k, float* out_v, int K, int N_q, int N_k, int N_v,
                           int64_t row_stride_bytes, ptm_stream_t stream);
/* RMSNorm(x)*gamma computed in the kernel, then the projection(s).  Replace
 * launch_q4km_fused_rmsnorm_gemv / _qkv_gemv / _gate_up_gemv (CUDAOps.h:589-628). */
int ptm_q4k_fused_rmsnorm_gemv(const float* x, const float* norm_w, const void* W, float* y, int K,
                               int N, int64_t row_stride_bytes, float eps, int add_one,
                               ptm_stream_t stream);
int ptm_q4k_fused_rmsnorm_qkv_gemv(const float* x, const float* norm_w, const void* w_q, const void* w_k,
                                   const void* w_v, float* out_q, float* out_k, float* out_v, int K,
                                   int N_q, int N_k, int N_v, int64_t row_stride_bytes, float eps,
                                   int add_one, ptm_stream_t stream);
int ptm_q4k_fused_rmsnorm_gate_up_gemv(const float* x, const float* norm_w, const void* w_gate,
                                       const void* w_up, float* y_gate, float* y_up, int K, int N_gate,
                                       int N_up, int64_t row_stride_bytes, float eps, int add_one,
                                       ptm_stream_t stream);
/* RMSNorm + gate/up projections + SiLU(gate)*up in one launch: act[N] (no counterpart launcher in
 * the reference; it is launch_q4km_fused_rmsnorm_gate_up_gemv followed by launch_silu_mul,
 * gguf_model.h:2954-2986). */
int ptm_q4k_fused_rmsnorm_gate_up_silu(const float* x, const float* norm_w, const void* w_gate,
                                       const void* w_up, float* act, int K, int N,
                                       int64_t row_stride_bytes, float eps, int add_one,
                                       ptm_stream_t stream);

/* ---- decode-step glue ------------------------------------------------------------ */
/* Row-wise RMSNorm: out = x * 1/sqrt(mean(x^2)+eps) * (gamma [+1]).  launch_rms_norm (CUDAOps.h:382-385).
 * If q8_out != NULL (rows must be 1, hidden % 256 == 0) the Q8 blocks of the result are written too. */
int ptm_rms_norm(const float* in, const float* weight, float* out, int rows, int hidden, float eps,
                 int add_one, void* q8_out, ptm_stream_t stream);
/* In-place per-head RMSNorm over [rows][n_heads][head_dim]. launch_per_head_rms_norm (CUDAOps.h:387-390). */
int ptm_per_head_rms_norm(float* data, const float* weight, int rows, int n_heads, int head_dim,
                          float eps, int add_one, ptm_stream_t stream);
/* Fused per-head QK-norm + RoPE + K/V cache append for one token.
 * Q [n_heads*head_dim] and K [n_kv_heads*head_dim] are updated in place; K and V rows are written
 * to the caches at row *d_past_len.  q_norm_w/k_norm_w may be NULL (no QK-norm).
 * neox != 0: pairs (d, d+head_dim/2) as the reference CPU path applies for qwen3
 * (hot_loops.cpp:2035-2061); neox == 0: interleaved pairs (2d, 2d+1) as the reference CUDA
 * kernel (FlashDecoding.cu:309-312).  kv_fp16 != 0: caches are fp16 [max_seq][kv_dim], else fp32.
 * rope_table: optional [max_seq][head_dim] fp32 rows of (cos[0..hd/2), sin[0..hd/2)); if NULL the
 * angles are computed on the device from rope_freq_base.
 * Replaces launch_fused_qknorm_rope_kvwrite(_graph) (CUDAOps.h:563-570, :653-659). */
int ptm_qknorm_rope_kvwrite(float* Q, float* K, const float* V, const float* q_norm_w,
                            const float* k_norm_w, void* K_cache, void* V_cache, int n_heads,
                            int n_kv_heads, int head_dim, const int64_t* d_past_len, int max_seq,
                            float rope_freq_base, const float* rope_table, float eps, int add_one,
                            int neox, int kv_fp16, ptm_stream_t stream);
/* The same with the position given by the host, for callers outside a captured graph: the rotation uses `position`, the
 * K and V rows land in cache row `cache_offset_row` (the two may differ).  Replaces the non-graph
 * launch_fused_qknorm_rope_kvwrite (CUDAOps.h:563-570; FlashDecoding.cu:256-395).  max_seq: height of the caches (and of
 * rope_table when given); a row or position outside it returns PTM_E_RANGE. */
int ptm_qknorm_rope_kvwrite_pos(float* Q, float* K, const float* V, const float* q_norm_w, const float* k_norm_w,
                                void* K_cache, void* V_cache, int n_heads, int n_kv_heads, int head_dim, int position,
                                int64_t cache_offset_row, int max_seq, float rope_freq_base, const float* rope_table,
                                float eps, int add_one, int neox, int kv_fp16, ptm_stream_t stream);
/* Host-side helper: fill table[max_seq][head_dim] with the reference's fp32 cos/sin
 * (hot_loops.cpp:1853-1876: freq = 1/powf(base, 2d/hd), theta = pos*freq). table is a HOST pointer. */
int ptm_rope_table_host(float* table, int max_seq, int head_dim, float rope_freq_base);
/* The same with linear position scaling: theta = (pos / scale) * freq when scale is positive and not 1
 * (the `scale` argument of rope_precompute, hot_loops.cpp:1853-1860; ModelConfig::rope_scale, gguf_model.h:71). */
int ptm_rope_table_host_scaled(float* table, int max_seq, int head_dim, float rope_freq_base, float scale);
/* The same with phi3's LongRoPE terms (hot_loops.cpp:1861-1873; ModelConfig::rope_factors_for, gguf_model.h:285-296): the
 * frequency of pair d is divided by factors[d] - row pos takes factors_short while pos + 1 <= orig_ctx and factors_long
 * beyond (host arrays of head_dim / 2 floats; NULL: no factors for that range; orig_ctx <= 0: none at all) - and cos and sin
 * are multiplied with attn_factor (0 or 1: not). */
int ptm_rope_table_host_factors(float* table, int max_seq, int head_dim, float rope_freq_base, float scale,
                                const float* factors_short, const float* factors_long, int orig_ctx, float attn_factor);
/* fp32 rows -> fp16 cache rows. launch_fp16_kv_cache_write (CUDAOps.h:635-638). */
int ptm_fp16_kv_cache_write(const float* src, void* dst_cache_fp16, int64_t num_new_rows, int64_t cols,
                            int64_t offset_row, ptm_stream_t stream);

/* Split-KV single-token GQA attention.  Attends positions [0, *d_past_len] (inclusive: the row
 * just appended).  Caches are [max_seq][n_kv_heads*head_dim] fp16 (kv_fp16 != 0) or fp32.
 * Scratch (caller-owned): partial_O [S*n_heads*head_dim], partial_lse [S*n_heads] (sum of exp),
 * partial_max [S*n_heads] with S = ptm_flash_decode_num_splits(max_seq).
 * Replaces launch_flash_decode(_fp16)(_graph) + flash_decode_num_splits / _kv_chunk_size
 * (CUDAOps.h:543-557, :641-673). head_dim must be 64, 128 or 256. */
int ptm_flash_decode_kv_chunk_size(void);
int ptm_flash_decode_num_splits(int total_seq);
int ptm_flash_decode(const float* Q, const void* K_cache, const void* V_cache, float* O,
                     float* partial_O, float* partial_lse, float* partial_max, int n_heads,
                     int n_kv_heads, int head_dim, const int64_t* d_past_len, int max_seq, float scale,
                     int kv_fp16, ptm_stream_t stream);
/* The same with the row count given by the host: attends rows [0, total_seq) of caches holding at least total_seq rows;
 * scratch sized with ptm_flash_decode_num_splits(total_seq) or more.  Replaces the non-graph launch_flash_decode /
 * launch_flash_decode_fp16 (CUDAOps.h:543-549, :641-647). */
int ptm_flash_decode_pos(const float* Q, const void* K_cache, const void* V_cache, float* O, float* partial_O,
                         float* partial_lse, float* partial_max, int n_heads, int n_kv_heads, int head_dim, int total_seq,
                         float scale, int kv_fp16, ptm_stream_t stream);
/* The same over a sliding window (window > 0: only the last `window` positions, gguf_model.h:3490-3500); o_q8, when not
 * NULL, also receives the output as Q8 activation blocks (ptm_q8_bytes(n_heads * head_dim), 16-byte aligned) for a Q4_K
 * output projection. */
int ptm_flash_decode_window(const float* Q, const void* K_cache, const void* V_cache, float* O, void* o_q8,
                            float* partial_O, float* partial_lse, float* partial_max, int n_heads, int n_kv_heads,
                            int head_dim, const int64_t* d_past_len, int max_seq, float scale, int kv_fp16, int window,
                            ptm_stream_t stream);

/* The two operators above fused: one launch does per-head QK-norm + NeoX RoPE of Q and of the new K
 * row, the K/V append at row *d_past_len and the split-KV attention over rows [0, *d_past_len]; a
 * second small launch merges the splits.  Q, K, V are the raw projections and are NOT modified.
 * rope_table: device [max_seq][head_dim] as filled by ptm_rope_table_host (required).
 * Stands in for launch_fused_qknorm_rope_kvwrite_graph + launch_flash_decode(_fp16)_graph
 * (CUDAOps.h:653-673) as forward_decode issues them back to back (gguf_model.h:2785-2832). */
int ptm_attn_decode_fused(const float* Q, const float* K, const float* V, const float* q_norm_w,
                          const float* k_norm_w, void* K_cache, void* V_cache, float* O, float* partial_O,
                          float* partial_lse, float* partial_max, const float* rope_table,
                          int n_heads, int n_kv_heads, int head_dim, const int64_t* d_past_len, int max_seq,
                          float scale, float eps, int add_one, int kv_fp16, int rope_interleaved,
                          ptm_stream_t stream);
/* The same over a sliding window: only the last `window` positions, the new one included, are attended to
 * (window <= 0: all).  The local layers of gemma3 (attn_start, gguf_model.h:3490-3500).  Both entries take head_dim
 * 64, 128 or 256; 256-wide heads run the split-KV kernel of ptm_flash_decode with the norm / rotation / append
 * prologue in front of it. */
int ptm_attn_decode_fused_window(const float* Q, const float* K, const float* V, const float* q_norm_w,
                                 const float* k_norm_w, void* K_cache, void* V_cache, float* O, float* partial_O,
                                 float* partial_lse, float* partial_max, const float* rope_table,
                                 int n_heads, int n_kv_heads, int head_dim, const int64_t* d_past_len, int max_seq,
                                 float scale, float eps, int add_one, int kv_fp16, int rope_interleaved, int window,
                                 ptm_stream_t stream);
/* q_norm_w / k_norm_w may both be NULL (models without QK-norm).  rope_interleaved: 0 rotates the NeoX pairs
 * (d, d + head_dim/2) of qwen / gemma / phi (rope_apply_fused_neox, hot_loops.cpp:2035-2061), 1 the pairs
 * (2d, 2d + 1) of llama / mistral (rope_apply_fused, hot_loops.cpp:1962-2030); config.rope_neox, gguf_model.h:98. */

/* out = silu(gate) * up. launch_silu_mul (CUDAOps.h:416-418). */
int ptm_silu_mul(const float* gate, const float* up, float* out, int64_t n, ptm_stream_t stream);
/* gemma-family glue.  out = gelu_tanh(gate) * up, the expression of the reference's CPU step (gguf_model.h:3730-3738;
 * config.ffn_gelu).  x[r][:] += RMSNorm(h[r][:]) * weight: a branch's post-norm and its residual add
 * (post_attention_norm / post_ffw_norm, gguf_model.h:3656-3680, :3787-3807).  x *= factor: embedding rows times
 * sqrt(hidden) (config.scale_embeddings, gguf_model.h:3252-3265; launch_mul_scalar, CUDAOps.h:67). */
int ptm_gelu_mul(const float* gate, const float* up, float* out, int64_t n, ptm_stream_t stream);
int ptm_rms_norm_add(const float* h, const float* weight, float* x, int rows, int hidden, float eps, int add_one,
                     ptm_stream_t stream);
int ptm_scale(float* x, float factor, int64_t n, ptm_stream_t stream);
/* out[hidden] = emb_table[*d_token_id][:]. launch_embedding_lookup (CUDAOps.h:149-152). */
int ptm_embedding_row(const float* emb_table, float* out, const int* d_token_id, int hidden,
                      ptm_stream_t stream);
/* Same, dequantising row *d_token_id of a Q6_K table (tied lm_head; gguf_model.h:6774 dequantises
 * the whole table at load instead). */
int ptm_embedding_row_q6k(const void* table_q6k, float* out, const int* d_token_id, int hidden,
                          int64_t row_stride_bytes, ptm_stream_t stream);
/* *out = index of the maximum (strict '>', lowest index on ties). launch_argmax (CUDAOps.h:145). */
int ptm_argmax(const float* in, int64_t* out, int64_t n, ptm_stream_t stream);
/* ---- sampling on the device ------------------------------------------------------------------
 * GGUFModel::sample_token (gguf_model.h:7658-7751) with the repetition penalty of generate() (:4926-4938)
 * applied first: penalty once per earlier occurrence (counts[i]; NULL = none), temperature, top-k (ties at the
 * k-th value kept), softmax, top-p, inverse CDF in index order against the uniform draw *d_uniform (device
 * memory; the reference draws it from a static std::mt19937(42) through uniform_real_distribution<float>).
 * temperature < 1e-6: argmax of the penalised logits, no draw.  1 <= top_k <= 1024 (and below the vocabulary) runs on a
 * gathered candidate list with the reference's sums in the reference's order; top-k off (top_k <= 0 or >= vocab) and
 * larger top_k run as passes over the whole vocabulary whose sums are order-independent 64-bit fixed-point ones (they
 * differ from the reference's sequential fp32 sums by rounding, ~1e-7 of the distribution); so does a top_k <= 1024 at
 * whose threshold more than 2048 logits tie (every tie stays, as in the reference; one workgroup then walks the whole
 * vocabulary).  workspace: ptm_sampler_workspace_bytes() device bytes, 8-byte aligned, contents irrelevant.  Replaces the 608 KB logits copy + CPU sampling per token. */
typedef struct ptm_sampling {
    float temperature;
    int32_t top_k;
    float top_p;
    float repeat_penalty;
} ptm_sampling;
int64_t ptm_sampler_workspace_bytes(void);
int ptm_sample_token(const float* logits, int vocab, const int32_t* counts, const ptm_sampling* params,
                     const float* d_uniform, void* workspace, int64_t* out_token, ptm_stream_t stream);
/* n draws of std::uniform_real_distribution<float>(0, 1) over std::mt19937(seed) after skipping `skip` draws:
 * the sequence the reference's sampler consumes (seed 42; one draw per sampled token).  Host memory. */
int ptm_mt19937_uniforms(uint32_t seed, int64_t skip, int64_t n, float* out_host);

/* out = a + b; out = in. launch_add / launch_copy (CUDAOps.h:63, :83). */
int ptm_add(const float* a, const float* b, float* out, int64_t n, ptm_stream_t stream);
int ptm_copy(const float* in, float* out, int64_t n, ptm_stream_t stream);
/* The q / k / v projection biases of a qwen2-style layer: Q[r][:] += q_bias, K[r][:] += k_bias, V[r][:] += v_bias for
 * `rows` rows of q_dim / kv_dim / kv_dim values, in one launch where the reference issues three launch_add calls
 * (gguf_model.h:2768-2779; CPU path :3413-3438): one fp32 add per element, before QK-norm and rotation. */
int ptm_add_qkv_bias(float* Q, float* K, float* V, const float* q_bias, const float* k_bias, const float* v_bias, int rows,
                     int q_dim, int kv_dim, ptm_stream_t stream);

/* ---- unquantised operators the reference's host code calls beside the k-quant kernels ------------------------
 * out = a * factor (launch_mul_scalar, CUDAOps.h:67; in place when out == a). */
int ptm_mul_scalar(const float* a, float factor, float* out, int64_t n, ptm_stream_t stream);
/* fp32 rows [num_new_rows][cols] copied into a cache [.][cols] from row offset_row (launch_kv_cache_write,
 * CUDAOps.h:410-413; KVCache::append, gguf_model.h:520-525). */
int ptm_kv_cache_write(const float* src, float* dst_cache, int64_t num_new_rows, int64_t cols, int64_t offset_row,
                       ptm_stream_t stream);
/* out[a_rows + b_rows][cols] = rows of a, then rows of b (launch_concat, CUDAOps.h:404-407). */
int ptm_concat_rows(const float* a, const float* b, float* out, int64_t a_rows, int64_t b_rows, int64_t cols,
                    ptm_stream_t stream);
/* In-place rotation of data[seq_len][n_heads * head_dim], row s at position position_offset + s (launch_rope,
 * CUDAOps.h:392-395; CUDAInference.cu:149-189 rotates the interleaved pairs (2d, 2d + 1): neox = 0; neox != 0 rotates
 * (d, d + head_dim / 2) as the reference's CPU path does for qwen / gemma / phi).  rope_table (device, table_rows rows as
 * ptm_rope_table_host fills them) gives the host-libm angles; NULL computes them on the device from rope_freq_base. */
int ptm_rope(float* data, int seq_len, int n_heads, int head_dim, int position_offset, float rope_freq_base,
             const float* rope_table, int table_rows, int neox, ptm_stream_t stream);
/* y[N] = W . x for unquantised weights.  fp32: k_major = 0 is W[N][K] row-major (launch_gemv, CUDAOps.h:188-192),
 * k_major != 0 is W[K][N] (launch_inference_gemv, CUDAOps.h:422-424).  fp16: k_major = 0 is W[N][K] row-major
 * (launch_fp16_gemv, CUDAOps.h:493-495; launch_cublas_hgemv with row_major), k_major != 0 the [K][N] order that
 * ptm_dequant_q4k_to_fp16 writes (launch_cublas_hgemv's default, CUDAOps.h:484-489); round_x != 0 rounds x to fp16 first,
 * as launch_cublas_hgemv does.  fp32 accumulation.  Plain kernels, not tuned: no Q4_K_M model takes these paths. */
int ptm_f32_gemv(const float* W, const float* x, float* y, int K, int N, int k_major, ptm_stream_t stream);
int ptm_f16_gemv(const void* W_fp16, const float* x, float* y, int K, int N, int k_major, int round_x, ptm_stream_t stream);

/* ---- prefill: quantised-weight GEMM, Y[M,N] = X[M,K] . W[N,K]^T ------------------ */
/* The reference has no quantised GEMM: matmul_q loops M single-row GEMVs
 * (gguf_model.h:7029-7036, :7056-7061).  These read each weight tile once per 64 rows of X and
 * use MFMA.  X is bf16 row-major [M][K] (16-byte aligned); Y fp32 row-major [M][N]; K % 256 == 0.
 * Q4_K: rows of X are quantised to Q8 blocks (same rule as ptm_quantize_q8, applied to the
 * bf16->fp32 values); int8 MFMA (K = 32 = one sub-block) gives the exact integer dots, scaled and
 * accumulated in the GEMV's order, so every row equals ptm_q4k_gemv of that row bit for bit.
 * Q6_K: (q - 32) as bf16 times bf16 X on bf16 MFMA (K = 16 = one scale group; products exact),
 * each group sum scaled by d * scale in fp32.  Rows agree with ptm_q6k_gemv to fp32 rounding.
 * workspace: ptm_qgemm_workspace_bytes(M, K) device bytes, 16-byte aligned (Q4_K only; Q6_K
 * ignores it and accepts NULL). */
int64_t ptm_qgemm_workspace_bytes(int M, int K);
int ptm_qgemm_q4k(const void* W, const void* X_bf16, float* Y, int M, int K, int N,
                  int64_t row_stride_bytes, void* workspace, ptm_stream_t stream);
int ptm_qgemm_q6k(const void* W, const void* X_bf16, float* Y, int M, int K, int N,
                  int64_t row_stride_bytes, void* workspace, ptm_stream_t stream);
/* Fast variant of the same product (Q4_K or Q6_K by ggml type id): rows of X are rounded to the
 * reference's Q8 values (d*q per block of 32) and stored as fp16, weights are dequantised in
 * registers and rounded to fp16, v_mfma_f32_32x32x16_f16 accumulates in fp32 over all of K.  Rows
 * equal the reference GEMV up to the fp16 rounding of the operands (~1e-3 of rms(y) at most),
 * inside the 1e-2 bar of the prefill path; use ptm_qgemm_q4k for bit-identical rows.
 * workspace: ptm_qgemm_f16_workspace_bytes(M, K) device bytes, 16-byte aligned. */
int64_t ptm_qgemm_f16_workspace_bytes(int M, int K);
int ptm_qgemm_f16(uint32_t ggml_type, const void* W, const void* X_bf16, float* Y, int M, int K, int N,
                  int64_t row_stride_bytes, void* workspace, ptm_stream_t stream);
/* The same with fp32 rows of X (what the reference's prefill holds) and an optional Y += result.  When N gives
 * too few column tiles to fill the chip, K is split over several workgroups whose partial sums (held in the
 * workspace) are added in a fixed order, so results are reproducible; the split depends on N, K and the class of M (<= 128,
 * <= 256, more).
 * workspace: ptm_qgemm_f16_f32_workspace_bytes(M, K, N) bytes, 16-byte aligned. */
int64_t ptm_qgemm_f16_f32_workspace_bytes(int M, int K, int N);
int ptm_qgemm_f16_f32(uint32_t ggml_type, const void* W, const float* X_f32, float* Y, int M, int K, int N,
                      int64_t row_stride_bytes, void* workspace, int accumulate, ptm_stream_t stream);

/* ---- prefill glue: the decode-step pieces batched over prompt rows ----------------------- */
/* out[r][:] = embedding of d_tokens[r] from an fp32 table [vocab][hidden], or (table_f32 NULL) from Q6_K rows
 * dequantised on the fly.  embedding_lookup, gguf_model.h:2513. */
int ptm_embedding_rows(const float* table_f32, const void* table_q6k, int64_t q6k_row_stride_bytes, const int* d_tokens,
                       int rows, int hidden, int vocab, float* out, ptm_stream_t stream);
/* Row r (position pos0 + r): per-head RMSNorm (norm weights may both be NULL) + NeoX RoPE in place on
 * Q [rows][n_heads*head_dim] and K [rows][kv_dim], K and V rows appended to the caches.  The row-batched form of
 * ptm_qknorm_rope_kvwrite (launch_fused_qknorm_rope_kvwrite, CUDAOps.h:563-570). */
int ptm_qknorm_rope_kvwrite_rows(float* Q, float* K, const float* V, const float* q_norm_w, const float* k_norm_w,
                                 void* K_cache, void* V_cache, const float* rope_table, int rows, int n_heads,
                                 int n_kv_heads, int head_dim, int64_t pos0, int max_seq, float eps, int add_one,
                                 int kv_fp16, int rope_interleaved, ptm_stream_t stream);
/* Causal GQA attention of prompt row r over cache positions [0, pos0 + r] (the rows' own K/V already appended);
 * O [rows][n_heads*head_dim].  launch_causal_attention (gguf_model.h:7400; CUDAInference.cu:202-315). */
int ptm_prefill_attention(const float* Q, const void* K_cache, const void* V_cache, float* O, int rows, int n_heads,
                          int n_kv_heads, int head_dim, int64_t pos0, int max_seq, float scale, int kv_fp16,
                          ptm_stream_t stream);
/* The same over a sliding window: row r sees positions (pos0 + r - window, pos0 + r] only (window <= 0: everything).
 * The local layers of gemma3 (attn_start, gguf_model.h:3490-3500); windowed calls run on the fp32 kernel. */
int ptm_prefill_attention_window(const float* Q, const void* K_cache, const void* V_cache, float* O, int rows, int n_heads,
                                 int n_kv_heads, int head_dim, int64_t pos0, int max_seq, float scale, int kv_fp16,
                                 int window, ptm_stream_t stream);

/* ---- batch-1 decode runtime (GGUFModel::forward_decode, gguf_model.h:2575-3113) --- */
typedef struct {
    const void* data;         /* device, raw super-blocks */
    uint32_t ggml_type;       /* PTM_TYPE_Q4_K / Q6_K (fused kernels) or Q5_K / Q8_0 / Q5_0 (plain kernels; prompts of a
                               * decoder holding any of these are stepped token by token) */
    int32_t rows, cols;       /* N, K */
    int64_t row_stride_bytes;
} ptm_qweight; /* the device half of QuantizedWeight, gguf_model.h:336-385 */

typedef struct {
    ptm_qweight q, k, v, o, gate, up, down;
    const float *attn_norm, *ffn_norm, *q_norm, *k_norm; /* device fp32; q_norm and k_norm both NULL: no QK-norm */
    void *k_cache, *v_cache; /* device [max_seq][kv_dim], fp16 or fp32 per kv_fp16 */
    const float *q_bias, *k_bias, *v_bias; /* device fp32 [q_dim], [kv_dim], [kv_dim] (qwen2; LayerWeights::attn_*_bias,
                                            * gguf_model.h:410-412); all three or all NULL */
    const float *post_attn_norm, *post_ffn_norm; /* device fp32 [hidden] (gemma2 / gemma3: RMSNorm of the attention / the
                                                  * feed-forward branch's output before the residual add); each may be NULL */
} ptm_layer;

typedef struct {
    int32_t vocab, hidden, n_layers, n_heads, n_kv_heads, head_dim, inter, max_seq;
    float rope_freq_base, rms_eps;
    int32_t kv_fp16;              /* 1: fp16 KV cache, 0: fp32 (as the reference's decode) */
    int32_t use_graph;            /* 1: capture the token step in a hipGraph and replay it */
    const float* embedding_f32;   /* device [vocab][hidden] fp32, or NULL to use lm_head rows (Q6_K, tied) */
    const ptm_layer* layers;      /* HOST array of n_layers descriptors (copied) */
    const float* out_norm;        /* device */
    ptm_qweight lm_head;
    int32_t rope_interleaved;     /* 0: NeoX rotation pairs (qwen3); 1: pairs (2d, 2d+1) (llama, mistral) */
    float rope_scale;             /* linear position scaling, theta = (pos / rope_scale) * freq (gguf_model.h:71); 0 or 1: none */
    /* gemma family (ModelConfig, gguf_model.h:74-88): embedding rows times sqrt(hidden); tanh-GELU instead of SiLU on the
     * gate; layers li with (li + 1) % swa_pattern != 0 attend to the last swa_window positions only and rotate with
     * rope_swa_freq_base without position scaling (swa_window or swa_pattern 0: no local layers) */
    int32_t scale_embeddings, ffn_gelu, swa_window, swa_pattern;
    float rope_swa_freq_base;
    /* phi3 LongRoPE (ModelConfig::rope_factors_short / _long / rope_orig_ctx / rope_attn_factor, gguf_model.h:89-96): HOST
     * arrays of head_dim / 2 per-frequency factors (copied at create; NULL: none), the context length up to which the short
     * set applies (0: no factors), and the factor cos / sin are scaled by (0 or 1: none); see ptm_rope_table_host_factors */
    const float *rope_factors_short, *rope_factors_long;
    int32_t rope_orig_ctx;
    float rope_attn_factor;
} ptm_decode_config;

typedef struct ptm_decoder ptm_decoder;

/* Allocates the decode scratch, the RoPE table, the decode stream and device scalars once: no decode step allocates
 * afterwards.  The row scratch of prompt prefill is separate: ptm_decode_reserve_prefill allocates it up front, otherwise
 * the first ptm_decode_prefill (or one with more rows per chunk than any before) does.  The KV caches and weights stay
 * caller-owned.  Each matrix is read with its own row_stride_bytes (at least a dense row, 16-byte multiples for Q4_K, even for
 * Q6_K; the Q4_K matrices among q / k / v share one stride), PTM_E_SHAPE otherwise. */
int ptm_decode_create(const ptm_decode_config* cfg, ptm_decoder** out);
/* Allocate the prefill row scratch for chunks of up to `rows` prompt rows (capped at 2048) now, so that no later
 * ptm_decode_prefill with chunk_rows <= rows allocates. */
int ptm_decode_reserve_prefill(ptm_decoder* d, int rows);
void ptm_decode_destroy(ptm_decoder* d);
/* Set the number of positions already present in the KV caches (after prefill). */
int ptm_decode_set_past_len(ptm_decoder* d, int64_t past_len);
/* One greedy step: feeds token_id at position past_len, returns the argmax token through
 * *next_token (host), advances past_len.  Synchronous like forward_decode + GPU argmax
 * (gguf_model.h:3107, :4850-4859).  The token id reaches the host through pinned memory the step's last kernel
 * writes (no copy launch); when token_id is the token the previous greedy call returned (a generate loop), the step
 * starts from the token, position and step index the device already holds. */
int ptm_decode_step(ptm_decoder* d, int token_id, int64_t* next_token);
/* One greedy step run as plain launches that also copies out the residual stream after every layer's attention branch and
 * after its feed-forward branch: trace_device[n_layers][2][hidden] fp32 (device).  The hook the reference has as
 * PT_DUMP_HIDDEN (gguf_model.h:3268-3289): for comparing a run layer by layer, not for serving. */
int ptm_decode_step_trace(ptm_decoder* d, int token_id, int64_t* next_token, float* trace_device);
/* n greedy steps feeding each output back in, without host round trips between tokens:
 * tokens_out[n] (host). */
/* Prefill: run n prompt tokens (host array) through the model at once, append their K/V rows at positions
 * past_len .. past_len + n - 1 and return the greedy token that follows the prompt; logits of the last
 * prompt token are left for ptm_decode_logits.  Rows go through the layers in chunks of chunk_rows
 * (<= 0 or above 2048: 2048) with the fast quantised GEMM, row-batched QK-norm + RoPE + KV append and causal attention.
 * The counterpart of GGUFModel::forward(tokens, use_cache = true) (gguf_model.h:2510-2571); row m equals
 * a decode step of token m up to the fp16 rounding of the GEMM operands.  Allocates its row scratch on first use unless
 * ptm_decode_reserve_prefill has reserved enough rows. */
int ptm_decode_prefill(ptm_decoder* d, const int32_t* tokens, int n, int chunk_rows, int64_t* next_token);
/* Sampled generation (the decode loop of promeserve/api_handlers.h:848-923 with the sampling kept on the GPU).
 * ptm_decode_sampling_begin starts a generation: stores the parameters and forgets the tokens generated so far
 * (the repetition penalty only sees tokens generated since).  ptm_decode_sample then runs n chained steps from
 * `token`, drawing with uniforms_host[0..n) (ptm_mt19937_uniforms gives the reference's sequence); ids land in
 * out_tokens.  Stop tokens are the caller's business: generate in short runs and cut at the first one. */
int ptm_decode_sampling_begin(ptm_decoder* d, const ptm_sampling* params);
int ptm_decode_sample(ptm_decoder* d, int token_id, int n, const float* uniforms_host, int64_t* out_tokens);
/* The whole serving loop of api_handlers.h:848-923 in one call: the prompt (all but its last token through
 * ptm_decode_prefill), then sample / stop check / feed back for up to max_new tokens; a stop token ends the output and
 * is not part of it.  out_tokens must hold max_new ids; uniforms_host max_new draws.  On return past_len counts the
 * prompt and every generated token that was fed back (the last generated token is not fed yet). */
int ptm_decode_generate(ptm_decoder* d, const int32_t* prompt, int n_prompt, const ptm_sampling* params,
                        const float* uniforms_host, int max_new, const int32_t* stop_ids, int n_stop,
                        int64_t* out_tokens, int* n_out);
int ptm_decode_greedy(ptm_decoder* d, int first_token, int n, int64_t* tokens_out);
/* How the greedy (sampled = 0) or the sampled (1) token step runs: 0 plain launches so far (use_graph = 0, or no second
 * step yet), 1 replaying its captured hipGraph, 2 plain launches because capturing or instantiating the graph failed
 * once - not an error: the reference likewise falls back to eager launches (gguf_model.h:2660-2665, :3093-3104). */
int ptm_decode_graph_state(const ptm_decoder* d, int sampled);
/* Test seam for that fallback: the decoder's next capture attempt reports failure on the host before anything is recorded
 * (no GPU error is provoked), so the steps that follow run as plain launches and ptm_decode_graph_state returns 2.  The
 * reference has no such switch; its fallback (gguf_model.h:2660-2665) is reached only by a real capture failure. */
int ptm_decode_debug_fail_next_capture(ptm_decoder* d);
/* Device pointers to the last step's logits [vocab] and final-normed hidden [hidden]. */
const float* ptm_decode_logits(ptm_decoder* d);
const float* ptm_decode_hidden(ptm_decoder* d);
void* ptm_decode_stream(ptm_decoder* d);

/* ---- GGUF files: container reader and model loader --------------------------------------- */
/* Reader for GGUF v2/v3 (the reference's GGUFReader, torch/io/gguf_loader.h:386-630): the file is
 * memory-mapped; tensor data pointers are HOST pointers into the mapping, valid until close.
 * dims[0] is the contiguous dimension (K), dims[1] the rows (N); nbytes is -1 for a ggml type this
 * library does not size (anything but F32, F16, Q4_K, Q6_K). */
typedef struct ptm_gguf ptm_gguf;
typedef struct {
    const char* name;
    uint32_t ggml_type;
    int32_t n_dims;
    int64_t dims[4];
    int64_t nbytes;
    const void* data;
} ptm_gguf_tensor;
int ptm_gguf_open(const char* path, ptm_gguf** out);
void ptm_gguf_close(ptm_gguf* g);
int ptm_gguf_version(const ptm_gguf* g);
int64_t ptm_gguf_alignment(const ptm_gguf* g);
int64_t ptm_gguf_n_tensors(const ptm_gguf* g);
int ptm_gguf_tensor_at(const ptm_gguf* g, int64_t i, ptm_gguf_tensor* out);
int ptm_gguf_find_tensor(const ptm_gguf* g, const char* name, ptm_gguf_tensor* out);
/* Metadata: integers and bools widened to int64, floats to double (an integer key also reads as
 * float); strings by pointer (NULL if absent or not a string); arrays are not exposed. */
int ptm_gguf_get_int(const ptm_gguf* g, const char* key, int64_t* out);
int ptm_gguf_get_float(const ptm_gguf* g, const char* key, double* out);
const char* ptm_gguf_get_string(const ptm_gguf* g, const char* key);
/* Array-valued metadata: element type (GGUF code: 0 u8, 1 i8, 2 u16, 3 i16, 4 u32, 5 i32, 6 f32, 7 bool, 8 string,
 * 10 u64, 11 i64, 12 f64) and count; element i of a string array as (pointer into the mapping, length), not
 * NUL-terminated; the packed little-endian elements of a numeric array.  GGUFValue::as_array (gguf_loader.h:69-89). */
int ptm_gguf_get_array(const ptm_gguf* g, const char* key, uint32_t* elem_type, int64_t* count);
int ptm_gguf_array_string(const ptm_gguf* g, const char* key, int64_t i, const char** data, int64_t* len);
const void* ptm_gguf_array_data(const ptm_gguf* g, const char* key);

/* From a .gguf file to a ready decoder: reads the `qwen3`, `qwen2` (no QK-norm tensors; blk.N.attn_{q,k,v}.bias
 * vectors where the file has them, gguf_model.h:6750-6754), `gemma3` (sliding-window keys, post-norm vectors, scaled
 * embeddings and GELU gate: gguf_model.h:157-197) or `llama` (no QK-norm tensors, interleaved rotation
 * pairs: gguf_model.h:202-217) hyper-parameters
 * (<arch>.block_count, embedding_length, feed_forward_length, attention.head_count(_kv),
 * attention.key_length, rope.freq_base, attention.layer_norm_rms_epsilon; gguf_model.h:126-181),
 * uploads every blk.N.{attn_q,attn_k,attn_v,attn_output,ffn_gate,ffn_up,ffn_down}.weight and
 * output.weight (or the tied token_embd.weight) verbatim (gguf_model.h:1177-1360), norm vectors as
 * fp32, allocates zeroed KV caches for max_seq positions and creates the decode runtime.
 * Matrices may be of any type the GEMV dispatcher takes (Q4_K, Q6_K: the tuned path; Q5_K, Q8_0, Q5_0: plain
 * kernels); other architectures and other types: PTM_E_UNSUPPORTED. */
typedef struct ptm_model ptm_model;
int ptm_model_load_gguf(const char* path, int max_seq, int kv_fp16, int use_graph, ptm_model** out);
ptm_decoder* ptm_model_decoder(ptm_model* m); /* owned by the model */
int ptm_model_config(const ptm_model* m, ptm_decode_config* out);
int ptm_model_layer(const ptm_model* m, int i, ptm_layer* out);
void ptm_model_free(ptm_model* m);

/* ---- tokenizer and chat template (host only) ----------------------------------------------------
 * GGUFTokenizer (torch/io/tokenizer.h:24-643): byte-level BPE ("gpt2": Qwen, Llama-3) or word-marker BPE /
 * greedy longest match (any other tokenizer.ggml.model), special tokens matched first, <0xNN> byte fallback.
 * Same ids and same decoded bytes as the reference.  One difference: on a UTF-8 continuation byte that does not
 * follow a letter the reference's "gpt2" splitter never returns; here the byte becomes a word of its own.
 * Buffers are the caller's: a result that does not fit returns PTM_E_RANGE with the needed size in *n_ids / *len. */
typedef struct ptm_tokenizer ptm_tokenizer;
int ptm_tokenizer_create(const char* const* tokens, const int32_t* token_lens, int32_t n_tokens, const char* const* merges,
                         const int32_t* merge_lens, int32_t n_merges, const char* model_type, int32_t bos_id,
                         int32_t eos_id, int32_t pad_id, int32_t unk_id, int add_bos, ptm_tokenizer** out);
/* GGUFTokenizer::load (tokenizer.h:42-121): tokenizer.ggml.{model,tokens,merges,*_token_id,add_bos_token}. */
int ptm_tokenizer_from_gguf(const ptm_gguf* g, ptm_tokenizer** out);
void ptm_tokenizer_free(ptm_tokenizer* t);
int32_t ptm_tokenizer_vocab_size(const ptm_tokenizer* t);
int ptm_tokenizer_special_ids(const ptm_tokenizer* t, int32_t* bos, int32_t* eos, int32_t* pad, int32_t* unk);
/* encode (tokenizer.h:127-155), decode (:161-175), decode_token (:177-182). */
int ptm_tokenizer_encode(const ptm_tokenizer* t, const char* text, int64_t text_len, int use_bos, int32_t* ids,
                         int64_t cap, int64_t* n_ids);
int ptm_tokenizer_decode(const ptm_tokenizer* t, const int32_t* ids, int64_t n_ids, int skip_special, char* out,
                         int64_t cap, int64_t* len);
int ptm_tokenizer_token(const ptm_tokenizer* t, int32_t id, char* out, int64_t cap, int64_t* len);
/* GGUFModel::apply_chat_template (gguf_model.h:4178-4236): ChatML for qwen2/qwen3 (no_think adds "/no_think" to the
 * system turn of qwen3), Phi-3, Gemma, Llama-3, Mistral (architecture "llama" with "mistral" in the model name), the
 * bare prompt otherwise.  system: NULL = "You are a helpful assistant.", "" = no system turn (the reference reads
 * PT_SYSTEM_PROMPT / PT_NO_THINK from the environment instead). */
int ptm_chat_template(const char* architecture, const char* model_name, const char* system, int no_think,
                      const char* prompt, char* out, int64_t cap, int64_t* len);

#ifdef __cplusplus
}
#endif
#endif /* PTM_H */
