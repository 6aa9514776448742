/* TEST INFRASTRUCTURE ONLY.
 *
 * CPU restatement of the reference's GGUF k-quant decode path (PromeTorch
 * torch/io/gguf_dequant.h, torch/io/cpu_quant_gemv.h, torch/io/gguf_model.h
 * forward_decode_cpu, aten/src/ATen/native/cpu/hot_loops.cpp RoPE,
 * aten/src/ATen/native/cpu/VectorizedOps.h exp256_ps).  It is the checker the
 * GPU kernels are compared against and the timed "port" CPU baseline; it is
 * never linked into, loaded by, or called from the shipped library.
 *
 * Pinning status (what fixes each function independently of this file):
 *   po_fp16_to_fp32        all 65536 inputs vs numpy float16->float32, and vs the compiled reference
 *   po_get_scale_min_k4    exhaustive 6-bit pack/unpack round trip + compiled reference
 *   po_dequantize_q4_k/q6_k golden blocks from the compiled reference (bit-exact) + closed form in numpy
 *   po_quantize_x_q8       golden vectors from the compiled reference (bit-exact) + numpy rint invariants
 *   po_q4k_gemv            golden y from the compiled reference (bit-exact) + exact int dots vs numpy
 *   po_q6k_gemv            golden y from the compiled reference (bit-exact) + float64 dot of dequant
 *   po_q8_0_gemv, po_q5k_gemv, po_q5_0_gemv, po_dequantize_q8_0, po_dequantize_q5_k
 *                          golden y / values from the compiled reference's dispatcher and dequantisers
 *                          (golden_formats.npz, bit-exact) + closed-form numpy dequantisation and its float64 dot
 *   po_rmsnorm_*           compiled reference + float64 numpy
 *   po_rope_*              compiled reference + float64 closed form (NeoX and interleaved pairing)
 *   po_exp256              compiled reference + float64 exp
 *   po_attn_head, po_silu_mul, po_argmax, po_decode_step
 *                          golden logits / token ids of the compiled reference's
 *                          forward_decode_cpu on a tiny and the full-size model
 *   po_decode_step's model switches (no QK-norm, interleaved pairs, position scaling, q / k / v biases, scaled
 *                          embeddings, GELU gate via po_gelu_mul, post-norms, sliding windows via
 *                          po_attn_head_window with per-layer rotation bases): golden logits of the compiled
 *                          reference on one tiny model per switch family (golden_llama / qwen2 / gemma .npz, each
 *                          switch shown to move the logits) and on ten models with all switches drawn at random
 *                          (golden_random_arch.npz), bit-exact; po_gelu_mul also against float64
 *   po_mt19937_*, po_uniform01   the 10000th output of the default-seeded generator (4123659995, ISO C++
 *                          [rand.predef]) + the tokens the compiled reference's sample_token draws with its
 *                          mt19937(42) (golden_sampling.npz)
 *   po_sample_token        golden tokens of the compiled reference's sample_token over seeded logits and
 *                          parameter sets + numpy float64 restatement (top-k by partition, softmax,
 *                          nucleus cut, inverse CDF)
 *   (tokenizer, chat template: no restatement here; the library's host code is compared directly with
 *                          the compiled reference's outputs in tests/golden/golden_tokenizer.json)
 *   po_repetition_penalty  numpy restatement with repeated ids (the reference applies the penalty once per
 *                          occurrence); the reference holds it inline in generate(), so no compiled check
 */
#ifndef PTM_ORACLE_H
#define PTM_ORACLE_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { PO_Q5_0 = 6, PO_Q8_0 = 8, PO_Q4_K = 12, PO_Q5_K = 13, PO_Q6_K = 14 };

float po_fp16_to_fp32(uint16_t h);
uint16_t po_fp32_to_fp16(float f); /* round-to-nearest-even, IEEE */
void po_get_scale_min_k4(int j, const uint8_t* q, uint8_t* sc, uint8_t* m);
void po_dequantize_q4_k(const void* src, float* dst, int64_t n);
void po_dequantize_q6_k(const void* src, float* dst, int64_t n);
void po_dequantize_q8_0(const void* src, float* dst, int64_t n);   /* gguf_dequant.h:237 */
void po_dequantize_q5_k(const void* src, float* dst, int64_t n);   /* gguf_dequant.h:348 */
void po_q8_0_gemv(const void* W, const float* x, float* y, int64_t K, int64_t N, int64_t stride); /* cpu_quant_gemv.h:784 */
void po_q5k_gemv(const void* W, const float* x, float* y, int64_t K, int64_t N, int64_t stride);  /* cpu_quant_gemv.h:1091 */
void po_q5_0_gemv(const void* W, const float* x, float* y, int64_t K, int64_t N, int64_t stride); /* cpu_quant_gemv.h:1572 */

/* Q8 activation blocks, flat: d[K/32], sum[K/32], qs[K] */
void po_quantize_x_q8(const float* x, int64_t K, float* d, float* sum, int8_t* qs);

void po_q4k_gemv(const void* W, const float* x, float* y, int64_t K, int64_t N, int64_t stride);
void po_q4k_gemv_f32(const void* W, const float* x, float* y, int64_t K, int64_t N, int64_t stride);
void po_q6k_gemv(const void* W, const float* x, float* y, int64_t K, int64_t N, int64_t stride);
void po_q6k_gemv_f32(const void* W, const float* x, float* y, int64_t K, int64_t N, int64_t stride);
/* dispatcher: type 12 -> po_q4k_gemv, 14 -> po_q6k_gemv, anything else: silent no-op */
void po_cpu_quant_gemv(uint32_t type, const void* W, const float* x, float* y,
                       int64_t K, int64_t N, int64_t stride);
/* Integer sub-block dots of one Q4_K row against Q8 x: isum[K/32] (exact int32). */
void po_q4k_row_isums(const void* row, const int8_t* qs, int64_t K, int32_t* isum);

void po_rmsnorm_seq(const float* x, const float* gamma, float eps, int add_one, int64_t H, float* out);
void po_rmsnorm_vec(const float* x, const float* gamma, float eps, int add_one, int64_t H, float* out);
void po_rope_precompute(float* c, float* s, int64_t pos, int64_t head_dim, float base);
void po_rope_precompute_scaled(float* c, float* s, int64_t pos, int64_t head_dim, float base, float scale);
void po_rope_precompute_factors(float* c, float* s, int64_t pos, int64_t head_dim, float base, float scale,
                                const float* factors, float attn_factor);
void po_rope_apply_norm(float* q, float* k, const float* c, const float* s, int64_t n_heads, int64_t n_kv_heads,
                        int64_t head_dim);
void po_rope_apply_neox(float* q, float* k, const float* c, const float* s,
                        int64_t n_heads, int64_t n_kv_heads, int64_t head_dim);
void po_exp256(const float* in, float* out, int64_t n8);
/* one query head against T cached positions; k,v point at this kv-head's column
 * block of row 0, row pitch kv_dim floats; scores is scratch[T] */
void po_attn_head(const float* q, const float* k, const float* v, int64_t T, int64_t kv_dim,
                  int64_t head_dim, float scale, float* scores, float* out);
void po_attn_head_window(const float* q, const float* k, const float* v, int64_t T, int64_t t_start, int64_t kv_dim,
                         int64_t head_dim, float scale, float* scores, float* out);
void po_silu_mul(float* gate, const float* up, int64_t n);
void po_gelu_mul(float* gate, const float* up, int64_t n);
int64_t po_argmax(const float* x, int64_t n);

typedef struct {
    const void* data; uint32_t type; int64_t rows, cols, stride;
} po_qweight;

typedef struct {
    po_qweight q, k, v, o, gate, up, down;
    const float *attn_norm, *ffn_norm, *q_norm, *k_norm; /* q_norm, k_norm: NULL for models without QK-norm */
    float *k_cache, *v_cache; /* [max_seq][kv_dim] fp32 storage */
    const float *q_bias, *k_bias, *v_bias; /* added to the projections' outputs (qwen2); all three or all NULL */
    const float *post_attn_norm, *post_ffn_norm; /* gemma2 / gemma3: RMSNorm of a branch's output before the residual add */
} po_layer;

typedef struct {
    int64_t vocab, hidden, n_layers, n_heads, n_kv_heads, head_dim, inter, max_seq;
    float rope_base, eps;
    int kv_fp16;            /* 1: round appended K/V rows to fp16 (what an fp16 cache stores) */
    const float* embedding; /* fp32 [vocab][hidden], or NULL to dequantize rows of lm_head (Q6_K, tied) */
    po_layer* layers;
    const float* out_norm;
    po_qweight lm_head;
    int64_t seq_len;
    int rope_interleaved;   /* 0: NeoX pairs (d, d + half) as qwen / gemma / phi; 1: pairs (2d, 2d + 1) as llama / mistral */
    float rope_scale;       /* linear position scaling (ModelConfig::rope_scale, gguf_model.h:71); 0 or 1: none */
    /* gemma family (gguf_model.h:74-88, :184-197): embedding rows times sqrt(hidden); tanh-GELU instead of SiLU in the
     * feed-forward gate; layers li with (li + 1) % swa_pattern != 0 attend to the last swa_window positions only and
     * rotate with rope_swa_base and no position scaling (swa_window or swa_pattern 0: every layer is global) */
    int scale_embeddings, ffn_gelu;
    int64_t swa_window, swa_pattern;
    float rope_swa_base;
    /* phi3 LongRoPE (ModelConfig, gguf_model.h:89-96, :285-296): per-frequency factors [head_dim / 2], the short set while
     * past + 1 <= rope_orig_ctx and the long set beyond (rope_orig_ctx 0: none; a NULL set: none for its range), and the
     * factor cos and sin are multiplied with (0 or 1: none) */
    const float *rope_factors_short, *rope_factors_long;
    int64_t rope_orig_ctx;
    float rope_attn_factor;
} po_model;

/* One decode step (forward_decode_cpu order, Q4_K_M fallbacks); writes logits[vocab],
 * advances seq_len, returns greedy argmax. hidden_out (optional) gets the final-normed hidden. */
int64_t po_decode_step(po_model* m, int64_t token, float* logits, float* hidden_out);
/* The same, also writing the residual stream after every layer's attention branch and after its feed-forward branch:
 * trace[n_layers][2][hidden] (may be NULL). */
int64_t po_decode_step_trace(po_model* m, int64_t token, float* logits, float* hidden_out, float* trace);
int po_num_threads(void);

/* ---- sampling (reference: GGUFModel::sample_token, gguf_model.h:7658-7751; penalty loop :4926-4938) ---- */
typedef struct { uint32_t mt[624]; int idx; } po_mt19937;
void po_mt19937_seed(po_mt19937* g, uint32_t seed);
uint32_t po_mt19937_next(po_mt19937* g);
/* std::uniform_real_distribution<float>(0, 1)(std::mt19937) as libstdc++ evaluates it */
float po_uniform01(po_mt19937* g);
void po_repetition_penalty(float* logits, int64_t vocab, const int32_t* generated, int64_t n, float penalty);
/* r is the uniform draw.  probs_out (optional, [vocab]) receives the final distribution; gap_out (optional)
 * the distance from r to the nearest edge of the chosen token's CDF interval (how robust the choice is). */
int32_t po_sample_token(const float* logits, int64_t vocab, float temperature, int top_k, float top_p, float r,
                        float* probs_out, float* gap_out);

#ifdef __cplusplus
}
#endif
#endif
