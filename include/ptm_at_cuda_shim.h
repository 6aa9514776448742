/*
 * ptm_at_cuda_shim.h — the reference's operator names on top of the ptm C ABI.
 *
 * PromeTorch's host code (torch/io/gguf_model.h: forward_decode, forward, gemv_scratch, matmul_q, KVCache)
 * calls free functions `at::cuda::launch_*` declared in aten/src/ATen/cuda/CUDAOps.h.  Including
 * this header instead (on a ROCm build) gives the same names, argument order and default stream
 * argument as inline forwards to libptm_hip.so, so that host code compiles unchanged for the
 * hot path.  Each forward cites the CUDAOps.h declaration it stands in for.  The reference's
 * launchers return void and check nothing; these keep that contract and drop the status code
 * (call the ptm_* function directly to see it).
 *
 * Two facts the reference's signatures do not carry are set once per thread with
 * at::cuda::ptm_shim_set_context(max_seq, rope_neox[, rope_table]) before the first decode step:
 *   max_seq    height of the KV caches handed to launch_fused_qknorm_rope_kvwrite_graph (its signature has no
 *              bound; the kernels here never write past it);
 *   rope_neox  1: rotation pairs (d, d + head_dim/2) as the reference's CPU path applies for qwen / gemma / phi
 *              (config.rope_neox, gguf_model.h:98, :3464-3470); 0: pairs (2d, 2d + 1), which is what the reference's
 *              CUDA kernels always rotate (FlashDecoding.cu:309-312, CUDAInference.cu:149-175);
 *   rope_table optional device table [max_seq][head_dim] from ptm_rope_table_host (host-libm angles, bit-identical
 *              to the CPU path); NULL computes the angles on the device.
 * Not provided on purpose: launch_quantize_q8_1 and launch_q4km_q8_gemv (CUDAOps.h:462-470).  Their contract is a
 * caller-sized buffer of (K/32)*36 bytes of {half d, half s, int8 qs[32]} blocks; this library's Q8 blocks follow
 * the CPU path ({int8 qs[K], float d[K/32], float sum[K/32]}: K + K/4 bytes), which would overrun such a buffer.
 * No host code of the reference calls them; use ptm_quantize_q8 / ptm_q4k_gemv_q8 with ptm_q8_bytes(K).
 */
#ifndef PTM_AT_CUDA_SHIM_H
#define PTM_AT_CUDA_SHIM_H

#include <hip/hip_runtime_api.h>
#include <stdint.h>

#include "ptm.h"

typedef hipStream_t cudaStream_t; /* the reference spells the stream type the CUDA way */

namespace at {
namespace cuda {

struct PtmShimContext {
    int max_seq = 4096;   /* PromeServe's fixed KV height, promeserve/api_handlers.h:769 */
    int rope_neox = 1;
    const float* rope_table = nullptr;
};
inline PtmShimContext& ptm_shim_context() {
    static thread_local PtmShimContext ctx;
    return ctx;
}
inline void ptm_shim_set_context(int max_seq, int rope_neox, const float* rope_table = nullptr) {
    PtmShimContext& c = ptm_shim_context();
    c.max_seq = max_seq;
    c.rope_neox = rope_neox;
    c.rope_table = rope_table;
}

/* CUDAOps.h:427-448 */
inline void launch_q4km_gemv(const void* w, const float* x, float* y, int K, int N, int64_t stride, cudaStream_t s = nullptr) { (void)ptm_q4k_gemv(w, x, y, K, N, stride, 0, s); }
inline void launch_q4km_persistent_gemv(const void* w, const float* x, float* y, int K, int N, int64_t stride, cudaStream_t s = nullptr) { (void)ptm_q4k_gemv(w, x, y, K, N, stride, 0, s); }
inline void launch_q4km_persistent_gemv_v2(const void* w, const float* x, float* y, int K, int N, int64_t stride, cudaStream_t s = nullptr) { (void)ptm_q4k_gemv(w, x, y, K, N, stride, 0, s); }
/* CUDAOps.h:613-616 */
inline void launch_q4km_persistent_gemv_accumulate(const void* w, const float* x, float* y, int K, int N, int64_t stride, cudaStream_t s = nullptr) { (void)ptm_q4k_gemv(w, x, y, K, N, stride, 1, s); }
/* CUDAOps.h:498-501 */
inline void launch_q6k_gemv(const void* w, const float* x, float* y, int K, int N, int64_t stride, cudaStream_t s = nullptr) { (void)ptm_q6k_gemv(w, x, y, K, N, stride, 0, s); }
/* CUDAOps.h:503-507 */
inline void launch_q5k_gemv(const void* w, const float* x, float* y, int K, int N, int64_t stride, cudaStream_t s = nullptr) { (void)ptm_q5k_gemv(w, x, y, K, N, stride, 0, s); }
/* CUDAOps.h:453-458 */
inline void launch_q4km_fused_gate_up_gemv(const void* wg, const void* wu, const float* x, float* yg, float* yu, int K, int Ng, int Nu, int64_t stride, cudaStream_t s = nullptr) { (void)ptm_q4k_fused_gate_up_gemv(wg, wu, x, yg, yu, K, Ng, Nu, stride, s); }
/* CUDAOps.h:578-583 */
inline void launch_q4km_fused_qkv_gemv(const void* wq, const void* wk, const void* wv, const float* x, float* oq, float* ok, float* ov, int K, int Nq, int Nk, int Nv, int64_t stride, cudaStream_t s = nullptr) { (void)ptm_q4k_fused_qkv_gemv(wq, wk, wv, x, oq, ok, ov, K, Nq, Nk, Nv, stride, s); }
/* CUDAOps.h:589-594 */
inline void launch_q4km_fused_rmsnorm_gemv(const float* x, const float* nw, const void* w, float* y, int K, int N, int64_t stride, float eps, bool add_one, cudaStream_t s = nullptr) { (void)ptm_q4k_fused_rmsnorm_gemv(x, nw, w, y, K, N, stride, eps, add_one, s); }
/* CUDAOps.h:600-607 */
inline void launch_q4km_fused_rmsnorm_qkv_gemv(const float* x, const float* nw, const void* wq, const void* wk, const void* wv, float* oq, float* ok, float* ov, int K, int Nq, int Nk, int Nv, int64_t stride, float eps, bool add_one, cudaStream_t s = nullptr) { (void)ptm_q4k_fused_rmsnorm_qkv_gemv(x, nw, wq, wk, wv, oq, ok, ov, K, Nq, Nk, Nv, stride, eps, add_one, s); }
/* CUDAOps.h:621-628 */
inline void launch_q4km_fused_rmsnorm_gate_up_gemv(const float* x, const float* nw, const void* wg, const void* wu, float* yg, float* yu, int K, int Ng, int Nu, int64_t stride, float eps, bool add_one, cudaStream_t s = nullptr) { (void)ptm_q4k_fused_rmsnorm_gate_up_gemv(x, nw, wg, wu, yg, yu, K, Ng, Nu, stride, eps, add_one, s); }
/* CUDAOps.h:477-480 */
inline void launch_dequant_q4k_to_fp16(const void* w, void* out, int K, int N, int64_t stride, cudaStream_t s = nullptr) { (void)ptm_dequant_q4k_to_fp16(w, out, K, N, stride, s); }
/* CUDAOps.h:474: dynamic-LDS limits need no up-front call here; kept so call sites compile */
inline void init_cuda_kernel_smem_attributes(int, int) {}

/* Unquantised weights.  CUDAOps.h:188-192 (y[M] = A[M][N] . x), :422-424 (W is [K][N]), :493-495 (fp16 W[N][K]),
 * :484-489 (fp16, x rounded to fp16; the two scratch buffers are not needed here) */
inline void launch_gemv(const float* A, const float* x, float* y, int M, int N, cudaStream_t s = nullptr) { (void)ptm_f32_gemv(A, x, y, N, M, 0, s); }
inline void launch_inference_gemv(const float* x, const float* W, float* y, int K, int N, cudaStream_t s = nullptr) { (void)ptm_f32_gemv(W, x, y, K, N, 1, s); }
inline void launch_fp16_gemv(const void* w, const float* x, float* y, int K, int N, cudaStream_t s = nullptr) { (void)ptm_f16_gemv(w, x, y, K, N, 0, 0, s); }
inline void launch_cublas_hgemv(const void* w, const float* x, float* y, int K, int N, void* /*x_fp16_buf*/, void* /*y_fp16_buf*/, cudaStream_t s = nullptr, bool row_major = false) { (void)ptm_f16_gemv(w, x, y, K, N, row_major ? 0 : 1, 1, s); }

/* CUDAOps.h:382-390 */
inline void launch_rms_norm(const float* in, const float* w, float* out, int rows, int hidden, float eps, bool add_one, cudaStream_t s = nullptr) { (void)ptm_rms_norm(in, w, out, rows, hidden, eps, add_one, nullptr, s); }
inline void launch_per_head_rms_norm(float* data, const float* w, int rows, int n_heads, int head_dim, float eps, bool add_one, cudaStream_t s = nullptr) { (void)ptm_per_head_rms_norm(data, w, rows, n_heads, head_dim, eps, add_one, s); }
/* CUDAOps.h:416-418 */
inline void launch_silu_mul(const float* g, const float* u, float* o, int64_t n, cudaStream_t s = nullptr) { (void)ptm_silu_mul(g, u, o, n, s); }
/* CUDAOps.h:149-152 */
inline void launch_embedding_lookup(const float* table, float* out, const int* d_token_id, int hidden, cudaStream_t s = nullptr) { (void)ptm_embedding_row(table, out, d_token_id, hidden, s); }
/* CUDAOps.h:145 */
inline void launch_argmax(const float* in, int64_t* out, int64_t n, cudaStream_t s = nullptr) { (void)ptm_argmax(in, out, n, s); }
/* CUDAOps.h:63, :67, :83 */
inline void launch_add(const float* a, const float* b, float* o, int64_t n, cudaStream_t s = nullptr) { (void)ptm_add(a, b, o, n, s); }
inline void launch_mul_scalar(const float* a, float scalar, float* o, int64_t n, cudaStream_t s = nullptr) { (void)ptm_mul_scalar(a, scalar, o, n, s); }
inline void launch_copy(const float* in, float* out, int64_t n, cudaStream_t s = nullptr) { (void)ptm_copy(in, out, n, s); }
/* CUDAOps.h:404-413, :635-638 */
inline void launch_concat(const float* a, const float* b, float* o, int64_t a_rows, int64_t b_rows, int64_t cols, cudaStream_t s = nullptr) { (void)ptm_concat_rows(a, b, o, a_rows, b_rows, cols, s); }
inline void launch_kv_cache_write(const float* src, float* dst, int64_t rows, int64_t cols, int64_t off, cudaStream_t s = nullptr) { (void)ptm_kv_cache_write(src, dst, rows, cols, off, s); }
inline void launch_fp16_kv_cache_write(const float* src, void* dst, int64_t rows, int64_t cols, int64_t off, cudaStream_t s = nullptr) { (void)ptm_fp16_kv_cache_write(src, dst, rows, cols, off, s); }
/* CUDAOps.h:392-395: prompt rows rotated in place */
inline void launch_rope(float* data, int seq_len, int n_heads, int head_dim, int position_offset, float freq_base, cudaStream_t s = nullptr) {
    const PtmShimContext& c = ptm_shim_context();
    (void)ptm_rope(data, seq_len, n_heads, head_dim, position_offset, freq_base, c.rope_table, c.max_seq, c.rope_neox, s);
}
/* CUDAOps.h:397-402: K and V hold total_seq = past_len + seq_len rows (the prompt rows' own K/V included) */
inline void launch_causal_attention(const float* Q, const float* K, const float* V, float* out, int seq_len, int total_seq, int n_heads, int n_kv_heads, int head_dim, int past_len, float scale, cudaStream_t s = nullptr) {
    (void)ptm_prefill_attention(Q, K, V, out, seq_len, n_heads, n_kv_heads, head_dim, past_len, total_seq, scale, 0, s);
}

/* CUDAOps.h:556-557 */
inline int flash_decode_num_splits(int total_seq) { return ptm_flash_decode_num_splits(total_seq); }
inline int flash_decode_kv_chunk_size() { return ptm_flash_decode_kv_chunk_size(); }

/* CUDAOps.h:563-570 (position and cache row from the host) and :653-659 (both read from *d_past_len) */
inline void launch_fused_qknorm_rope_kvwrite(float* Q, float* K, const float* V, const float* qw, const float* kw, float* Kc, float* Vc, int n_heads, int n_kv_heads, int head_dim, int position, float base, float eps, bool add_one, int64_t cache_offset_row, cudaStream_t s = nullptr) {
    const PtmShimContext& c = ptm_shim_context();
    (void)ptm_qknorm_rope_kvwrite_pos(Q, K, V, qw, kw, Kc, Vc, n_heads, n_kv_heads, head_dim, position, cache_offset_row, c.max_seq, base, c.rope_table, eps, add_one, c.rope_neox, 0, s);
}
inline void launch_fused_qknorm_rope_kvwrite_graph(float* Q, float* K, const float* V, const float* qw, const float* kw, float* Kc, float* Vc, int n_heads, int n_kv_heads, int head_dim, const int64_t* d_past_len, float base, float eps, bool add_one, cudaStream_t s = nullptr) {
    const PtmShimContext& c = ptm_shim_context();
    (void)ptm_qknorm_rope_kvwrite(Q, K, V, qw, kw, Kc, Vc, n_heads, n_kv_heads, head_dim, d_past_len, c.max_seq, base, c.rope_table, eps, add_one, c.rope_neox, 0, s);
}
/* CUDAOps.h:543-549, :641-647: row count from the host */
inline void launch_flash_decode(const float* Q, const float* Kc, const float* Vc, float* O, float* pO, float* pL, float* pM, int n_heads, int n_kv_heads, int head_dim, int total_seq, float scale, cudaStream_t s = nullptr) {
    (void)ptm_flash_decode_pos(Q, Kc, Vc, O, pO, pL, pM, n_heads, n_kv_heads, head_dim, total_seq, scale, 0, s);
}
inline void launch_flash_decode_fp16(const float* Q, const void* Kc, const void* Vc, float* O, float* pO, float* pL, float* pM, int n_heads, int n_kv_heads, int head_dim, int total_seq, float scale, cudaStream_t s = nullptr) {
    (void)ptm_flash_decode_pos(Q, Kc, Vc, O, pO, pL, pM, n_heads, n_kv_heads, head_dim, total_seq, scale, 1, s);
}
/* CUDAOps.h:661-673: row count read from *d_past_len */
inline void launch_flash_decode_graph(const float* Q, const float* Kc, const float* Vc, float* O, float* pO, float* pL, float* pM, int n_heads, int n_kv_heads, int head_dim, const int64_t* d_past_len, int max_seq, float scale, cudaStream_t s = nullptr) {
    (void)ptm_flash_decode(Q, Kc, Vc, O, pO, pL, pM, n_heads, n_kv_heads, head_dim, d_past_len, max_seq, scale, 0, s);
}
inline void launch_flash_decode_fp16_graph(const float* Q, const void* Kc, const void* Vc, float* O, float* pO, float* pL, float* pM, int n_heads, int n_kv_heads, int head_dim, const int64_t* d_past_len, int max_seq, float scale, cudaStream_t s = nullptr) {
    (void)ptm_flash_decode(Q, Kc, Vc, O, pO, pL, pM, n_heads, n_kv_heads, head_dim, d_past_len, max_seq, scale, 1, s);
}

}  // namespace cuda
}  // namespace at

#endif /* PTM_AT_CUDA_SHIM_H */
