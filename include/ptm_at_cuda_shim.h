/*
 * ptm_at_cuda_shim.h — the reference's operator names on top of the ptm C ABI.
 *
 * PromeTorch's host code (torch/io/gguf_model.h forward_decode, gemv_scratch, matmul_q, KVCache)
 * calls free functions `at::cuda::launch_*` declared in aten/src/ATen/cuda/CUDAOps.h.  Including
 * this header instead (on a ROCm build) gives the same names, argument order and default stream
 * argument as inline forwards to libptm_hip.so, so that host code compiles unchanged for the
 * hot path.  Each forward cites the CUDAOps.h declaration it stands in for.  The reference's
 * launchers return void and check nothing; these keep that contract and drop the status code
 * (call the ptm_* function directly to see it).
 */
#ifndef PTM_AT_CUDA_SHIM_H
#define PTM_AT_CUDA_SHIM_H

#include <hip/hip_runtime_api.h>
#include <stdint.h>

#include "ptm.h"

typedef hipStream_t cudaStream_t; /* the reference spells the stream type the CUDA way */

namespace at {
namespace cuda {

/* CUDAOps.h:427-448 */
inline void launch_q4km_gemv(const void* w, const float* x, float* y, int K, int N, int64_t stride, cudaStream_t s = nullptr) { (void)ptm_q4k_gemv(w, x, y, K, N, stride, 0, s); }
inline void launch_q4km_persistent_gemv(const void* w, const float* x, float* y, int K, int N, int64_t stride, cudaStream_t s = nullptr) { (void)ptm_q4k_gemv(w, x, y, K, N, stride, 0, s); }
inline void launch_q4km_persistent_gemv_v2(const void* w, const float* x, float* y, int K, int N, int64_t stride, cudaStream_t s = nullptr) { (void)ptm_q4k_gemv(w, x, y, K, N, stride, 0, s); }
/* CUDAOps.h:613-616 */
inline void launch_q4km_persistent_gemv_accumulate(const void* w, const float* x, float* y, int K, int N, int64_t stride, cudaStream_t s = nullptr) { (void)ptm_q4k_gemv(w, x, y, K, N, stride, 1, s); }
/* CUDAOps.h:462-470 (Q8 blocks use the CPU path's layout: ptm_q8_bytes(K) bytes) */
inline void launch_quantize_q8_1(const float* x, void* y_q8, int K, cudaStream_t s = nullptr) { (void)ptm_quantize_q8(x, y_q8, K, s); }
inline void launch_q4km_q8_gemv(const void* w, const void* x_q8, float* y, int K, int N, int64_t stride, cudaStream_t s = nullptr) { (void)ptm_q4k_gemv_q8(w, x_q8, y, K, N, stride, 0, s); }
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

/* CUDAOps.h:382-390 */
inline void launch_rms_norm(const float* in, const float* w, float* out, int rows, int hidden, float eps, bool add_one, cudaStream_t s = nullptr) { (void)ptm_rms_norm(in, w, out, rows, hidden, eps, add_one, nullptr, s); }
inline void launch_per_head_rms_norm(float* data, const float* w, int rows, int n_heads, int head_dim, float eps, bool add_one, cudaStream_t s = nullptr) { (void)ptm_per_head_rms_norm(data, w, rows, n_heads, head_dim, eps, add_one, s); }
/* CUDAOps.h:416-418 */
inline void launch_silu_mul(const float* g, const float* u, float* o, int64_t n, cudaStream_t s = nullptr) { (void)ptm_silu_mul(g, u, o, n, s); }
/* CUDAOps.h:149-152 */
inline void launch_embedding_lookup(const float* table, float* out, const int* d_token_id, int hidden, cudaStream_t s = nullptr) { (void)ptm_embedding_row(table, out, d_token_id, hidden, s); }
/* CUDAOps.h:145 */
inline void launch_argmax(const float* in, int64_t* out, int64_t n, cudaStream_t s = nullptr) { (void)ptm_argmax(in, out, n, s); }
/* CUDAOps.h:63, :83 */
inline void launch_add(const float* a, const float* b, float* o, int64_t n, cudaStream_t s = nullptr) { (void)ptm_add(a, b, o, n, s); }
inline void launch_copy(const float* in, float* out, int64_t n, cudaStream_t s = nullptr) { (void)ptm_copy(in, out, n, s); }
/* CUDAOps.h:635-638 */
inline void launch_fp16_kv_cache_write(const float* src, void* dst, int64_t rows, int64_t cols, int64_t off, cudaStream_t s = nullptr) { (void)ptm_fp16_kv_cache_write(src, dst, rows, cols, off, s); }

/* CUDAOps.h:556-557 */
inline int flash_decode_num_splits(int total_seq) { return ptm_flash_decode_num_splits(total_seq); }
inline int flash_decode_kv_chunk_size() { return ptm_flash_decode_kv_chunk_size(); }

/* CUDAOps.h:653-659.  The reference's CUDA kernel rotates interleaved pairs while its CPU path uses
 * NeoX pairs for qwen3 (gguf_model.h:3464-3470); `PTM_SHIM_ROPE_NEOX` selects (default: NeoX, the
 * CPU behaviour).  max_seq is not part of the reference signature: the caller's cache height is
 * taken from PTM_SHIM_MAX_SEQ. */
#ifndef PTM_SHIM_ROPE_NEOX
#define PTM_SHIM_ROPE_NEOX 1
#endif
#ifndef PTM_SHIM_MAX_SEQ
#define PTM_SHIM_MAX_SEQ 4096 /* PromeServe's fixed KV height, promeserve/api_handlers.h:769 */
#endif
inline void launch_fused_qknorm_rope_kvwrite_graph(float* Q, float* K, const float* V, const float* qw, const float* kw, float* Kc, float* Vc, int n_heads, int n_kv_heads, int head_dim, const int64_t* d_past_len, float base, float eps, bool add_one, cudaStream_t s = nullptr) {
    (void)ptm_qknorm_rope_kvwrite(Q, K, V, qw, kw, Kc, Vc, n_heads, n_kv_heads, head_dim, d_past_len, PTM_SHIM_MAX_SEQ, base, nullptr, eps, add_one, PTM_SHIM_ROPE_NEOX, 0, s);
}
/* CUDAOps.h:661-673 */
inline void launch_flash_decode_graph(const float* Q, const float* Kc, const float* Vc, float* O, float* pO, float* pL, float* pM, int n_heads, int n_kv_heads, int head_dim, const int64_t* d_past_len, int max_seq, float scale, cudaStream_t s = nullptr) {
    (void)ptm_flash_decode(Q, Kc, Vc, O, pO, pL, pM, n_heads, n_kv_heads, head_dim, d_past_len, max_seq, scale, 0, s);
}
inline void launch_flash_decode_fp16_graph(const float* Q, const void* Kc, const void* Vc, float* O, float* pO, float* pL, float* pM, int n_heads, int n_kv_heads, int head_dim, const int64_t* d_past_len, int max_seq, float scale, cudaStream_t s = nullptr) {
    (void)ptm_flash_decode(Q, Kc, Vc, O, pO, pL, pM, n_heads, n_kv_heads, head_dim, d_past_len, max_seq, scale, 1, s);
}

}  // namespace cuda
}  // namespace at

#endif /* PTM_AT_CUDA_SHIM_H */
