"""Python mirror of the reference's quantized-linear / decode operators.

Each function carries the name and argument order of the `at::cuda::launch_*` function it
stands in for (reference: aten/src/ATen/cuda/CUDAOps.h; line cited per function) and forwards to
the C ABI of libptm_hip.so.  Arguments are torch CUDA tensors (used only as device memory) or
raw integer device pointers; `stream` is a `torch.cuda.Stream`, an integer hipStream_t, or None
for torch's current stream.  Unlike the reference launchers (void, unchecked), a violated
precondition raises `PtmError`.  There is no CPU or PyTorch fallback."""
from __future__ import annotations

import ctypes as C

import torch

from . import _lib
from ._lib import PtmError, check  # noqa: F401

Q4_K, Q6_K = 12, 14


def _ptr(t):
    if t is None:
        return None
    if isinstance(t, int):
        return t
    if not t.is_cuda:
        raise ValueError("expected a CUDA (HIP) tensor")
    return t.data_ptr()


def _stream(s):
    if s is None:
        return torch.cuda.current_stream().cuda_stream
    if isinstance(s, int):
        return s
    return s.cuda_stream


def _L():
    return _lib.load()


# ---- dequantisation -------------------------------------------------------------------
def dequant_q4k(blocks, out, n_elems, stream=None):
    check(_L().ptm_dequant_q4k(_ptr(blocks), _ptr(out), n_elems, _stream(stream)), "dequant_q4k")


def dequant_q6k(blocks, out, n_elems, stream=None):
    check(_L().ptm_dequant_q6k(_ptr(blocks), _ptr(out), n_elems, _stream(stream)), "dequant_q6k")


def dequant_q8_0(blocks, out, n_elems, stream=None):
    """dequantize_q8_0 (gguf_dequant.h:237-255)"""
    check(_L().ptm_dequant_q8_0(_ptr(blocks), _ptr(out), n_elems, _stream(stream)), "dequant_q8_0")


def dequant_q5k(blocks, out, n_elems, stream=None):
    """dequantize_q5_k (gguf_dequant.h:348-388)"""
    check(_L().ptm_dequant_q5k(_ptr(blocks), _ptr(out), n_elems, _stream(stream)), "dequant_q5k")


def launch_dequant_q4k_to_fp16(weights, out_fp16, K, N, row_stride_bytes, stream=None):
    """CUDAOps.h:477-480"""
    check(_L().ptm_dequant_q4k_to_fp16(_ptr(weights), _ptr(out_fp16), K, N, row_stride_bytes, _stream(stream)),
          "dequant_q4k_to_fp16")


# ---- activations ----------------------------------------------------------------------
def q8_bytes(K):
    return _L().ptm_q8_bytes(K)


def launch_quantize_q8(x, y_q8, K, stream=None):
    """Role of launch_quantize_q8_1 (CUDAOps.h:462-464) with the CPU path's Q8 block rule."""
    check(_L().ptm_quantize_q8(_ptr(x), _ptr(y_q8), K, _stream(stream)), "quantize_q8")


# ---- GEMV -----------------------------------------------------------------------------
def launch_q4km_persistent_gemv(weights, x, y, K, N, row_stride_bytes, stream=None):
    """CUDAOps.h:435-438 (also launch_q4km_gemv :427-430 and _v2 :445-448)"""
    check(_L().ptm_q4k_gemv(_ptr(weights), _ptr(x), _ptr(y), K, N, row_stride_bytes, 0, _stream(stream)), "q4k_gemv")


launch_q4km_gemv = launch_q4km_persistent_gemv
launch_q4km_persistent_gemv_v2 = launch_q4km_persistent_gemv


def launch_q4km_persistent_gemv_accumulate(weights, x, y, K, N, row_stride_bytes, stream=None):
    """CUDAOps.h:613-616: y += W.x"""
    check(_L().ptm_q4k_gemv(_ptr(weights), _ptr(x), _ptr(y), K, N, row_stride_bytes, 1, _stream(stream)),
          "q4k_gemv_accumulate")


def launch_q4km_q8_gemv(weights, x_q8, y, K, N, row_stride_bytes, stream=None, accumulate=False):
    """CUDAOps.h:467-470"""
    check(_L().ptm_q4k_gemv_q8(_ptr(weights), _ptr(x_q8), _ptr(y), K, N, row_stride_bytes, int(accumulate),
                              _stream(stream)), "q4k_gemv_q8")


def launch_q6k_gemv(weights, x, y, K, N, row_stride_bytes, stream=None, accumulate=False):
    """CUDAOps.h:498-501"""
    check(_L().ptm_q6k_gemv(_ptr(weights), _ptr(x), _ptr(y), K, N, row_stride_bytes, int(accumulate), _stream(stream)),
          "q6k_gemv")


def argmax_workspace_bytes(N):
    return _L().ptm_argmax_workspace_bytes(N)


def q6k_gemv_argmax(weights, x, logits, K, N, row_stride_bytes, out_index, workspace, stream=None):
    """launch_q6k_gemv + launch_argmax fused (CUDAOps.h:498-501, :145)."""
    check(_L().ptm_q6k_gemv_argmax(_ptr(weights), _ptr(x), _ptr(logits), K, N, row_stride_bytes, _ptr(out_index),
                                  _ptr(workspace), _stream(stream)), "q6k_gemv_argmax")


def quant_gemv(quant_type, weights, x, y, K, N, row_stride_bytes, stream=None, accumulate=False):
    """cpu_quant_gemv / gemv_scratch dispatch (cpu_quant_gemv.h:1635-1688, gguf_model.h:3117-3140)."""
    check(_L().ptm_quant_gemv(quant_type, _ptr(weights), _ptr(x), _ptr(y), K, N, row_stride_bytes, int(accumulate),
                             _stream(stream)), "quant_gemv")


def quant_gemv_supported(quant_type) -> bool:
    """cpu_quant_gemv_supported (cpu_quant_gemv.h:1691-1694)"""
    return bool(_L().ptm_quant_gemv_supported(quant_type))


def launch_q4km_fused_gate_up_gemv(w_gate, w_up, x, y_gate, y_up, K, N_gate, N_up, row_stride_bytes, stream=None):
    """CUDAOps.h:453-458"""
    check(_L().ptm_q4k_fused_gate_up_gemv(_ptr(w_gate), _ptr(w_up), _ptr(x), _ptr(y_gate), _ptr(y_up), K, N_gate, N_up,
                                         row_stride_bytes, _stream(stream)), "fused_gate_up_gemv")


def launch_q4km_fused_qkv_gemv(w_q, w_k, w_v, x, out_q, out_k, out_v, K, N_q, N_k, N_v, row_stride_bytes, stream=None):
    """CUDAOps.h:578-583"""
    check(_L().ptm_q4k_fused_qkv_gemv(_ptr(w_q), _ptr(w_k), _ptr(w_v), _ptr(x), _ptr(out_q), _ptr(out_k), _ptr(out_v),
                                     K, N_q, N_k, N_v, row_stride_bytes, _stream(stream)), "fused_qkv_gemv")


def launch_q4km_fused_rmsnorm_gemv(x, norm_weight, weights, y, K, N, row_stride_bytes, eps, add_one, stream=None):
    """CUDAOps.h:589-594"""
    check(_L().ptm_q4k_fused_rmsnorm_gemv(_ptr(x), _ptr(norm_weight), _ptr(weights), _ptr(y), K, N, row_stride_bytes,
                                         eps, int(add_one), _stream(stream)), "fused_rmsnorm_gemv")


def launch_q4km_fused_rmsnorm_qkv_gemv(x, norm_weight, w_q, w_k, w_v, out_q, out_k, out_v, K, N_q, N_k, N_v,
                                       row_stride_bytes, eps, add_one, stream=None):
    """CUDAOps.h:600-607"""
    check(_L().ptm_q4k_fused_rmsnorm_qkv_gemv(_ptr(x), _ptr(norm_weight), _ptr(w_q), _ptr(w_k), _ptr(w_v), _ptr(out_q),
                                             _ptr(out_k), _ptr(out_v), K, N_q, N_k, N_v, row_stride_bytes, eps,
                                             int(add_one), _stream(stream)), "fused_rmsnorm_qkv_gemv")


def launch_q4km_fused_rmsnorm_gate_up_gemv(x, norm_weight, w_gate, w_up, y_gate, y_up, K, N_gate, N_up,
                                           row_stride_bytes, eps, add_one, stream=None):
    """CUDAOps.h:621-628"""
    check(_L().ptm_q4k_fused_rmsnorm_gate_up_gemv(_ptr(x), _ptr(norm_weight), _ptr(w_gate), _ptr(w_up), _ptr(y_gate),
                                                 _ptr(y_up), K, N_gate, N_up, row_stride_bytes, eps, int(add_one),
                                                 _stream(stream)), "fused_rmsnorm_gate_up_gemv")


def fused_rmsnorm_gate_up_silu(x, norm_weight, w_gate, w_up, act, K, N, row_stride_bytes, eps, add_one, stream=None):
    """launch_q4km_fused_rmsnorm_gate_up_gemv + launch_silu_mul in one launch (gguf_model.h:2954-2986)."""
    check(_L().ptm_q4k_fused_rmsnorm_gate_up_silu(_ptr(x), _ptr(norm_weight), _ptr(w_gate), _ptr(w_up), _ptr(act), K, N,
                                                 row_stride_bytes, eps, int(add_one), _stream(stream)),
          "fused_rmsnorm_gate_up_silu")


# ---- glue -----------------------------------------------------------------------------
def launch_rms_norm(input, weight, output, rows, hidden, eps, add_one, stream=None, q8_out=None):
    """CUDAOps.h:382-385"""
    check(_L().ptm_rms_norm(_ptr(input), _ptr(weight), _ptr(output), rows, hidden, eps, int(add_one), _ptr(q8_out),
                           _stream(stream)), "rms_norm")


def launch_per_head_rms_norm(data, weight, rows, n_heads, head_dim, eps, add_one, stream=None):
    """CUDAOps.h:387-390"""
    check(_L().ptm_per_head_rms_norm(_ptr(data), _ptr(weight), rows, n_heads, head_dim, eps, int(add_one),
                                    _stream(stream)), "per_head_rms_norm")


def launch_fused_qknorm_rope_kvwrite_graph(Q, K, V, q_norm_w, k_norm_w, K_cache, V_cache, n_heads, n_kv_heads,
                                           head_dim, d_past_len, rope_freq_base, eps, add_one, stream=None, *,
                                           max_seq, rope_table=None, neox=True, kv_fp16=True):
    """CUDAOps.h:653-659 (and :563-570 with the position in device memory)."""
    check(_L().ptm_qknorm_rope_kvwrite(_ptr(Q), _ptr(K), _ptr(V), _ptr(q_norm_w), _ptr(k_norm_w), _ptr(K_cache),
                                      _ptr(V_cache), n_heads, n_kv_heads, head_dim, _ptr(d_past_len), max_seq,
                                      rope_freq_base, _ptr(rope_table), eps, int(add_one), int(neox), int(kv_fp16),
                                      _stream(stream)), "qknorm_rope_kvwrite")


def rope_table(max_seq, head_dim, rope_freq_base, scale=1.0):
    """Host-computed cos/sin rows [max_seq, head_dim] (hot_loops.cpp:1853-1876), returned as a CPU tensor; scale: linear
    position scaling, theta = (pos / scale) * freq."""
    t = torch.empty(max_seq, head_dim, dtype=torch.float32)
    check(_L().ptm_rope_table_host_scaled(t.data_ptr(), max_seq, head_dim, rope_freq_base, scale), "rope_table_host")
    return t


def launch_fp16_kv_cache_write(src, dst_cache_fp16, num_new_rows, cols, offset_row, stream=None):
    """CUDAOps.h:635-638"""
    check(_L().ptm_fp16_kv_cache_write(_ptr(src), _ptr(dst_cache_fp16), num_new_rows, cols, offset_row,
                                      _stream(stream)), "fp16_kv_cache_write")


def flash_decode_num_splits(total_seq):
    """CUDAOps.h:556"""
    return _L().ptm_flash_decode_num_splits(total_seq)


def flash_decode_kv_chunk_size():
    """CUDAOps.h:557"""
    return _L().ptm_flash_decode_kv_chunk_size()


def launch_flash_decode_graph(Q, K_cache, V_cache, O, partial_O, partial_lse, partial_max, n_heads, n_kv_heads,
                              head_dim, d_past_len, max_seq, scale, stream=None, *, kv_fp16=False):
    """CUDAOps.h:661-666 (fp32 KV) / :668-673 (fp16 KV)"""
    check(_L().ptm_flash_decode(_ptr(Q), _ptr(K_cache), _ptr(V_cache), _ptr(O), _ptr(partial_O), _ptr(partial_lse),
                               _ptr(partial_max), n_heads, n_kv_heads, head_dim, _ptr(d_past_len), max_seq, scale,
                               int(kv_fp16), _stream(stream)), "flash_decode")


def launch_flash_decode_fp16_graph(Q, K_cache_fp16, V_cache_fp16, O, partial_O, partial_lse, partial_max, n_heads,
                                   n_kv_heads, head_dim, d_past_len, max_seq, scale, stream=None):
    launch_flash_decode_graph(Q, K_cache_fp16, V_cache_fp16, O, partial_O, partial_lse, partial_max, n_heads,
                              n_kv_heads, head_dim, d_past_len, max_seq, scale, stream, kv_fp16=True)


def attn_decode_fused(Q, K, V, q_norm_w, k_norm_w, K_cache, V_cache, O, partial_O, partial_lse, partial_max,
                      rope_table, n_heads, n_kv_heads, head_dim, d_past_len, max_seq, scale, eps, add_one=False,
                      kv_fp16=True, stream=None, rope_interleaved=False, window=0):
    """launch_fused_qknorm_rope_kvwrite_graph + launch_flash_decode(_fp16)_graph fused (one launch + a small merge launch)
    (CUDAOps.h:653-673; issued back to back at gguf_model.h:2785-2832).  window > 0: only the last `window` positions."""
    check(_L().ptm_attn_decode_fused_window(_ptr(Q), _ptr(K), _ptr(V), _ptr(q_norm_w), _ptr(k_norm_w), _ptr(K_cache),
                                           _ptr(V_cache), _ptr(O), _ptr(partial_O), _ptr(partial_lse), _ptr(partial_max),
                                           _ptr(rope_table), n_heads, n_kv_heads, head_dim, _ptr(d_past_len),
                                           max_seq, scale, eps, int(add_one), int(kv_fp16), int(rope_interleaved),
                                           int(window), _stream(stream)),
          "attn_decode_fused")


def flash_decode_window(Q, K_cache, V_cache, O, partial_O, partial_lse, partial_max, n_heads, n_kv_heads, head_dim, d_past_len,
                        max_seq, scale, kv_fp16=True, window=0, o_q8=None, stream=None):
    """launch_flash_decode(_fp16)_graph over the last `window` positions (0: all); head_dim 64, 128 or 256."""
    check(_L().ptm_flash_decode_window(_ptr(Q), _ptr(K_cache), _ptr(V_cache), _ptr(O), _ptr(o_q8), _ptr(partial_O),
                                      _ptr(partial_lse), _ptr(partial_max), n_heads, n_kv_heads, head_dim, _ptr(d_past_len),
                                      max_seq, scale, int(kv_fp16), int(window), _stream(stream)), "flash_decode_window")


def gelu_mul(gate, up, out, n, stream=None):
    """tanh-GELU(gate) * up (gguf_model.h:3730-3738)."""
    check(_L().ptm_gelu_mul(_ptr(gate), _ptr(up), _ptr(out), n, _stream(stream)), "gelu_mul")


def rms_norm_add(h, weight, x, rows, hidden, eps, add_one=False, stream=None):
    """x[r] += RMSNorm(h[r]) * weight: a gemma post-norm with its residual add (gguf_model.h:3656-3680)."""
    check(_L().ptm_rms_norm_add(_ptr(h), _ptr(weight), _ptr(x), rows, hidden, eps, int(add_one), _stream(stream)), "rms_norm_add")


def scale(x, factor, n, stream=None):
    check(_L().ptm_scale(_ptr(x), factor, n, _stream(stream)), "scale")


def prefill_attention_window(Q, K_cache, V_cache, O, rows, n_heads, n_kv_heads, head_dim, pos0, max_seq, scale, kv_fp16, window,
                             stream=None):
    """Causal attention of prompt rows over the last `window` positions each (gguf_model.h:3490-3500)."""
    check(_L().ptm_prefill_attention_window(_ptr(Q), _ptr(K_cache), _ptr(V_cache), _ptr(O), rows, n_heads, n_kv_heads, head_dim,
                                           pos0, max_seq, scale, int(kv_fp16), int(window), _stream(stream)),
          "prefill_attention_window")


def launch_silu_mul(gate, up, output, n, stream=None):
    """CUDAOps.h:416-418"""
    check(_L().ptm_silu_mul(_ptr(gate), _ptr(up), _ptr(output), n, _stream(stream)), "silu_mul")


def launch_embedding_lookup(emb_table, output, d_token_id, hidden_size, stream=None):
    """CUDAOps.h:149-152"""
    check(_L().ptm_embedding_row(_ptr(emb_table), _ptr(output), _ptr(d_token_id), hidden_size, _stream(stream)),
          "embedding_lookup")


def embedding_lookup_q6k(table_q6k, output, d_token_id, hidden_size, row_stride_bytes, stream=None):
    check(_L().ptm_embedding_row_q6k(_ptr(table_q6k), _ptr(output), _ptr(d_token_id), hidden_size, row_stride_bytes,
                                    _stream(stream)), "embedding_lookup_q6k")


def launch_argmax(input, output, n, stream=None):
    """CUDAOps.h:145"""
    check(_L().ptm_argmax(_ptr(input), _ptr(output), n, _stream(stream)), "argmax")


def sampler_workspace_bytes():
    return int(_L().ptm_sampler_workspace_bytes())


def sample_token(logits, vocab, counts, temperature, top_k, top_p, repeat_penalty, d_uniform, workspace, out_token,
                 stream=None):
    """GGUFModel::sample_token (gguf_model.h:7658-7751) after the repetition penalty of generate() (:4926-4938), on
    the device; d_uniform holds the uniform draw, out_token (int64, device) receives the id."""
    from ._lib import Sampling
    p = Sampling(temperature, top_k, top_p, repeat_penalty)
    check(_L().ptm_sample_token(_ptr(logits), vocab, _ptr(counts), p, _ptr(d_uniform), _ptr(workspace), _ptr(out_token),
                                _stream(stream)), "sample_token")


def mt19937_uniforms(seed, skip, n):
    """The reference sampler's uniform draws: std::uniform_real_distribution<float>(0, 1) over std::mt19937(seed)."""
    import ctypes as C
    buf = (C.c_float * n)()
    check(_L().ptm_mt19937_uniforms(seed, skip, n, buf), "mt19937_uniforms")
    return list(buf)


def launch_add(a, b, out, n, stream=None):
    """CUDAOps.h:63"""
    check(_L().ptm_add(_ptr(a), _ptr(b), _ptr(out), n, _stream(stream)), "add")


def add_qkv_bias(Q, K, V, q_bias, k_bias, v_bias, rows, q_dim, kv_dim, stream=None):
    """The three launch_add calls of a qwen2-style layer (gguf_model.h:2768-2779) as one launch, for `rows` rows."""
    check(_L().ptm_add_qkv_bias(_ptr(Q), _ptr(K), _ptr(V), _ptr(q_bias), _ptr(k_bias), _ptr(v_bias), rows, q_dim, kv_dim,
                                _stream(stream)), "add_qkv_bias")


def launch_copy(input, output, n, stream=None):
    """CUDAOps.h:83"""
    check(_L().ptm_copy(_ptr(input), _ptr(output), n, _stream(stream)), "copy")


# ---- prefill GEMM ---------------------------------------------------------------------
def qgemm_workspace_bytes(M, K):
    return _L().ptm_qgemm_workspace_bytes(M, K)


def qgemm_f16_workspace_bytes(M, K):
    return _L().ptm_qgemm_f16_workspace_bytes(M, K)


def matmul_q_f16(quant_type, weights, x_bf16, y, M, K, N, row_stride_bytes, workspace, stream=None):
    """Fast quantised-weight GEMM for M > 1 rows (fp16 MFMA on dequantised weights, Q8-rounded activations);
    stands in for the M-GEMV loop of matmul_q (gguf_model.h:7029-7036) within the 1e-2 bar of the prefill path."""
    check(_L().ptm_qgemm_f16(quant_type, _ptr(weights), _ptr(x_bf16), _ptr(y), M, K, N, row_stride_bytes,
                             _ptr(workspace), _stream(stream)), "matmul_q_f16")


def qgemm_f16_f32_workspace_bytes(M, K, N):
    return int(_L().ptm_qgemm_f16_f32_workspace_bytes(M, K, N))


def matmul_q_f16_f32(quant_type, weights, x_f32, y, M, K, N, row_stride_bytes, workspace, accumulate=False, stream=None):
    """matmul_q_f16 on fp32 rows of X, optionally Y += result (the prefill's o-proj / down-proj residual adds)."""
    check(_L().ptm_qgemm_f16_f32(quant_type, _ptr(weights), _ptr(x_f32), _ptr(y), M, K, N, row_stride_bytes,
                                 _ptr(workspace), int(accumulate), _stream(stream)), "matmul_q_f16_f32")


def embedding_rows(table_f32, table_q6k, q6k_row_stride_bytes, d_tokens, rows, hidden, vocab, out, stream=None):
    """Rows of the token embedding for a batch of token ids (embedding_lookup, gguf_model.h:2513)."""
    check(_L().ptm_embedding_rows(_ptr(table_f32), _ptr(table_q6k), q6k_row_stride_bytes, _ptr(d_tokens), rows, hidden,
                                  vocab, _ptr(out), _stream(stream)), "embedding_rows")


def qknorm_rope_kvwrite_rows(Q, K, V, q_norm_w, k_norm_w, K_cache, V_cache, rope, rows, n_heads, n_kv_heads, head_dim,
                             pos0, max_seq, eps, add_one, kv_fp16, stream=None, rope_interleaved=False):
    """launch_fused_qknorm_rope_kvwrite (CUDAOps.h:563-570) over `rows` prompt rows at positions pos0 + r."""
    check(_L().ptm_qknorm_rope_kvwrite_rows(_ptr(Q), _ptr(K), _ptr(V), _ptr(q_norm_w), _ptr(k_norm_w), _ptr(K_cache),
                                            _ptr(V_cache), _ptr(rope), rows, n_heads, n_kv_heads, head_dim, pos0, max_seq,
                                            eps, int(add_one), int(kv_fp16), int(rope_interleaved), _stream(stream)),
          "qknorm_rope_kvwrite_rows")


def prefill_attention(Q, K_cache, V_cache, O, rows, n_heads, n_kv_heads, head_dim, pos0, max_seq, scale, kv_fp16,
                      stream=None):
    """Causal GQA attention of prompt rows over the cache (launch_causal_attention, gguf_model.h:7400)."""
    check(_L().ptm_prefill_attention(_ptr(Q), _ptr(K_cache), _ptr(V_cache), _ptr(O), rows, n_heads, n_kv_heads, head_dim,
                                     pos0, max_seq, scale, int(kv_fp16), _stream(stream)), "prefill_attention")


def matmul_q(quant_type, weights, x_bf16, y, M, K, N, row_stride_bytes, workspace, stream=None):
    """Quantised-weight GEMM for M > 1 rows with the GEMV's arithmetic per row (Q4_K: bit-identical rows);
    stands in for the M-GEMV loop of matmul_q (gguf_model.h:7029-7036)."""
    fn = _L().ptm_qgemm_q4k if quant_type == Q4_K else _L().ptm_qgemm_q6k
    if quant_type not in (Q4_K, Q6_K):
        raise PtmError(-4, "matmul_q: unsupported quant type")
    check(fn(_ptr(weights), _ptr(x_bf16), _ptr(y), M, K, N, row_stride_bytes, _ptr(workspace), _stream(stream)),
          "matmul_q")
