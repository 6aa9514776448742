"""ctypes binding of libptm_hip.so (the C ABI declared in include/ptm.h).

There is no fallback: if the library has not been built, or an entry point is missing,
loading raises.  Build it with `python -m prometorch_amd.build` (hipcc, gfx950)."""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("PTM_LIB_PATH") or os.path.join(HERE, "libptm_hip.so")  # PTM_LIB_PATH: load another build

vp, i64, i32, u32, f32 = C.c_void_p, C.c_int64, C.c_int, C.c_uint32, C.c_float


class PtmError(RuntimeError):
    def __init__(self, code: int, what: str):
        super().__init__(f"{what}: {code}")
        self.code = code


# ggml type id -> (bytes per block, values per block) of the formats the GEMV dispatcher takes (gguf_dequant.h:29-58)
BLOCK = {12: (144, 256), 14: (210, 256), 13: (176, 256), 8: (34, 32), 6: (22, 32)}


def weight_cols(qtype: int, row_bytes: int) -> int:
    """Values per row of a matrix whose rows are row_bytes of qtype blocks."""
    b, per = BLOCK[qtype]
    return row_bytes // b * per


class QWeight(C.Structure):
    _fields_ = [("data", vp), ("ggml_type", u32), ("rows", C.c_int32), ("cols", C.c_int32), ("row_stride_bytes", i64)]


class Layer(C.Structure):
    _fields_ = [(n, QWeight) for n in ("q", "k", "v", "o", "gate", "up", "down")] + \
               [(n, vp) for n in ("attn_norm", "ffn_norm", "q_norm", "k_norm", "k_cache", "v_cache",
                                  "q_bias", "k_bias", "v_bias", "post_attn_norm", "post_ffn_norm")]


class DecodeConfig(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("vocab", "hidden", "n_layers", "n_heads", "n_kv_heads", "head_dim", "inter", "max_seq")] + \
               [("rope_freq_base", f32), ("rms_eps", f32), ("kv_fp16", C.c_int32), ("use_graph", C.c_int32),
                ("embedding_f32", vp), ("layers", C.POINTER(Layer)), ("out_norm", vp), ("lm_head", QWeight),
                ("rope_interleaved", C.c_int32), ("rope_scale", f32), ("scale_embeddings", C.c_int32),
                ("ffn_gelu", C.c_int32), ("swa_window", C.c_int32), ("swa_pattern", C.c_int32), ("rope_swa_freq_base", f32),
                ("rope_factors_short", vp), ("rope_factors_long", vp), ("rope_orig_ctx", C.c_int32), ("rope_attn_factor", f32)]


class Sampling(C.Structure):
    _fields_ = [("temperature", f32), ("top_k", C.c_int32), ("top_p", f32), ("repeat_penalty", f32)]


class GgufTensor(C.Structure):
    _fields_ = [("name", C.c_char_p), ("ggml_type", u32), ("n_dims", C.c_int32), ("dims", i64 * 4), ("nbytes", i64),
                ("data", vp)]


# name -> (restype, argtypes); every function declared in include/ptm.h
SIGNATURES = {
    "ptm_strerror": (C.c_char_p, [i32]),
    "ptm_last_hip_error": (i32, []),
    "ptm_version": (i32, []),
    "ptm_device_cus": (i32, []),
    "ptm_dequant_q4k": (i32, [vp, vp, i64, vp]),
    "ptm_dequant_q6k": (i32, [vp, vp, i64, vp]),
    "ptm_dequant_q8_0": (i32, [vp, vp, i64, vp]),
    "ptm_dequant_q5k": (i32, [vp, vp, i64, vp]),
    "ptm_q8_0_gemv": (i32, [vp, vp, vp, i32, i32, i64, i32, vp]),
    "ptm_q5k_gemv": (i32, [vp, vp, vp, i32, i32, i64, i32, vp]),
    "ptm_q5_0_gemv": (i32, [vp, vp, vp, i32, i32, i64, i32, vp]),
    "ptm_quant_gemv_supported": (i32, [u32]),
    "ptm_dequant_q4k_to_fp16": (i32, [vp, vp, i32, i32, i64, vp]),
    "ptm_q8_bytes": (i64, [i32]),
    "ptm_quantize_q8": (i32, [vp, vp, i32, vp]),
    "ptm_q4k_gemv": (i32, [vp, vp, vp, i32, i32, i64, i32, vp]),
    "ptm_q4k_gemv_q8": (i32, [vp, vp, vp, i32, i32, i64, i32, vp]),
    "ptm_q4k_gemv_f32act": (i32, [vp, vp, vp, i32, i32, i64, i32, vp]),
    "ptm_q6k_gemv": (i32, [vp, vp, vp, i32, i32, i64, i32, vp]),
    "ptm_argmax_workspace_bytes": (i64, [i32]),
    "ptm_q6k_gemv_argmax": (i32, [vp, vp, vp, i32, i32, i64, vp, vp, vp]),
    "ptm_q6k_gemv_argmax_noalloc_max_rows": (i32, []),
    "ptm_q6k_gemv_argmax_noalloc_init": (i32, []),
    "ptm_q6k_gemv_argmax_noalloc": (i32, [vp, vp, vp, i32, i32, i64, vp, vp]),
    "ptm_quant_gemv": (i32, [u32, vp, vp, vp, i32, i32, i64, i32, vp]),
    "ptm_q4k_fused_gate_up_gemv": (i32, [vp, vp, vp, vp, vp, i32, i32, i32, i64, vp]),
    "ptm_q4k_fused_qkv_gemv": (i32, [vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, i64, vp]),
    "ptm_q4k_fused_rmsnorm_gemv": (i32, [vp, vp, vp, vp, i32, i32, i64, f32, i32, vp]),
    "ptm_q4k_fused_rmsnorm_qkv_gemv": (i32, [vp, vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, i64, f32, i32, vp]),
    "ptm_q4k_fused_rmsnorm_gate_up_gemv": (i32, [vp, vp, vp, vp, vp, vp, i32, i32, i32, i64, f32, i32, vp]),
    "ptm_q4k_fused_rmsnorm_gate_up_silu": (i32, [vp, vp, vp, vp, vp, i32, i32, i64, f32, i32, vp]),
    "ptm_rms_norm": (i32, [vp, vp, vp, i32, i32, f32, i32, vp, vp]),
    "ptm_per_head_rms_norm": (i32, [vp, vp, i32, i32, i32, f32, i32, vp]),
    "ptm_qknorm_rope_kvwrite": (i32, [vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, vp, i32, f32, vp, f32, i32, i32, i32, vp]),
    "ptm_qknorm_rope_kvwrite_pos": (i32, [vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, i64, i32, f32, vp, f32, i32, i32, i32, vp]),
    "ptm_flash_decode_pos": (i32, [vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, f32, i32, vp]),
    "ptm_mul_scalar": (i32, [vp, f32, vp, i64, vp]),
    "ptm_kv_cache_write": (i32, [vp, vp, i64, i64, i64, vp]),
    "ptm_concat_rows": (i32, [vp, vp, vp, i64, i64, i64, vp]),
    "ptm_rope": (i32, [vp, i32, i32, i32, i32, f32, vp, i32, i32, vp]),
    "ptm_f32_gemv": (i32, [vp, vp, vp, i32, i32, i32, vp]),
    "ptm_f16_gemv": (i32, [vp, vp, vp, i32, i32, i32, i32, vp]),
    "ptm_rope_table_host": (i32, [vp, i32, i32, f32]),
    "ptm_rope_table_host_scaled": (i32, [vp, i32, i32, f32, f32]),
    "ptm_rope_table_host_factors": (i32, [vp, i32, i32, f32, f32, vp, vp, i32, f32]),
    "ptm_fp16_kv_cache_write": (i32, [vp, vp, i64, i64, i64, vp]),
    "ptm_flash_decode_kv_chunk_size": (i32, []),
    "ptm_flash_decode_num_splits": (i32, [i32]),
    "ptm_flash_decode": (i32, [vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, vp, i32, f32, i32, vp]),
    "ptm_attn_decode_fused": (i32, [vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, vp, i32, f32, f32, i32, i32, i32, vp]),
    "ptm_flash_decode_window": (i32, [vp, vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, vp, i32, f32, i32, i32, vp]),
    "ptm_attn_decode_fused_window": (i32, [vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, vp, i32, f32, f32, i32, i32, i32, i32, vp]),
    "ptm_silu_mul": (i32, [vp, vp, vp, i64, vp]),
    "ptm_embedding_row": (i32, [vp, vp, vp, i32, vp]),
    "ptm_embedding_row_q6k": (i32, [vp, vp, vp, i32, i64, vp]),
    "ptm_argmax": (i32, [vp, vp, i64, vp]),
    "ptm_add": (i32, [vp, vp, vp, i64, vp]),
    "ptm_add_qkv_bias": (i32, [vp, vp, vp, vp, vp, vp, i32, i32, i32, vp]),
    "ptm_gelu_mul": (i32, [vp, vp, vp, i64, vp]),
    "ptm_rms_norm_add": (i32, [vp, vp, vp, i32, i32, f32, i32, vp]),
    "ptm_scale": (i32, [vp, f32, i64, vp]),
    "ptm_prefill_attention_window": (i32, [vp, vp, vp, vp, i32, i32, i32, i32, i64, i32, f32, i32, i32, vp]),
    "ptm_copy": (i32, [vp, vp, i64, vp]),
    "ptm_qgemm_workspace_bytes": (i64, [i32, i32]),
    "ptm_qgemm_q4k": (i32, [vp, vp, vp, i32, i32, i32, i64, vp, vp]),
    "ptm_qgemm_q6k": (i32, [vp, vp, vp, i32, i32, i32, i64, vp, vp]),
    "ptm_qgemm_f16_workspace_bytes": (i64, [i32, i32]),
    "ptm_qgemm_f16": (i32, [u32, vp, vp, vp, i32, i32, i32, i64, vp, vp]),
    "ptm_decode_create": (i32, [C.POINTER(DecodeConfig), C.POINTER(vp)]),
    "ptm_decode_destroy": (None, [vp]),
    "ptm_decode_set_past_len": (i32, [vp, i64]),
    "ptm_decode_reserve_prefill": (i32, [vp, i32]),
    "ptm_decode_step": (i32, [vp, i32, C.POINTER(i64)]),
    "ptm_decode_greedy": (i32, [vp, i32, i32, C.POINTER(i64)]),
    "ptm_decode_step_trace": (i32, [vp, i32, C.POINTER(i64), vp]),
    "ptm_decode_prefill": (i32, [vp, C.POINTER(C.c_int32), i32, i32, C.POINTER(i64)]),
    "ptm_qgemm_f16_f32_workspace_bytes": (i64, [i32, i32, i32]),
    "ptm_qgemm_f16_f32": (i32, [u32, vp, vp, vp, i32, i32, i32, i64, vp, i32, vp]),
    "ptm_embedding_rows": (i32, [vp, vp, i64, vp, i32, i32, i32, vp, vp]),
    "ptm_qknorm_rope_kvwrite_rows": (i32, [vp, vp, vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, i64, i32, f32, i32, i32, i32, vp]),
    "ptm_prefill_attention": (i32, [vp, vp, vp, vp, i32, i32, i32, i32, i64, i32, f32, i32, vp]),
    "ptm_decode_generate": (i32, [vp, C.POINTER(C.c_int32), i32, C.POINTER(Sampling), C.POINTER(f32), i32, C.POINTER(C.c_int32),
                                  i32, C.POINTER(i64), C.POINTER(i32)]),
    "ptm_decode_sampling_begin": (i32, [vp, C.POINTER(Sampling)]),
    "ptm_decode_sample": (i32, [vp, i32, i32, C.POINTER(f32), C.POINTER(i64)]),
    "ptm_sampler_workspace_bytes": (i64, []),
    "ptm_sample_token": (i32, [vp, i32, vp, C.POINTER(Sampling), vp, vp, vp, vp]),
    "ptm_mt19937_uniforms": (i32, [u32, i64, i64, C.POINTER(f32)]),
    "ptm_decode_graph_state": (i32, [vp, i32]),
    "ptm_decode_debug_fail_next_capture": (i32, [vp]),
    "ptm_decode_logits": (vp, [vp]),
    "ptm_decode_hidden": (vp, [vp]),
    "ptm_decode_stream": (vp, [vp]),
    "ptm_gguf_open": (i32, [C.c_char_p, C.POINTER(vp)]),
    "ptm_gguf_close": (None, [vp]),
    "ptm_gguf_version": (i32, [vp]),
    "ptm_gguf_alignment": (i64, [vp]),
    "ptm_gguf_n_tensors": (i64, [vp]),
    "ptm_gguf_tensor_at": (i32, [vp, i64, C.POINTER(GgufTensor)]),
    "ptm_gguf_find_tensor": (i32, [vp, C.c_char_p, C.POINTER(GgufTensor)]),
    "ptm_gguf_get_int": (i32, [vp, C.c_char_p, C.POINTER(i64)]),
    "ptm_gguf_get_float": (i32, [vp, C.c_char_p, C.POINTER(C.c_double)]),
    "ptm_gguf_get_string": (C.c_char_p, [vp, C.c_char_p]),
    "ptm_gguf_get_array": (i32, [vp, C.c_char_p, C.POINTER(u32), C.POINTER(i64)]),
    "ptm_gguf_array_string": (i32, [vp, C.c_char_p, i64, C.POINTER(vp), C.POINTER(i64)]),
    "ptm_gguf_array_data": (vp, [vp, C.c_char_p]),
    "ptm_tokenizer_create": (i32, [C.POINTER(C.c_char_p), C.POINTER(C.c_int32), C.c_int32, C.POINTER(C.c_char_p),
                                   C.POINTER(C.c_int32), C.c_int32, C.c_char_p, C.c_int32, C.c_int32, C.c_int32, C.c_int32,
                                   i32, C.POINTER(vp)]),
    "ptm_tokenizer_from_gguf": (i32, [vp, C.POINTER(vp)]),
    "ptm_tokenizer_free": (None, [vp]),
    "ptm_tokenizer_vocab_size": (C.c_int32, [vp]),
    "ptm_tokenizer_special_ids": (i32, [vp] + [C.POINTER(C.c_int32)] * 4),
    "ptm_tokenizer_encode": (i32, [vp, C.c_char_p, i64, i32, C.POINTER(C.c_int32), i64, C.POINTER(i64)]),
    "ptm_tokenizer_decode": (i32, [vp, C.POINTER(C.c_int32), i64, i32, C.c_char_p, i64, C.POINTER(i64)]),
    "ptm_tokenizer_token": (i32, [vp, C.c_int32, C.c_char_p, i64, C.POINTER(i64)]),
    "ptm_chat_template": (i32, [C.c_char_p, C.c_char_p, C.c_char_p, i32, C.c_char_p, C.c_char_p, i64, C.POINTER(i64)]),
    "ptm_model_load_gguf": (i32, [C.c_char_p, i32, i32, i32, C.POINTER(vp)]),
    "ptm_model_decoder": (vp, [vp]),
    "ptm_model_config": (i32, [vp, C.POINTER(DecodeConfig)]),
    "ptm_model_layer": (i32, [vp, i32, C.POINTER(Layer)]),
    "ptm_model_free": (None, [vp]),
}

_lib = None


def load():
    """Load the library and bind every declared symbol; raises if anything is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(f"{LIB_PATH} is not built: run `python -m prometorch_amd.build` (hipcc --offload-arch=gfx950)")
    L = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(L, name)  # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    _lib = L
    return L


def check(code: int, what: str) -> None:
    if code != 0:
        msg = load().ptm_strerror(code).decode()
        raise PtmError(code, f"{what}: {msg}")
