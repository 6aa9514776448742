"""TEST INFRASTRUCTURE ONLY: ctypes bindings for oracle/libptm_oracle.so (this repo's CPU
restatement) and, where it has been built, oracle/_ref/libptm_ref.so (the reference's own
CPU code compiled from the reference checkout).  Imported by tests/, the smoke check and the
cpu_baseline leg of the benchmark; never by the product package."""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(_HERE, "libptm_oracle.so")
REF_SO = os.path.join(_HERE, "_ref", "libptm_ref.so")

_vp, _i64, _i32, _u32, _f32 = C.c_void_p, C.c_int64, C.c_int, C.c_uint32, C.c_float


def build(ref: bool = True) -> None:
    """Compile the C restatement, and the reference build when its checkout is present."""
    subprocess.check_call(["make", "-s", "-C", _HERE, "oracle"])
    if ref and os.path.isdir(os.environ.get("PTM_REF", "/root/reference")):
        subprocess.check_call(["make", "-s", "-C", _HERE, "ref", "REF=" + os.environ.get("PTM_REF", "/root/reference")])


def _p(a: np.ndarray):
    return a.ctypes.data_as(_vp)


class QW(C.Structure):
    _fields_ = [("data", _vp), ("type", _u32), ("rows", _i64), ("cols", _i64), ("stride", _i64)]


class Layer(C.Structure):
    _fields_ = [(n, QW) for n in ("q", "k", "v", "o", "gate", "up", "down")] + \
               [(n, _vp) for n in ("attn_norm", "ffn_norm", "q_norm", "k_norm", "k_cache", "v_cache",
                                   "q_bias", "k_bias", "v_bias", "post_attn_norm", "post_ffn_norm")]


class Model(C.Structure):
    _fields_ = [(n, _i64) for n in ("vocab", "hidden", "n_layers", "n_heads", "n_kv_heads", "head_dim", "inter", "max_seq")] + \
               [("rope_base", _f32), ("eps", _f32), ("kv_fp16", _i32), ("embedding", _vp),
                ("layers", C.POINTER(Layer)), ("out_norm", _vp), ("lm_head", QW), ("seq_len", _i64), ("rope_interleaved", _i32),
                ("rope_scale", _f32), ("scale_embeddings", _i32), ("ffn_gelu", _i32), ("swa_window", _i64),
                ("swa_pattern", _i64), ("rope_swa_base", _f32), ("rope_factors_short", _vp), ("rope_factors_long", _vp),
                ("rope_orig_ctx", _i64), ("rope_attn_factor", _f32)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(ORACLE_SO):
            build(ref=False)
        L = C.CDLL(ORACLE_SO)
        L.po_fp16_to_fp32.restype = _f32
        L.po_fp16_to_fp32.argtypes = [C.c_uint16]
        L.po_fp32_to_fp16.restype = C.c_uint16
        L.po_fp32_to_fp16.argtypes = [_f32]
        L.po_argmax.restype = _i64
        L.po_decode_step.restype = _i64
        L.po_decode_step.argtypes = [C.POINTER(Model), _i64, _vp, _vp]
        L.po_num_threads.restype = _i32
        for name in ("po_q4k_gemv", "po_q4k_gemv_f32", "po_q6k_gemv", "po_q6k_gemv_f32"):
            getattr(L, name).argtypes = [_vp, _vp, _vp, _i64, _i64, _i64]
        L.po_cpu_quant_gemv.argtypes = [_u32, _vp, _vp, _vp, _i64, _i64, _i64]
        for name in ("po_dequantize_q4_k", "po_dequantize_q6_k", "po_dequantize_q8_0", "po_dequantize_q5_k"):
            getattr(L, name).argtypes = [_vp, _vp, _i64]
        L.po_quantize_x_q8.argtypes = [_vp, _i64, _vp, _vp, _vp]
        L.po_q4k_row_isums.argtypes = [_vp, _vp, _i64, _vp]
        L.po_rmsnorm_seq.argtypes = [_vp, _vp, _f32, _i32, _i64, _vp]
        L.po_rmsnorm_vec.argtypes = [_vp, _vp, _f32, _i32, _i64, _vp]
        L.po_rope_precompute.argtypes = [_vp, _vp, _i64, _i64, _f32]
        L.po_rope_precompute_scaled.argtypes = [_vp, _vp, _i64, _i64, _f32, _f32]
        L.po_rope_apply_neox.argtypes = [_vp, _vp, _vp, _vp, _i64, _i64, _i64]
        L.po_rope_apply_norm.argtypes = [_vp, _vp, _vp, _vp, _i64, _i64, _i64]
        L.po_exp256.argtypes = [_vp, _vp, _i64]
        L.po_attn_head.argtypes = [_vp, _vp, _vp, _i64, _i64, _i64, _f32, _vp, _vp]
        L.po_silu_mul.argtypes = [_vp, _vp, _i64]
        L.po_argmax.argtypes = [_vp, _i64]
        L.po_get_scale_min_k4.argtypes = [_i32, _vp, _vp, _vp]
        L.po_mt19937_seed.argtypes = [_vp, _u32]
        L.po_mt19937_next.restype = _u32
        L.po_mt19937_next.argtypes = [_vp]
        L.po_uniform01.restype = _f32
        L.po_uniform01.argtypes = [_vp]
        L.po_repetition_penalty.argtypes = [_vp, _i64, _vp, _i64, _f32]
        L.po_sample_token.restype = _i32
        L.po_sample_token.argtypes = [_vp, _i64, _f32, _i32, _f32, _f32, _vp, _vp]
        _lib = L
    return _lib


# ---- array-level helpers ---------------------------------------------------------------
def fp16_to_fp32(h: int) -> float:
    return lib().po_fp16_to_fp32(h)


# ggml type id -> (bytes per block, values per block): gguf_dequant.h:29-58
BLOCK = {12: (144, 256), 14: (210, 256), 13: (176, 256), 8: (34, 32), 6: (22, 32)}
_DEQUANT = {12: "dequantize_q4_k", 14: "dequantize_q6_k", 8: "dequantize_q8_0", 13: "dequantize_q5_k"}


def dequant(qtype: int, raw: np.ndarray) -> np.ndarray:
    raw = np.ascontiguousarray(raw, dtype=np.uint8).reshape(-1)
    bb, per = BLOCK[qtype]
    n = raw.size // bb * per
    out = np.empty(n, dtype=np.float32)
    getattr(lib(), "po_" + _DEQUANT[qtype])(_p(raw), _p(out), n)
    return out


def ref_dequant(qtype: int, raw: np.ndarray) -> np.ndarray:
    """The compiled reference's dequantiser (only where oracle/_ref is built)."""
    raw = np.ascontiguousarray(raw, dtype=np.uint8).reshape(-1)
    bb, per = BLOCK[qtype]
    n = raw.size // bb * per
    out = np.empty(n, dtype=np.float32)
    fn = getattr(ref(), "ref_" + _DEQUANT[qtype])
    fn.argtypes = [_vp, _vp, _i64]
    fn(_p(raw), _p(out), n)
    return out


def quantize_x_q8(x: np.ndarray):
    x = np.ascontiguousarray(x, dtype=np.float32)
    K = x.size
    d = np.empty(K // 32, np.float32)
    s = np.empty(K // 32, np.float32)
    q = np.empty(K, np.int8)
    lib().po_quantize_x_q8(_p(x), K, _p(d), _p(s), _p(q))
    return d, s, q


def gemv(qtype: int, W: np.ndarray, x: np.ndarray, variant: str = "ref") -> np.ndarray:
    """variant 'ref': what the reference's AVX2 build computes (Q8 activations for Q4_K,
    fp32 for Q6_K); 'f32': exact-math fp32-activation cross-check."""
    W = np.ascontiguousarray(W, dtype=np.uint8)
    N, stride = W.shape
    K = x.size if qtype not in (12, 14) else stride // BLOCK[qtype][0] * 256
    x = np.ascontiguousarray(x, dtype=np.float32)
    assert x.size == K and stride >= K // BLOCK[qtype][1] * BLOCK[qtype][0]
    y = np.empty(N, np.float32)
    if variant == "ref":
        lib().po_cpu_quant_gemv(qtype, _p(W), _p(x), _p(y), K, N, stride)
    else:
        fn = lib().po_q4k_gemv_f32 if qtype == 12 else lib().po_q6k_gemv_f32
        fn(_p(W), _p(x), _p(y), K, N, stride)
    return y


def q4k_row_isums(row: np.ndarray, qs: np.ndarray) -> np.ndarray:
    K = qs.size
    out = np.empty(K // 32, np.int32)
    lib().po_q4k_row_isums(_p(np.ascontiguousarray(row)), _p(np.ascontiguousarray(qs)), K, _p(out))
    return out


def rmsnorm(x, gamma, eps, seq=False):
    x = np.ascontiguousarray(x, np.float32)
    gamma = np.ascontiguousarray(gamma, np.float32)
    out = np.empty_like(x)
    (lib().po_rmsnorm_seq if seq else lib().po_rmsnorm_vec)(_p(x), _p(gamma), eps, 0, x.size, _p(out))
    return out


def rope_tables(pos, head_dim, base, scale=1.0, factors=None, attn_factor=1.0):
    c = np.empty(head_dim // 2, np.float32)
    s = np.empty(head_dim // 2, np.float32)
    L = lib()
    L.po_rope_precompute_factors.argtypes = [_vp, _vp, _i64, _i64, _f32, _f32, _vp, _f32]
    f = None if factors is None else np.ascontiguousarray(factors, np.float32)
    L.po_rope_precompute_factors(_p(c), _p(s), pos, head_dim, base, scale, None if f is None else _p(f), attn_factor)
    return c, s


def rope_norm(q, k, c, s, n_heads, n_kv_heads, head_dim):
    """Interleaved pairs (2d, 2d + 1): llama / mistral."""
    q = np.array(q, np.float32, copy=True)
    k = np.array(k, np.float32, copy=True)
    lib().po_rope_apply_norm(_p(q), _p(k), _p(c), _p(s), n_heads, n_kv_heads, head_dim)
    return q, k


def rope_neox(q, k, c, s, n_heads, n_kv_heads, head_dim):
    q = np.array(q, np.float32, copy=True)
    k = np.array(k, np.float32, copy=True)
    lib().po_rope_apply_neox(_p(q), _p(k), _p(c), _p(s), n_heads, n_kv_heads, head_dim)
    return q, k


def exp256(x):
    x = np.ascontiguousarray(x, np.float32)
    assert x.size % 8 == 0
    out = np.empty_like(x)
    lib().po_exp256(_p(x), _p(out), x.size // 8)
    return out


def attn_head(q, kc, vc, T, kv_dim, head_dim, scale, col0=0, t_start=0):
    """kc, vc: fp32 [>=T, kv_dim]; col0 = kv_head*head_dim; positions before t_start are masked."""
    q = np.ascontiguousarray(q, np.float32)
    sc = np.empty(T + 8, np.float32)
    out = np.empty(head_dim, np.float32)
    L = lib()
    L.po_attn_head_window.argtypes = [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _f32, _vp, _vp]
    L.po_attn_head_window(_p(q), C.c_void_p(kc.ctypes.data + 4 * col0), C.c_void_p(vc.ctypes.data + 4 * col0),
                          T, t_start, kv_dim, head_dim, scale, _p(sc), _p(out))
    return out


def silu_mul(gate, up):
    g = np.array(gate, np.float32, copy=True)
    up = np.ascontiguousarray(up, np.float32)
    lib().po_silu_mul(_p(g), _p(up), g.size)
    return g


def argmax(x):
    x = np.ascontiguousarray(x, np.float32)
    return int(lib().po_argmax(_p(x), x.size))


def _qw(qtype, W):
    W = np.ascontiguousarray(W, np.uint8)
    N, stride = W.shape
    return QW(W.ctypes.data, qtype, N, stride // BLOCK[qtype][0] * BLOCK[qtype][1], stride), W


class MT19937:
    """std::mt19937 and the uniform float draw the reference's sampler makes from it."""

    def __init__(self, seed: int = 42):
        self.state = (C.c_uint32 * 625)()
        lib().po_mt19937_seed(self.state, seed)

    def next_u32(self) -> int:
        return int(lib().po_mt19937_next(self.state))

    def uniform01(self) -> float:
        return float(lib().po_uniform01(self.state))


def repetition_penalty(logits, generated, penalty):
    out = np.array(logits, np.float32, copy=True)
    g = np.ascontiguousarray(generated, np.int32)
    lib().po_repetition_penalty(_p(out), out.size, _p(g), g.size, penalty)
    return out


def sample_token(logits, temperature, top_k, top_p, r, want_probs=False):
    """-> (token, gap[, probs]); gap = distance from r to the nearest edge of the token's CDF interval."""
    x = np.ascontiguousarray(logits, np.float32)
    gap = C.c_float()
    probs = np.empty(x.size, np.float32) if want_probs else None
    tok = int(lib().po_sample_token(_p(x), x.size, temperature, top_k, top_p, r, _p(probs) if want_probs else None,
                                    C.byref(gap)))
    return (tok, gap.value, probs) if want_probs else (tok, gap.value)


class OracleModel:
    """Host-side model for po_decode_step; keeps every numpy buffer alive."""

    def __init__(self, cfg: dict, layers: list, head: dict, max_seq: int, kv_fp16: bool, embedding=None):
        """cfg may carry 'rope_interleaved' (llama-style rotation pairs); layers without 'q_norm' / 'k_norm' have no QK-norm;
        layers with 'q_bias', 'k_bias', 'v_bias' add them to the projections (qwen2)."""
        self.cfg = cfg
        self._keep = []
        kvd = cfg["n_kv_heads"] * cfg["head_dim"]
        self.layers = (Layer * cfg["n_layers"])()
        self.k_cache, self.v_cache = [], []
        for i, L in enumerate(layers):
            for name in ("q", "k", "v", "o", "gate", "up", "down"):
                qt, W = L[name]
                qw, Wc = _qw(qt, W)
                self._keep.append(Wc)
                setattr(self.layers[i], name, qw)
            for name in ("attn_norm", "ffn_norm", "q_norm", "k_norm", "q_bias", "k_bias", "v_bias", "post_attn_norm",
                         "post_ffn_norm"):
                if L.get(name) is None:
                    setattr(self.layers[i], name, None)
                    continue
                a = np.ascontiguousarray(L[name], np.float32)
                self._keep.append(a)
                setattr(self.layers[i], name, a.ctypes.data)
            kc = np.zeros((max_seq, kvd), np.float32)
            vc = np.zeros((max_seq, kvd), np.float32)
            self.k_cache.append(kc)
            self.v_cache.append(vc)
            self.layers[i].k_cache = kc.ctypes.data
            self.layers[i].v_cache = vc.ctypes.data
        lm, lmW = _qw(head.get("lm_head_type", 14), head["lm_head"])
        on = np.ascontiguousarray(head["out_norm"], np.float32)
        self._keep += [lmW, on]
        self.m = Model()
        for k in ("vocab", "hidden", "n_layers", "n_heads", "n_kv_heads", "head_dim", "inter"):
            setattr(self.m, k, cfg[k])
        self.m.max_seq = max_seq
        self.m.rope_base = cfg["rope_base"]
        self.m.eps = cfg["eps"]
        self.m.kv_fp16 = 1 if kv_fp16 else 0
        if embedding is not None:
            embedding = np.ascontiguousarray(embedding, np.float32)
            self._keep.append(embedding)
            self.m.embedding = embedding.ctypes.data
        else:
            self.m.embedding = None
        self.m.layers = self.layers
        self.m.out_norm = on.ctypes.data
        self.m.lm_head = lm
        self.m.seq_len = 0
        self.m.rope_interleaved = int(bool(cfg.get("rope_interleaved", False)))
        self.m.rope_scale = float(cfg.get("rope_scale", 1.0))
        self.m.scale_embeddings = int(bool(cfg.get("scale_embeddings", False)))
        self.m.ffn_gelu = int(bool(cfg.get("ffn_gelu", False)))
        self.m.swa_window = int(cfg.get("swa_window", 0))
        self.m.swa_pattern = int(cfg.get("swa_pattern", 0))
        self.m.rope_swa_base = float(cfg.get("rope_swa_base", 10000.0))
        for key in ("rope_factors_short", "rope_factors_long"):   # phi3 LongRoPE
            if cfg.get(key) is not None:
                f = np.ascontiguousarray(cfg[key], np.float32)
                self._keep.append(f)
                setattr(self.m, key, f.ctypes.data)
        self.m.rope_orig_ctx = int(cfg.get("rope_orig_ctx", 0))
        self.m.rope_attn_factor = float(cfg.get("rope_attn_factor", 1.0))
        self.logits = np.empty(cfg["vocab"], np.float32)
        self.hidden = np.empty(cfg["hidden"], np.float32)

    def set_kv(self, layer, k16, v16):
        n = k16.shape[0]
        self.k_cache[layer][:n] = k16.astype(np.float32)
        self.v_cache[layer][:n] = v16.astype(np.float32)
        self.m.seq_len = n

    def step(self, token: int) -> int:
        return int(lib().po_decode_step(C.byref(self.m), token, _p(self.logits), _p(self.hidden)))

    def step_trace(self, token: int):
        """One step that also returns the residual stream after every layer's attention branch and feed-forward branch:
        (token, trace[n_layers, 2, hidden])."""
        L = lib()
        L.po_decode_step_trace.restype = _i64
        trace = np.empty((self.cfg["n_layers"], 2, self.cfg["hidden"]), np.float32)
        tok = int(L.po_decode_step_trace(C.byref(self.m), token, _p(self.logits), _p(self.hidden), _p(trace)))
        return tok, trace


# ---- compiled reference (only where oracle/_ref has been built) --------------------------
_ref = None


def have_ref() -> bool:
    return os.path.exists(REF_SO)


def ref():
    global _ref
    if _ref is None:
        R = C.CDLL(REF_SO)
        R.ref_fp16_to_fp32.restype = _f32
        R.ref_fp16_to_fp32.argtypes = [C.c_uint16]
        R.ref_get_scale_min_k4.argtypes = [_i32, _vp, _vp, _vp]
        R.ref_dequantize_q4_k.argtypes = [_vp, _vp, _i64]
        R.ref_dequantize_q6_k.argtypes = [_vp, _vp, _i64]
        R.ref_quantize_x_q8.argtypes = [_vp, _i64, _vp, _vp, _vp]
        R.ref_cpu_quant_gemv.argtypes = [_u32, _vp, _vp, _vp, _i64, _i64, _i64]
        R.ref_q4k_gemv_scalar.argtypes = [_vp, _vp, _vp, _i64, _i64, _i64]
        R.ref_q6k_gemv_scalar.argtypes = [_vp, _vp, _vp, _i64, _i64, _i64]
        R.ref_fused_rmsnorm_gate_up.argtypes = [_vp, _vp, _f32, _i32, _u32, _vp, _u32, _vp, _vp, _vp,
                                                _i64, _i64, _i64, _i64, _i64]
        R.ref_rmsnorm_inplace.argtypes = [_vp, _vp, _f32, _i32, _i64]
        R.ref_rope_precompute.argtypes = [_vp, _vp, _i64, _i64, _f32]
        R.ref_rope_precompute_scaled.argtypes = [_vp, _vp, _i64, _i64, _f32, _f32]
        R.ref_model_set_rope_scale.argtypes = [_vp, _f32]
        R.ref_model_set_rope_factors.argtypes = [_vp, _vp, _i64, _vp, _i64, _i64, _f32]
        R.ref_rope_precompute_factors.argtypes = [_vp, _vp, _i64, _i64, _f32, _f32, _vp, _f32]
        R.ref_model_set_gemma.argtypes = [_vp, _i32, _i32, _i32, _i64, _i64, _f32]
        R.ref_rope_apply_neox.argtypes = [_vp, _vp, _vp, _vp, _i64, _i64, _i64]
        R.ref_rope_apply_norm.argtypes = [_vp, _vp, _vp, _vp, _i64, _i64, _i64]
        R.ref_model_set_arch.argtypes = [_vp, _i32, _i32]
        R.ref_exp256.argtypes = [_vp, _vp, _i64]
        R.ref_num_threads.restype = _i32
        R.ref_model_create.restype = _vp
        R.ref_model_create.argtypes = [_i64] * 7 + [_f32, _f32, _i64]
        R.ref_model_destroy.argtypes = [_vp]
        R.ref_model_set_weight.argtypes = [_vp, _i64, _i32, _vp, _u32, _i64, _i64]
        R.ref_model_set_norm.argtypes = [_vp, _i64, _i32, _vp, _i64]
        R.ref_model_set_output.argtypes = [_vp, _vp, _vp, _u32]
        R.ref_model_set_embedding.argtypes = [_vp, _vp]
        R.ref_model_set_kv.argtypes = [_vp, _i64, _vp, _vp, _i64]
        R.ref_model_get_kv_row.argtypes = [_vp, _i64, _i64, _vp, _vp]
        R.ref_model_put_kv_row.argtypes = [_vp, _i64, _i64, _vp, _vp]
        R.ref_model_seq_len.restype = _i64
        R.ref_model_seq_len.argtypes = [_vp]
        R.ref_model_decode.restype = _i64
        R.ref_model_decode.argtypes = [_vp, _i64, _vp]
        R.ref_sample_token.restype = _i32
        R.ref_sample_token.argtypes = [_vp, _vp, _i64, _f32, _i32, _f32]
        R.ref_tokenizer_load.restype = _vp
        R.ref_tokenizer_load.argtypes = [C.c_char_p]
        R.ref_tokenizer_free.argtypes = [_vp]
        R.ref_tokenizer_encode.restype = _i64
        R.ref_tokenizer_encode.argtypes = [_vp, C.c_char_p, _i64, _i32, _vp, _i64]
        R.ref_tokenizer_decode.restype = _i64
        R.ref_tokenizer_decode.argtypes = [_vp, _vp, _i64, _i32, C.c_char_p, _i64]
        R.ref_tokenizer_token.restype = _i64
        R.ref_tokenizer_token.argtypes = [_vp, _i32, C.c_char_p, _i64]
        R.ref_chat_template.restype = _i64
        R.ref_chat_template.argtypes = [C.c_char_p, C.c_char_p, C.c_char_p, C.c_char_p, _i64]
        R.ref_gguf_n_tensors.restype = _i64
        R.ref_gguf_n_tensors.argtypes = [C.c_char_p]
        R.ref_model_load_gguf.restype = _vp
        R.ref_model_load_gguf.argtypes = [C.c_char_p, _i64]
        R.ref_model_free_loaded.argtypes = [_vp]
        R.ref_model_describe.argtypes = [_vp, _vp, _vp, _vp]
        _ref = R
    return _ref


def ref_gemv(qtype, W, x):
    W = np.ascontiguousarray(W, np.uint8)
    N, stride = W.shape
    x = np.ascontiguousarray(x, np.float32)
    K = x.size
    y = np.empty(N, np.float32)
    ref().ref_cpu_quant_gemv(qtype, _p(W), _p(x), _p(y), K, N, stride)
    return y


LOADED_INT_FIELDS = ("vocab", "hidden", "n_layers", "n_heads", "n_kv_heads", "head_dim", "inter", "tied", "has_qk_norm",
                     "rope_neox", "scale_embeddings", "ffn_gelu", "has_post_norm", "swa_window", "swa_pattern", "use_quant_gemv")
LOADED_FLOAT_FIELDS = ("rope_base", "eps", "rope_scale", "rope_swa_base", "rope_swa_scale")


class RefLoadedModel:
    """The reference's GGUFModel::load on a .gguf file (its own metadata parser, tensor-name mapping and quantised-weight
    registration), stepped with forward_decode_cpu."""

    def __init__(self, path: str, max_seq: int):
        R = ref()
        self.h = R.ref_model_load_gguf(path.encode(), max_seq)
        if not self.h:
            raise RuntimeError("the reference could not load " + path)
        ints = np.zeros(16, np.int64)
        floats = np.zeros(5, np.float32)
        self.ints, self.floats = ints, floats
        n_layers = self._describe(None)
        self.types = np.zeros(7 * n_layers + 1, np.uint32)
        self._describe(self.types)
        self.cfg = dict(zip(LOADED_INT_FIELDS, (int(v) for v in self.ints)))
        self.cfg.update(zip(LOADED_FLOAT_FIELDS, (float(v) for v in self.floats)))
        self.logits = np.empty(self.cfg["vocab"], np.float32)

    def _describe(self, types):
        R = ref()
        scratch = np.zeros(7 * 4096 + 1, np.uint32) if types is None else types
        R.ref_model_describe(self.h, _p(self.ints), _p(self.floats), _p(scratch))
        return int(self.ints[2])

    def set_kv(self, layer, k16, v16):
        k = np.ascontiguousarray(k16.astype(np.float32))
        v = np.ascontiguousarray(v16.astype(np.float32))
        ref().ref_model_set_kv(self.h, layer, _p(k), _p(v), k.shape[0])

    def step(self, token: int) -> int:
        return int(ref().ref_model_decode(self.h, token, _p(self.logits)))

    def close(self):
        if self.h:
            ref().ref_model_free_loaded(self.h)
            self.h = None


class RefModel:
    """The reference's GGUFModel populated from numpy buffers and stepped with forward_decode_cpu."""

    def __init__(self, cfg, layers, head, max_seq, embedding):
        R = ref()
        self._keep = []
        self.cfg = cfg
        self.h = R.ref_model_create(cfg["vocab"], cfg["hidden"], cfg["n_layers"], cfg["n_heads"], cfg["n_kv_heads"],
                                    cfg["head_dim"], cfg["inter"], cfg["rope_base"], cfg["eps"], max_seq)
        if cfg.get("rope_interleaved") or layers[0].get("q_norm") is None:
            R.ref_model_set_arch(self.h, int(layers[0].get("q_norm") is not None), int(not cfg.get("rope_interleaved")))
        if cfg.get("rope_scale", 1.0) != 1.0:
            R.ref_model_set_rope_scale(self.h, float(cfg["rope_scale"]))
        if cfg.get("rope_orig_ctx", 0) > 0 or cfg.get("rope_attn_factor", 1.0) != 1.0:
            fs = np.ascontiguousarray(cfg.get("rope_factors_short", []), np.float32)
            fl = np.ascontiguousarray(cfg.get("rope_factors_long", []), np.float32)
            R.ref_model_set_rope_factors(self.h, _p(fs), fs.size, _p(fl), fl.size, int(cfg.get("rope_orig_ctx", 0)),
                                         float(cfg.get("rope_attn_factor", 1.0)))
        if any(cfg.get(k) for k in ("scale_embeddings", "ffn_gelu", "swa_window")) or layers[0].get("post_attn_norm") is not None:
            R.ref_model_set_gemma(self.h, int(bool(cfg.get("scale_embeddings"))), int(bool(cfg.get("ffn_gelu"))),
                                  int(layers[0].get("post_attn_norm") is not None), int(cfg.get("swa_window", 0)),
                                  int(cfg.get("swa_pattern", 0)), float(cfg.get("rope_swa_base", 10000.0)))
        names = ("q", "k", "v", "o", "gate", "up", "down")
        for i, L in enumerate(layers):
            for w, name in enumerate(names):
                qt, W = L[name]
                W = np.ascontiguousarray(W, np.uint8)
                self._keep.append(W)
                K = W.shape[1] // BLOCK[qt][0] * BLOCK[qt][1]
                R.ref_model_set_weight(self.h, i, w, _p(W), qt, W.shape[0], K)
            for w, name in enumerate(("attn_norm", "ffn_norm", "q_norm", "k_norm", "q_bias", "k_bias", "v_bias",
                                      "post_attn_norm", "post_ffn_norm")):
                if L.get(name) is None:
                    continue
                a = np.ascontiguousarray(L[name], np.float32)
                R.ref_model_set_norm(self.h, i, w, _p(a), a.size)
        lm = np.ascontiguousarray(head["lm_head"], np.uint8)
        on = np.ascontiguousarray(head["out_norm"], np.float32)
        self._keep += [lm, on]
        R.ref_model_set_output(self.h, _p(on), _p(lm), head.get("lm_head_type", 14))
        emb = np.ascontiguousarray(embedding, np.float32)
        R.ref_model_set_embedding(self.h, _p(emb))
        self.logits = np.empty(cfg["vocab"], np.float32)

    def set_kv(self, layer, k16, v16):
        k = np.ascontiguousarray(k16.astype(np.float32))
        v = np.ascontiguousarray(v16.astype(np.float32))
        ref().ref_model_set_kv(self.h, layer, _p(k), _p(v), k.shape[0])

    def round_last_kv_to_fp16(self):
        """Round the K/V rows appended by the last step to fp16 precision, which is what an
        fp16 KV cache holds (the reference's CPU cache itself stays fp32)."""
        R = ref()
        pos = R.ref_model_seq_len(self.h) - 1
        kvd = self.cfg["n_kv_heads"] * self.cfg["head_dim"]
        k = np.empty(kvd, np.float32)
        v = np.empty(kvd, np.float32)
        for i in range(self.cfg["n_layers"]):
            R.ref_model_get_kv_row(self.h, i, pos, _p(k), _p(v))
            k2 = k.astype(np.float16).astype(np.float32)
            v2 = v.astype(np.float16).astype(np.float32)
            R.ref_model_put_kv_row(self.h, i, pos, _p(k2), _p(v2))

    def step(self, token):
        return int(ref().ref_model_decode(self.h, token, _p(self.logits)))

    def close(self):
        if self.h:
            ref().ref_model_destroy(self.h)
            self.h = None
