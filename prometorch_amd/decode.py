"""Host-side wrapper of the decode runtime (ptm_decode_*), the counterpart of
GGUFModel::load_quantized_to_cuda + forward_decode + greedy generate
(reference: torch/io/gguf_model.h:1177-1360, :2575-3113, :4737-4901).

Weights are uploaded verbatim as raw super-blocks; torch is used only to own device memory."""
from __future__ import annotations

import ctypes as C

import numpy as np
import torch

from . import _lib
from ._lib import DecodeConfig, Layer, QWeight, check

_NAMES = ("q", "k", "v", "o", "gate", "up", "down")


def _upload_bytes(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.uint8)).cuda()


class Decoder:
    """Greedy batch-1 decoder over caller-provided quantised weights.

    layers: list of dicts with (qtype, uint8[rows, stride]) per projection name and fp32 norm
    vectors 'attn_norm', 'ffn_norm', 'q_norm', 'k_norm' (the last two None for a model without QK-norm; optional
    'q_bias', 'k_bias', 'v_bias' added to the projections' outputs; optional 'post_attn_norm', 'post_ffn_norm' and the cfg keys
    'scale_embeddings', 'ffn_gelu', 'swa_window', 'swa_pattern', 'rope_swa_base', 'rope_scale' of a gemma-style model;
    cfg['rope_interleaved'] selects llama-style rotation pairs); head: {'lm_head': uint8 table (Q6_K unless 'lm_head_type' says otherwise),
    'out_norm': fp32}.  The token-embedding is the tied Q6_K table unless embedding_f32 is given."""

    def __init__(self, cfg: dict, layers: list, head: dict, max_seq: int, kv_fp16: bool = True,
                 use_graph: bool = True, embedding_f32=None, device: str = "cuda:0"):
        self.L = _lib.load()
        self.cfg = dict(cfg)
        self.max_seq = max_seq
        self.kv_fp16 = kv_fp16
        torch.cuda.set_device(device)
        self._keep = []
        kvd = cfg["n_kv_heads"] * cfg["head_dim"]
        kv_dtype = torch.float16 if kv_fp16 else torch.float32
        self.k_cache, self.v_cache = [], []
        arr = (Layer * cfg["n_layers"])()
        for i, Ld in enumerate(layers):
            for name in _NAMES:
                qt, W = Ld[name]
                t = _upload_bytes(W)
                self._keep.append(t)
                setattr(arr[i], name, QWeight(t.data_ptr(), qt, W.shape[0], _lib.weight_cols(qt, W.shape[1]), W.shape[1]))
            for name in ("attn_norm", "ffn_norm", "q_norm", "k_norm", "q_bias", "k_bias", "v_bias", "post_attn_norm",
                         "post_ffn_norm"):
                if Ld.get(name) is None:  # q_norm / k_norm: a model without QK-norm; biases: qwen2-style only
                    setattr(arr[i], name, None)
                    continue
                t = torch.from_numpy(np.ascontiguousarray(Ld[name], np.float32)).cuda()
                self._keep.append(t)
                setattr(arr[i], name, t.data_ptr())
            kc = torch.zeros(max_seq, kvd, dtype=kv_dtype, device="cuda")
            vc = torch.zeros(max_seq, kvd, dtype=kv_dtype, device="cuda")
            self.k_cache.append(kc)
            self.v_cache.append(vc)
            arr[i].k_cache = kc.data_ptr()
            arr[i].v_cache = vc.data_ptr()
        self._layers = arr
        lm = _upload_bytes(head["lm_head"])
        on = torch.from_numpy(np.ascontiguousarray(head["out_norm"], np.float32)).cuda()
        self._keep += [lm, on]
        c = DecodeConfig()
        for k in ("vocab", "hidden", "n_layers", "n_heads", "n_kv_heads", "head_dim", "inter"):
            setattr(c, k, cfg[k])
        c.max_seq = max_seq
        c.rope_freq_base = cfg["rope_base"]
        c.rms_eps = cfg["eps"]
        c.kv_fp16 = int(kv_fp16)
        c.use_graph = int(use_graph)
        c.rope_interleaved = int(bool(cfg.get("rope_interleaved", False)))
        c.rope_scale = float(cfg.get("rope_scale", 1.0))
        c.scale_embeddings = int(bool(cfg.get("scale_embeddings", False)))
        c.ffn_gelu = int(bool(cfg.get("ffn_gelu", False)))
        c.swa_window = int(cfg.get("swa_window", 0))
        c.swa_pattern = int(cfg.get("swa_pattern", 0))
        c.rope_swa_freq_base = float(cfg.get("rope_swa_base", 10000.0))
        for key in ("rope_factors_short", "rope_factors_long"):   # phi3 LongRoPE: host arrays, read by decode_create
            if cfg.get(key) is not None:
                f = np.ascontiguousarray(cfg[key], np.float32)
                self._keep.append(f)
                setattr(c, key, f.ctypes.data)
        c.rope_orig_ctx = int(cfg.get("rope_orig_ctx", 0))
        c.rope_attn_factor = float(cfg.get("rope_attn_factor", 1.0))
        if embedding_f32 is not None:
            e = embedding_f32 if isinstance(embedding_f32, torch.Tensor) else torch.from_numpy(embedding_f32)
            e = e.to(device="cuda", dtype=torch.float32).contiguous()
            self._keep.append(e)
            c.embedding_f32 = e.data_ptr()
        else:
            c.embedding_f32 = None
        c.layers = arr
        c.out_norm = on.data_ptr()
        c.lm_head = QWeight(lm.data_ptr(), head.get("lm_head_type", 14), cfg["vocab"], cfg["hidden"], head["lm_head"].shape[1])
        self._cfg = c
        torch.cuda.synchronize()
        h = C.c_void_p()
        check(self.L.ptm_decode_create(C.byref(c), C.byref(h)), "decode_create")
        self.h = h

    def set_kv(self, layer: int, k16: np.ndarray, v16: np.ndarray) -> None:
        """Prefill: write cache rows [0, n) (fp16 values; widened when the cache is fp32)."""
        n = k16.shape[0]
        self.k_cache[layer][:n].copy_(torch.from_numpy(k16).to(self.k_cache[layer].dtype))
        self.v_cache[layer][:n].copy_(torch.from_numpy(v16).to(self.v_cache[layer].dtype))

    def set_past_len(self, n: int) -> None:
        torch.cuda.synchronize()
        check(self.L.ptm_decode_set_past_len(self.h, n), "decode_set_past_len")

    def step(self, token: int) -> int:
        out = C.c_int64()
        check(self.L.ptm_decode_step(self.h, token, C.byref(out)), "decode_step")
        return out.value

    def step_trace(self, token: int):
        """One step as plain launches that also returns the residual stream after every layer's attention branch and after
        its feed-forward branch: (token, trace[n_layers, 2, hidden])."""
        trace = torch.empty(self.cfg["n_layers"], 2, self.cfg["hidden"], dtype=torch.float32, device="cuda")
        out = C.c_int64()
        check(self.L.ptm_decode_step_trace(self.h, token, C.byref(out), trace.data_ptr()), "decode_step_trace")
        return out.value, trace.cpu().numpy()

    def prefill(self, tokens, chunk_rows: int = 0) -> int:
        """Run the prompt through the model in row batches, appending its K/V rows; returns the greedy next token
        (GGUFModel::forward with use_cache, gguf_model.h:2510-2571)."""
        n = len(tokens)
        buf = (C.c_int32 * n)(*[int(t) for t in tokens])
        out = C.c_int64()
        check(self.L.ptm_decode_prefill(self.h, buf, n, chunk_rows, C.byref(out)), "decode_prefill")
        return out.value

    def generate(self, prompt, uniforms, temperature: float, top_k: int, top_p: float, repeat_penalty: float = 1.0,
                 stop_ids=()) -> list:
        """Prompt, then up to len(uniforms) sampled tokens, ending before the first stop token (the serving loop of
        promeserve/api_handlers.h:848-923 with everything but the token ids kept on the device)."""
        from ._lib import Sampling
        n, m, ns = len(prompt), len(uniforms), len(stop_ids)
        pa = (C.c_int32 * n)(*[int(t) for t in prompt])
        ua = (C.c_float * m)(*[float(u) for u in uniforms])
        sa = (C.c_int32 * max(1, ns))(*[int(t) for t in stop_ids])
        out = (C.c_int64 * m)()
        n_out = C.c_int()
        check(self.L.ptm_decode_generate(self.h, pa, n, Sampling(temperature, top_k, top_p, repeat_penalty), ua, m, sa, ns, out,
                                         C.byref(n_out)), "decode_generate")
        return list(out[:n_out.value])

    def sampling_begin(self, temperature: float, top_k: int, top_p: float, repeat_penalty: float = 1.0) -> None:
        """Start a sampled generation: store the parameters, forget previously generated tokens."""
        from ._lib import Sampling
        check(self.L.ptm_decode_sampling_begin(self.h, Sampling(temperature, top_k, top_p, repeat_penalty)),
              "decode_sampling_begin")

    def sample(self, token: int, uniforms) -> list:
        """len(uniforms) chained sampled steps from `token`, one uniform draw per step."""
        n = len(uniforms)
        u = (C.c_float * n)(*[float(x) for x in uniforms])
        buf = (C.c_int64 * n)()
        check(self.L.ptm_decode_sample(self.h, token, n, u, buf), "decode_sample")
        return list(buf)

    def greedy(self, first_token: int, n: int) -> list:
        buf = (C.c_int64 * n)()
        check(self.L.ptm_decode_greedy(self.h, first_token, n, buf), "decode_greedy")
        return list(buf)

    def _view(self, ptr: int, n: int) -> np.ndarray:
        out = torch.empty(n, dtype=torch.float32, device="cuda")
        _lib.check(self.L.ptm_copy(ptr, out.data_ptr(), n, None), "copy")
        torch.cuda.synchronize()
        return out.cpu().numpy()

    def logits(self) -> np.ndarray:
        return self._view(self.L.ptm_decode_logits(self.h), self.cfg["vocab"])

    def hidden(self) -> np.ndarray:
        return self._view(self.L.ptm_decode_hidden(self.h), self.cfg["hidden"])

    def close(self) -> None:
        if getattr(self, "h", None):
            self.L.ptm_decode_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
