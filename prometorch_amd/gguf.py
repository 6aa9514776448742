"""GGUF files: reader (ctypes over ptm_gguf_*) and the model loader
(ptm_model_load_gguf), the counterpart of GGUFReader + GGUFModel::load (reference:
torch/io/gguf_loader.h:386-630, torch/io/gguf_model.h:1177-1360)."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib
from ._lib import DecodeConfig, GgufTensor, Layer, check

F32, F16, Q4_K, Q6_K = 0, 1, 12, 14
_T_U32, _T_I32, _T_F32, _T_BOOL, _T_STR, _T_ARR, _T_U64 = 4, 5, 6, 7, 8, 9, 10


# ---------------------------------------------------------------------------------------------
# reader
# ---------------------------------------------------------------------------------------------
class GGUFFile:
    """Memory-mapped GGUF file; tensor data is exposed as numpy views of the mapping (valid until close)."""

    def __init__(self, path: str):
        self.L = _lib.load()
        h = C.c_void_p()
        check(self.L.ptm_gguf_open(path.encode(), C.byref(h)), f"gguf_open({path})")
        self.h = h

    @property
    def version(self) -> int:
        return self.L.ptm_gguf_version(self.h)

    @property
    def alignment(self) -> int:
        return self.L.ptm_gguf_alignment(self.h)

    def __len__(self) -> int:
        return self.L.ptm_gguf_n_tensors(self.h)

    def _wrap(self, t: GgufTensor) -> dict:
        data = None
        if t.nbytes >= 0:
            data = np.ctypeslib.as_array((C.c_uint8 * t.nbytes).from_address(t.data)) if t.nbytes else np.zeros(0, np.uint8)
        return {"name": t.name.decode(), "type": t.ggml_type, "dims": [t.dims[i] for i in range(t.n_dims)],
                "nbytes": t.nbytes, "data": data}

    def tensor(self, key) -> dict:
        t = GgufTensor()
        if isinstance(key, int):
            check(self.L.ptm_gguf_tensor_at(self.h, key, C.byref(t)), "gguf_tensor_at")
        else:
            check(self.L.ptm_gguf_find_tensor(self.h, key.encode(), C.byref(t)), f"gguf_find_tensor({key})")
        return self._wrap(t)

    def get_int(self, key: str) -> int:
        v = C.c_int64()
        check(self.L.ptm_gguf_get_int(self.h, key.encode(), C.byref(v)), f"gguf_get_int({key})")
        return v.value

    def get_float(self, key: str) -> float:
        v = C.c_double()
        check(self.L.ptm_gguf_get_float(self.h, key.encode(), C.byref(v)), f"gguf_get_float({key})")
        return v.value

    def get_string(self, key: str):
        s = self.L.ptm_gguf_get_string(self.h, key.encode())
        return None if s is None else s.decode()

    def get_array(self, key: str):
        """Array-valued metadata: a list of bytes for string arrays, a numpy array for numeric ones."""
        et, n = C.c_uint32(), C.c_int64()
        check(self.L.ptm_gguf_get_array(self.h, key.encode(), C.byref(et), C.byref(n)), f"gguf_get_array({key})")
        if et.value == _T_STR:
            out = []
            p, ln = C.c_void_p(), C.c_int64()
            for i in range(n.value):
                check(self.L.ptm_gguf_array_string(self.h, key.encode(), i, C.byref(p), C.byref(ln)), "gguf_array_string")
                out.append(C.string_at(p.value, ln.value) if ln.value else b"")
            return out
        dt = {0: np.uint8, 1: np.int8, 2: np.uint16, 3: np.int16, 4: np.uint32, 5: np.int32, 6: np.float32, 7: np.uint8,
              10: np.uint64, 11: np.int64, 12: np.float64}[et.value]
        ptr = self.L.ptm_gguf_array_data(self.h, key.encode())
        if not n.value:
            return np.zeros(0, dt)
        raw = C.string_at(ptr, n.value * np.dtype(dt).itemsize)
        return np.frombuffer(raw, dt).copy()

    def close(self) -> None:
        if getattr(self, "h", None):
            self.L.ptm_gguf_close(self.h)
            self.h = None

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


# ---------------------------------------------------------------------------------------------
# model loader
# ---------------------------------------------------------------------------------------------
class GGUFModel:
    """A decoder created straight from a .gguf file; same stepping interface as decode.Decoder."""

    def __init__(self, path: str, max_seq: int, kv_fp16: bool = True, use_graph: bool = True):
        self.L = _lib.load()
        m = C.c_void_p()
        check(self.L.ptm_model_load_gguf(path.encode(), max_seq, int(kv_fp16), int(use_graph), C.byref(m)),
              f"model_load_gguf({path})")
        self.m = m
        self._path = path
        self.h = self.L.ptm_model_decoder(m)
        c = DecodeConfig()
        check(self.L.ptm_model_config(m, C.byref(c)), "model_config")
        self.cfg = {k: getattr(c, k) for k in ("vocab", "hidden", "n_layers", "n_heads", "n_kv_heads", "head_dim", "inter", "max_seq")}
        self.cfg.update(rope_base=c.rope_freq_base, eps=c.rms_eps, kv_fp16=bool(c.kv_fp16), tied=not bool(c.embedding_f32),
                        rope_interleaved=bool(c.rope_interleaved), rope_scale=c.rope_scale,
                        scale_embeddings=bool(c.scale_embeddings), ffn_gelu=bool(c.ffn_gelu), swa_window=c.swa_window,
                        swa_pattern=c.swa_pattern, rope_swa_base=c.rope_swa_freq_base)

    def layer(self, i: int) -> Layer:
        out = Layer()
        check(self.L.ptm_model_layer(self.m, i, C.byref(out)), "model_layer")
        return out

    def set_kv(self, layer: int, k16: np.ndarray, v16: np.ndarray) -> None:
        import torch
        Ld = self.layer(layer)
        dt = torch.float16 if self.cfg["kv_fp16"] else torch.float32
        for ptr, src in ((Ld.k_cache, k16), (Ld.v_cache, v16)):
            t = torch.from_numpy(np.ascontiguousarray(src)).to(device="cuda", dtype=dt).contiguous()
            nbytes = t.numel() * t.element_size()
            n4 = nbytes // 4  # rows are multiples of 4 bytes: reuse the fp32 copy kernel for the raw bytes
            check(self.L.ptm_copy(t.data_ptr(), ptr, n4, None), "copy")
        torch.cuda.synchronize()

    def set_past_len(self, n: int) -> None:
        check(self.L.ptm_decode_set_past_len(self.h, n), "decode_set_past_len")

    def step(self, token: int) -> int:
        out = C.c_int64()
        check(self.L.ptm_decode_step(self.h, token, C.byref(out)), "decode_step")
        return out.value

    def prefill(self, tokens, chunk_rows: int = 0) -> int:
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

    # the reference's stop strings besides the file's eos id (GGUFModel::is_stop_token, gguf_model.h:5132-5139)
    STOP_TOKENS = ("<|im_end|>", "<|endoftext|>", "<end_of_turn>", "<|eot_id|>", "</s>", "<|end|>")

    def chat(self, prompt: str, system=None, max_new: int = 256, temperature: float = 0.7, top_k: int = 40,
             top_p: float = 0.9, repeat_penalty: float = 1.1, seed: int = 42, no_think: bool = False) -> str:
        """One chat turn from text to text on a fresh context: the file's chat template and tokenizer, prompt prefill,
        sampled decode on the device until a stop token (promeserve/api_handlers.h:848-923), the reply decoded."""
        from . import ops
        from .tokenizer import Tokenizer, chat_template
        if getattr(self, "_tok", None) is None:
            self._file = GGUFFile(self._path)
            self._tok = Tokenizer.from_gguf(self._file)
            stops = {self._tok.special_ids()["eos"]}
            for t in self.STOP_TOKENS:
                ids = self._tok.encode(t, use_bos=False)
                if len(ids) == 1:
                    stops.add(ids[0])
            self._stops = sorted(i for i in stops if i >= 0)
        arch = self._file.get_string("general.architecture")
        name = self._file.get_string("general.name") or ""
        ids = self._tok.encode(chat_template(arch, prompt, model_name=name, system=system, no_think=no_think))
        room = self.cfg["max_seq"] - len(ids)
        if room <= 0:
            raise ValueError("prompt of %d tokens does not fit a context of %d" % (len(ids), self.cfg["max_seq"]))
        self.set_past_len(0)
        out = self.generate(ids, ops.mt19937_uniforms(seed, 0, min(max_new, room)), temperature, top_k, top_p,
                            repeat_penalty, stop_ids=self._stops)
        return self._tok.decode(out).decode("utf-8", errors="replace")

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

    def logits(self) -> np.ndarray:
        import torch
        out = torch.empty(self.cfg["vocab"], dtype=torch.float32, device="cuda")
        check(self.L.ptm_copy(self.L.ptm_decode_logits(self.h), out.data_ptr(), self.cfg["vocab"], None), "copy")
        torch.cuda.synchronize()
        return out.cpu().numpy()

    def close(self) -> None:
        if getattr(self, "_tok", None) is not None:
            self._tok.close()
            self._file.close()
            self._tok = self._file = None
        if getattr(self, "m", None):
            self.L.ptm_model_free(self.m)
            self.m = None
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
