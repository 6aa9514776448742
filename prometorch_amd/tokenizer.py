"""Host-side wrapper of the tokenizer and chat template (ptm_tokenizer_*, ptm_chat_template), the counterpart of
GGUFTokenizer (reference: torch/io/tokenizer.h:24-643) and GGUFModel::apply_chat_template
(torch/io/gguf_model.h:4178-4236).  Text goes in and out as bytes: tokens are byte strings, not necessarily UTF-8."""
from __future__ import annotations

import ctypes as C

from . import _lib
from ._lib import check


def _b(x) -> bytes:
    return x if isinstance(x, (bytes, bytearray)) else str(x).encode("utf-8")


class Tokenizer:
    def __init__(self, handle):
        self.L = _lib.load()
        self.h = handle

    @classmethod
    def from_lists(cls, tokens, merges, model_type="gpt2", bos_id=1, eos_id=2, pad_id=-1, unk_id=0, add_bos=True):
        L = _lib.load()
        tk = [_b(t) for t in tokens]
        mg = [_b(m) for m in merges]
        ta = (C.c_char_p * max(1, len(tk)))(*tk)
        tl = (C.c_int32 * max(1, len(tk)))(*[len(t) for t in tk])
        ma = (C.c_char_p * max(1, len(mg)))(*mg)
        ml = (C.c_int32 * max(1, len(mg)))(*[len(m) for m in mg])
        h = C.c_void_p()
        check(L.ptm_tokenizer_create(ta, tl, len(tk), ma, ml, len(mg), _b(model_type), bos_id, eos_id, pad_id, unk_id,
                                     int(add_bos), C.byref(h)), "tokenizer_create")
        return cls(h)

    @classmethod
    def from_gguf(cls, gguf_file):
        """gguf_file: prometorch_amd.gguf.GGUFFile (tokenizer.ggml.* metadata)."""
        L = _lib.load()
        h = C.c_void_p()
        check(L.ptm_tokenizer_from_gguf(gguf_file.h, C.byref(h)), "tokenizer_from_gguf")
        return cls(h)

    @property
    def vocab_size(self) -> int:
        return self.L.ptm_tokenizer_vocab_size(self.h)

    def special_ids(self) -> dict:
        v = [C.c_int32() for _ in range(4)]
        check(self.L.ptm_tokenizer_special_ids(self.h, *[C.byref(x) for x in v]), "tokenizer_special_ids")
        return dict(zip(("bos", "eos", "pad", "unk"), (x.value for x in v)))

    def encode(self, text, use_bos: bool = True) -> list:
        t = _b(text)
        n = C.c_int64()
        cap = 4 * len(t) + 16
        buf = (C.c_int32 * cap)()
        rc = self.L.ptm_tokenizer_encode(self.h, t, len(t), int(use_bos), buf, cap, C.byref(n))
        if rc == -6:  # does not fit: n holds the needed size
            cap = n.value
            buf = (C.c_int32 * cap)()
            rc = self.L.ptm_tokenizer_encode(self.h, t, len(t), int(use_bos), buf, cap, C.byref(n))
        check(rc, "tokenizer_encode")
        return list(buf[:n.value])

    def decode(self, ids, skip_special: bool = True) -> bytes:
        a = (C.c_int32 * max(1, len(ids)))(*[int(i) for i in ids])
        n = C.c_int64()
        rc = self.L.ptm_tokenizer_decode(self.h, a, len(ids), int(skip_special), None, 0, C.byref(n))
        if rc not in (0, -6):
            check(rc, "tokenizer_decode")
        buf = C.create_string_buffer(max(1, n.value))
        check(self.L.ptm_tokenizer_decode(self.h, a, len(ids), int(skip_special), buf, n.value, C.byref(n)), "tokenizer_decode")
        return buf.raw[:n.value]

    def token(self, token_id: int) -> bytes:
        n = C.c_int64()
        buf = C.create_string_buffer(256)
        rc = self.L.ptm_tokenizer_token(self.h, token_id, buf, 256, C.byref(n))
        if rc == -6:
            buf = C.create_string_buffer(n.value)
            rc = self.L.ptm_tokenizer_token(self.h, token_id, buf, n.value, C.byref(n))
        check(rc, "tokenizer_token")
        return buf.raw[:n.value]

    def close(self) -> None:
        if getattr(self, "h", None):
            self.L.ptm_tokenizer_free(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def chat_template(architecture: str, prompt, model_name: str = "", system=None, no_think: bool = False) -> bytes:
    """system None: the reference's default system prompt; '' : no system turn."""
    L = _lib.load()
    n = C.c_int64()
    p = _b(prompt)
    sysb = None if system is None else _b(system)
    cap = len(p) + (len(sysb) if sysb else 64) + 512
    buf = C.create_string_buffer(cap)
    check(L.ptm_chat_template(_b(architecture), _b(model_name), sysb, int(no_think), p, buf, cap, C.byref(n)), "chat_template")
    return buf.raw[:n.value]
