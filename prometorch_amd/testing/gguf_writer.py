"""GGUF writer (v2 / v3, little endian) for tests, fixtures and benchmarks: no model file ships with the reference or this
repository, so synthetic ones are written with it.  Not part of the decode path."""
from __future__ import annotations

import struct

import numpy as np

from .. import _lib
from ..gguf import F32, Q6_K, _T_ARR, _T_BOOL, _T_F32, _T_I32, _T_STR, _T_U32, _T_U64


def _s(x) -> bytes:
    b = x if isinstance(x, bytes) else x.encode("utf-8")
    return struct.pack("<Q", len(b)) + b


def _kv(key: str, value) -> bytes:
    out = _s(key)
    if isinstance(value, bool):
        return out + struct.pack("<IB", _T_BOOL, int(value))
    if isinstance(value, int):
        return out + (struct.pack("<II", _T_U32, value) if 0 <= value < 2 ** 32 else struct.pack("<IQ", _T_U64, value))
    if isinstance(value, float):
        return out + struct.pack("<If", _T_F32, value)
    if isinstance(value, str):
        return out + struct.pack("<I", _T_STR) + _s(value)
    if isinstance(value, (list, tuple)):
        if all(isinstance(v, (str, bytes)) for v in value):
            return out + struct.pack("<IIQ", _T_ARR, _T_STR, len(value)) + b"".join(_s(v) for v in value)
        if all(isinstance(v, int) for v in value):
            return out + struct.pack("<IIQ", _T_ARR, _T_I32, len(value)) + struct.pack("<%di" % len(value), *value)
        return out + struct.pack("<IIQ", _T_ARR, _T_F32, len(value)) + struct.pack("<%df" % len(value), *value)
    raise TypeError(f"unsupported metadata value for {key}: {type(value)}")


def write_gguf(path: str, metadata: dict, tensors: list, alignment: int = 32, version: int = 3) -> None:
    """tensors: list of (name, ggml_type, dims, bytes-like) with dims[0] the contiguous dimension.
    Quantised matrices are passed as their raw super-blocks."""
    md = dict(metadata)
    if alignment != 32:
        md["general.alignment"] = alignment
    head = struct.pack("<IIQQ", 0x46554747, version, len(tensors), len(md))
    head += b"".join(_kv(k, v) for k, v in md.items())
    infos, blobs, off = b"", [], 0
    for name, gtype, dims, data in tensors:
        raw = np.ascontiguousarray(data).tobytes() if isinstance(data, np.ndarray) else bytes(data)
        infos += _s(name) + struct.pack("<I", len(dims)) + struct.pack("<%dQ" % len(dims), *dims) + struct.pack("<IQ", gtype, off)
        pad = (-len(raw)) % alignment
        blobs.append(raw + b"\0" * pad)
        off += len(raw) + pad
    pre = head + infos
    pre += b"\0" * ((-len(pre)) % alignment)
    with open(path, "wb") as f:
        f.write(pre)
        for b in blobs:
            f.write(b)


def model_to_gguf(path: str, cfg: dict, layers: list, head: dict, arch: str = "qwen3", tied: bool = True,
                  alignment: int = 32, tokenizer: dict | None = None, extra_metadata: dict | None = None) -> None:
    """Write a decoder (the dict form prometorch_amd.decode.Decoder takes) as a GGUF file with the
    tensor names and metadata keys a qwen3 GGUF carries.  tokenizer: tokenizer.ggml.* metadata to store
    (default: a three-token placeholder); extra_metadata: further keys, written as given."""
    md = {
        "general.architecture": arch, "general.name": "synthetic",
        f"{arch}.block_count": cfg["n_layers"], f"{arch}.embedding_length": cfg["hidden"],
        f"{arch}.feed_forward_length": cfg["inter"], f"{arch}.attention.head_count": cfg["n_heads"],
        f"{arch}.attention.head_count_kv": cfg["n_kv_heads"], f"{arch}.attention.key_length": cfg["head_dim"],
        f"{arch}.attention.value_length": cfg["head_dim"], f"{arch}.rope.freq_base": float(cfg["rope_base"]),
        f"{arch}.attention.layer_norm_rms_epsilon": float(cfg["eps"]), f"{arch}.context_length": 4096,
        "tokenizer.ggml.model": "gpt2", "tokenizer.ggml.tokens": ["a", "b", "c"], "tokenizer.ggml.token_type": [1, 1, 1],
    }
    if cfg.get("swa_window", 0) > 0:  # gemma3's alternating local / global layers
        md[f"{arch}.attention.sliding_window"] = int(cfg["swa_window"])
        if cfg.get("swa_pattern", 6) != 6:
            md[f"{arch}.attention.sliding_window_pattern"] = int(cfg["swa_pattern"])
        md[f"{arch}.rope.freq_base_swa"] = float(cfg.get("rope_swa_base", 10000.0))
    if cfg.get("rope_scale", 1.0) != 1.0:  # linear position scaling, the keys llama3 / qwen2 files use
        md[f"{arch}.rope.scaling.type"] = "linear"
        md[f"{arch}.rope.scaling.factor"] = float(cfg["rope_scale"])
    if tokenizer:
        md = {k: v for k, v in md.items() if not k.startswith("tokenizer.")}
        md.update(tokenizer)
    if extra_metadata:
        md.update(extra_metadata)
    H = cfg["hidden"]
    lm_type = head.get("lm_head_type", Q6_K)
    ts = [("token_embd.weight", lm_type, [H, cfg["vocab"]], head["lm_head"])]
    if not tied:
        ts.append(("output.weight", lm_type, [H, cfg["vocab"]], head["lm_head"]))
    ts.append(("output_norm.weight", F32, [H], np.asarray(head["out_norm"], np.float32)))
    names = {"q": "attn_q", "k": "attn_k", "v": "attn_v", "o": "attn_output", "gate": "ffn_gate", "up": "ffn_up", "down": "ffn_down"}
    for i, L in enumerate(layers):
        p = f"blk.{i}."
        ts.append((p + "attn_norm.weight", F32, [H], np.asarray(L["attn_norm"], np.float32)))
        for k, gname in names.items():
            qt, W = L[k]
            cols = _lib.weight_cols(qt, W.shape[1])
            ts.append((p + gname + ".weight", qt, [cols, W.shape[0]], W))
        if L.get("q_norm") is not None:  # absent in a llama-style model
            ts.append((p + "attn_q_norm.weight", F32, [cfg["head_dim"]], np.asarray(L["q_norm"], np.float32)))
            ts.append((p + "attn_k_norm.weight", F32, [cfg["head_dim"]], np.asarray(L["k_norm"], np.float32)))
        for key, gname in (("post_attn_norm", "post_attention_norm"), ("post_ffn_norm", "post_ffw_norm")):
            if L.get(key) is not None:  # gemma2 / gemma3
                ts.append((p + gname + ".weight", F32, [H], np.asarray(L[key], np.float32)))
        for k in ("q", "k", "v"):
            if L.get(k + "_bias") is not None:  # qwen2-style projections
                b = np.asarray(L[k + "_bias"], np.float32)
                ts.append((p + f"attn_{k}.bias", F32, [b.size], b))
        ts.append((p + "ffn_norm.weight", F32, [H], np.asarray(L["ffn_norm"], np.float32)))
    write_gguf(path, md, ts, alignment=alignment)
