"""Writes the golden fixtures under tests/golden/ by running the REFERENCE's own CPU code
(oracle/_ref/libptm_ref.so, compiled from the reference checkout by `make -C oracle ref`).

Run from the repo root in a container that has the reference checkout:
    make -C oracle ref && python tests/golden/make_golden.py [--full]

Inputs are regenerated from seeds by prometorch_amd.synth, so the fixtures hold only the
reference's OUTPUTS (plus a few hand-built edge-case input blocks).  --full also runs the
Qwen3-4B-shaped model for 128 greedy steps (about 3 GB of synthetic weights, a few minutes)."""
from __future__ import annotations

import argparse
import hashlib
import json
import os
import platform
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import pyoracle as po  # noqa: E402
from prometorch_amd.testing import synth  # noqa: E402

OUT = os.path.dirname(os.path.abspath(__file__))
SEEDS = {"blocks": 101, "cfg1": 1001, "cfg2": 1002, "cfg3": 1003, "tiny": 7, "cfg4": 25, "ragged": 1005}


def sha(a: np.ndarray) -> str:
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def edge_blocks_q4k() -> np.ndarray:
    """Hand-built Q4_K blocks: zero d, subnormal fp16 d/dmin, max scales, all-0 / all-15 quants."""
    rng = synth.rng_for(SEEDS["blocks"], 9)
    b = synth.make_q4k(rng, 8, 256).reshape(8, 144).copy()
    b[0, 0:4] = 0                                       # d = dmin = 0
    b[1, 0:2] = np.array([0x0001], np.uint16).view(np.uint8)  # smallest subnormal d
    b[1, 2:4] = np.array([0x03FF], np.uint16).view(np.uint8)  # largest subnormal dmin
    b[2, 4:16] = 0xFF                                   # all scales/mins 63
    b[3, 16:144] = 0x00
    b[4, 16:144] = 0xFF
    b[5, 0:2] = np.array([0x7BFF], np.uint16).view(np.uint8)  # max finite d
    b[6, 4:16] = 0x00
    return b


def edge_blocks_q6k() -> np.ndarray:
    rng = synth.rng_for(SEEDS["blocks"], 10)
    b = synth.make_q6k(rng, 8, 256).reshape(8, 210).copy()
    b[0, 208:210] = 0
    b[1, 208:210] = np.array([0x0001], np.uint16).view(np.uint8)
    b[2, 192:208] = np.array([-128], np.int8).view(np.uint8)   # most negative scale
    b[3, 192:208] = 127
    b[4, 0:192] = 0x00                                  # q = -32 everywhere
    b[5, 0:192] = 0xFF                                  # q = 31 everywhere
    b[6, 208:210] = np.array([0x83FF], np.uint16).view(np.uint8)  # negative subnormal d
    return b


def ref_dequant(qt, raw):
    raw = np.ascontiguousarray(raw, np.uint8).reshape(-1)
    n = raw.size // (144 if qt == 12 else 210) * 256
    out = np.empty(n, np.float32)
    (po.ref().ref_dequantize_q4_k if qt == 12 else po.ref().ref_dequantize_q6_k)(po._p(raw), po._p(out), n)
    return out


def ref_q8(x):
    K = x.size
    d = np.empty(K // 32, np.float32)
    s = np.empty(K // 32, np.float32)
    q = np.empty(K, np.int8)
    po.ref().ref_quantize_x_q8(po._p(x), K, po._p(d), po._p(s), po._p(q))
    return d, s, q


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--full", action="store_true")
    ap.add_argument("--sampling-only", action="store_true", help="write golden_sampling.npz and nothing else")
    ap.add_argument("--tokenizer-only", action="store_true", help="write golden_tokenizer.json and nothing else")
    ap.add_argument("--random-only", action="store_true", help="write golden_random_arch.npz and nothing else")
    ap.add_argument("--gemma-only", action="store_true", help="write golden_gemma.npz and nothing else")
    ap.add_argument("--qwen2-only", action="store_true", help="write golden_qwen2.npz and nothing else")
    ap.add_argument("--llama-only", action="store_true", help="write golden_llama.npz and nothing else")
    ap.add_argument("--mixed-only", action="store_true", help="write golden_mixed.npz and nothing else")
    ap.add_argument("--formats-only", action="store_true", help="write golden_formats.npz and nothing else")
    ap.add_argument("--f32act-only", action="store_true", help="write golden_q4k_f32act.npz and nothing else")
    ap.add_argument("--longrope-only", action="store_true", help="write golden_longrope.npz and nothing else")
    ap.add_argument("--loader-only", action="store_true", help="write golden_loader.npz and nothing else")
    ap.add_argument("--forced-only", action="store_true", help="add the teacher-forced runs to golden_llama / _qwen2 / _gemma.npz")
    ap.add_argument("--forced-full-only", action="store_true", help="add the teacher-forced Qwen3-4B-shaped run to golden_cfg4.npz")
    ap.add_argument("--centered-only", action="store_true", help="write golden_cfg4_centered.npz and nothing else")
    args = ap.parse_args()
    assert po.have_ref(), "build oracle/_ref first: make -C oracle ref"
    if args.forced_only:
        make_forced_tiny()
        print("added forced_* to golden_llama.npz, golden_qwen2.npz, golden_gemma.npz")
        return
    if args.centered_only:
        make_forced_centered()
        print("wrote golden_cfg4_centered.npz")
        return
    if args.forced_full_only:
        make_forced_full()
        print("added forced_* to golden_cfg4.npz")
        return
    if args.sampling_only:
        make_sampling()
        print("wrote golden_sampling.npz")
        return
    if args.tokenizer_only:
        make_tokenizer_golden()
        print("wrote golden_tokenizer.json")
        return
    if args.random_only:
        make_random_arch_golden()
        print("wrote golden_random_arch.npz")
        return
    if args.gemma_only:
        make_gemma_golden()
        print("wrote golden_gemma.npz")
        return
    if args.qwen2_only:
        make_qwen2_golden()
        print("wrote golden_qwen2.npz")
        return
    if args.llama_only:
        make_llama_golden()
        print("wrote golden_llama.npz")
        return
    if args.mixed_only:
        make_mixed_golden()
        print("wrote golden_mixed.npz, golden_formats_model.npz")
        return
    if args.f32act_only:
        make_f32act_golden()
        return
    if args.longrope_only:
        make_longrope_golden()
        return
    if args.loader_only:
        make_loader_golden()
        return
    if args.formats_only:
        make_formats_golden()
        print("wrote golden_formats.npz")
        return
    R = po.ref()
    meta = {"made_with": "oracle/_ref/libptm_ref.so (g++ -O2 -std=c++17 -mavx2 -mfma; see oracle/Makefile)",
            "python": platform.python_version(), "numpy": np.__version__, "threads": R.ref_num_threads(), "seeds": SEEDS}
    g = {}

    # ---- fp16 table: all 65536 inputs -----------------------------------------------
    g["fp16_table_sha"] = np.frombuffer(sha(np.array([R.ref_fp16_to_fp32(h) for h in range(65536)], np.float32)).encode(), np.uint8)

    # ---- blocks: 64 random + 8 edge blocks per format, reference dequant ----------------
    rng = synth.rng_for(SEEDS["blocks"])
    q4 = np.concatenate([synth.make_q4k(rng, 64, 256).reshape(64, 144), edge_blocks_q4k()])
    q6 = np.concatenate([synth.make_q6k(rng, 64, 256).reshape(64, 210), edge_blocks_q6k()])
    g["q4k_blocks"] = q4
    g["q4k_deq"] = ref_dequant(12, q4)
    g["q6k_blocks"] = q6
    g["q6k_deq"] = ref_dequant(14, q6)

    # ---- Q8 activation quantiser ---------------------------------------------------------
    x = synth.make_x(rng, 2560)
    x[32:64] = 0.0                       # all-zero block: d = 0, id = 0
    x[64] = 127.0; x[65] = 0.5; x[66] = 1.5; x[67] = 2.5; x[68] = -0.5; x[69] = -1.5  # exact .5 ties -> half-even
    x[64:96][6:] = 0.25
    g["q8_x"] = x
    g["q8_d"], g["q8_sum"], g["q8_qs"] = ref_q8(x)

    # ---- cfg1: Q4_K GEMV 9728 x 2560 ------------------------------------------------------
    r1 = synth.rng_for(SEEDS["cfg1"])
    W = synth.make_q4k(r1, 9728, 2560)
    x1 = synth.make_x(r1, 2560)
    y = po.ref_gemv(12, W, x1)
    g["cfg1_y256"] = y[:256].copy()
    g["cfg1_sha"] = np.frombuffer(sha(y).encode(), np.uint8)
    meta["cfg1_rms"] = float(np.sqrt((y.astype(np.float64) ** 2).mean()))
    t = time.time()
    for _ in range(5):
        po.ref_gemv(12, W, x1)
    meta["cfg1_ref_ms_8core_container"] = (time.time() - t) / 5 * 1e3

    # ---- ragged / odd shapes (odd N exercises the unpaired-row path) ----------------------
    rr = synth.rng_for(SEEDS["ragged"])
    for i, (qt, N, K) in enumerate([(12, 33, 512), (12, 1, 256), (12, 77, 2560), (14, 7, 256), (14, 45, 1024)]):
        Wr = synth.make_weight(rr, qt, N, K)
        xr = synth.make_x(rr, K)
        g[f"ragged{i}_y"] = po.ref_gemv(qt, Wr, xr)

    # ---- cfg2: Q6_K lm_head GEMV + argmax (full size) -------------------------------------
    r2 = synth.rng_for(SEEDS["cfg2"])
    W2 = synth.make_q6k(r2, 151936, 2560)
    x2 = synth.make_x(r2, 2560)
    y2 = po.ref_gemv(14, W2, x2)
    top = np.argsort(-y2, kind="stable")[:8]
    g["cfg2_top8_idx"] = top.astype(np.int64)
    g["cfg2_top8_val"] = y2[top]
    g["cfg2_y256"] = y2[:256].copy()
    g["cfg2_sha"] = np.frombuffer(sha(y2).encode(), np.uint8)
    g["cfg2_argmax"] = np.array([int(np.argmax(y2))], np.int64)
    del W2

    # ---- cfg3: one Qwen3-4B layer's seven GEMVs, independent N(0,1) inputs -----------------
    L = synth.make_layer(SEEDS["cfg3"], 0, synth.QWEN3_4B)
    for i, (name, qt) in enumerate(synth.LAYER_MATS):
        _, Wm = L[name]
        K = Wm.shape[1] // (144 if qt == 12 else 210) * 256
        xm = synth.make_x(synth.rng_for(SEEDS["cfg3"], 5, i), K)
        ym = po.ref_gemv(qt, Wm, xm)
        g[f"cfg3_{name}_y64"] = ym[:: max(1, ym.size // 64)][:64].copy()
        g[f"cfg3_{name}_sha"] = np.frombuffer(sha(ym).encode(), np.uint8)
    # fused RMSNorm + gate/up as the reference's CPU fusion computes it
    xg = (synth.make_x(synth.rng_for(SEEDS["cfg3"], 6), 2560) * 3.0).astype(np.float32)
    yg = np.empty(9728, np.float32)
    yu = np.empty(9728, np.float32)
    Wg = np.ascontiguousarray(L["gate"][1])
    Wu = np.ascontiguousarray(L["up"][1])
    gam = np.ascontiguousarray(L["ffn_norm"])
    R.ref_fused_rmsnorm_gate_up(po._p(xg), po._p(gam), 1e-6, 0, 12, po._p(Wg), 12, po._p(Wu), po._p(yg), po._p(yu),
                                2560, 9728, 9728, Wg.shape[1], Wu.shape[1])
    g["cfg3_fused_gate_y64"] = yg[::152][:64].copy()
    g["cfg3_fused_up_y64"] = yu[::152][:64].copy()

    # ---- glue: rmsnorm, rope, exp ------------------------------------------------------------
    rg = synth.rng_for(SEEDS["blocks"], 11)
    xn = synth.make_x(rg, 2560)
    gm = (1.0 + 0.1 * synth.make_x(rg, 2560)).astype(np.float32)
    o = xn.copy()
    R.ref_rmsnorm_inplace(po._p(o), po._p(gm), 1e-6, 0, 2560)
    g["rms_x"], g["rms_g"], g["rms_out"] = xn, gm, o
    for pos in (0, 1, 2048, 2175):
        c = np.empty(64, np.float32)
        s = np.empty(64, np.float32)
        R.ref_rope_precompute(po._p(c), po._p(s), pos, 128, 1e6)
        g[f"rope_cos_{pos}"], g[f"rope_sin_{pos}"] = c, s
    qv = synth.make_x(rg, 4096)
    kv = synth.make_x(rg, 1024)
    g["rope_q_in"], g["rope_k_in"] = qv.copy(), kv.copy()
    R.ref_rope_apply_neox(po._p(qv), po._p(kv), po._p(g["rope_cos_2048"]), po._p(g["rope_sin_2048"]), 32, 8, 128)
    g["rope_q_out"], g["rope_k_out"] = qv, kv
    e = np.linspace(-90, 20, 1024, dtype=np.float32)
    eo = np.empty_like(e)
    R.ref_exp256(po._p(e), po._p(eo), e.size // 8)
    g["exp_in"], g["exp_out"] = e, eo

    # ---- tiny model: full logits of the reference's forward_decode_cpu over 12 steps ----------
    cfg = dict(synth.TINY)
    layers = [synth.make_layer(SEEDS["tiny"], i, cfg) for i in range(cfg["n_layers"])]
    head = synth.make_head(SEEDS["tiny"], cfg)
    emb = po.dequant(14, head["lm_head"]).reshape(cfg["vocab"], cfg["hidden"])
    rm = po.RefModel(cfg, layers, head, 64, emb)
    for i in range(cfg["n_layers"]):
        k, v = synth.make_kv_prefill(SEEDS["tiny"], i, cfg, 19)
        rm.set_kv(i, k, v)
    tok, toks, lg = 3, [], []
    for _ in range(12):
        tok = rm.step(tok)
        toks.append(tok)
        lg.append(rm.logits.copy())
    g["tiny_tokens"] = np.array(toks, np.int64)
    g["tiny_logits"] = np.stack(lg)
    rm.close()

    np.savez_compressed(os.path.join(OUT, "golden_small.npz"), **g)
    make_sampling()
    make_tokenizer_golden()
    make_llama_golden()
    make_qwen2_golden()
    make_gemma_golden()
    make_random_arch_golden()
    make_formats_golden()
    make_mixed_golden()

    if args.full:
        make_full(meta)
    with open(os.path.join(OUT, "golden_meta.json"), "w") as f:
        json.dump(meta, f, indent=1, sort_keys=True)
    print("wrote", OUT)


def make_sampling():
    """The reference's sample_token over synth.SAMPLING_CASES, called in order in this (fresh) process: its
    generator is a function-local static std::mt19937(42), so call n with temperature >= 1e-6 uses draw n.
    (Nothing else in this script samples, so the draws start at the first.)"""
    R = po.ref()
    t = synth.TINY
    h = R.ref_model_create(t["vocab"], t["hidden"], t["n_layers"], t["n_heads"], t["n_kv_heads"], t["head_dim"], t["inter"],
                           t["rope_base"], t["eps"], 8)  # sample_token reads no model state
    toks = []
    for i, (vocab, kind, temperature, top_k, top_p) in enumerate(synth.SAMPLING_CASES):
        x = np.ascontiguousarray(synth.sampling_logits(i))
        toks.append(int(R.ref_sample_token(h, x.ctypes.data, vocab, temperature, top_k, top_p)))
    R.ref_model_destroy(h)
    np.savez_compressed(os.path.join(OUT, "golden_sampling.npz"), tokens=np.array(toks, np.int32))


CHAT_CASES = [  # (architecture, model name, PT_SYSTEM_PROMPT or None = unset, PT_NO_THINK, prompt)
    ("qwen3", "Qwen3-4B", None, False, "Hello!"), ("qwen3", "Qwen3-4B", None, True, "2+2?"), ("qwen3", "q", "", True, "x"),
    ("qwen3", "q", "", False, "no system"), ("qwen2", "q2", "Be brief.", True, "hi"), ("phi3", "Phi-3", None, False, "p"),
    ("phi3", "Phi-3", "", False, "p"), ("gemma3", "g", None, False, "hello"), ("gemma2", "g", "", False, "hello"),
    ("llama", "Meta-Llama-3-8B", None, False, "hey"), ("llama", "Meta-Llama-3-8B", "", False, "hey"),
    ("llama", "Mistral-7B-Instruct", None, False, "m"), ("llama", "MISTRAL", "", False, "m"), ("deepseek2", "x", None, False, "raw prompt"),
]


def make_tokenizer_golden():
    """The reference's GGUFTokenizer over the synthetic tokenizers of prometorch_amd.synth (written as GGUF files by
    this repository's writer and read back by the REFERENCE's GGUFReader) and its apply_chat_template."""
    import base64
    import tempfile
    import ctypes as C
    from prometorch_amd import gguf
    from prometorch_amd.testing import gguf_writer
    R = po.ref()
    b64 = lambda b: base64.b64encode(b).decode()
    out = {"tokenizers": {}, "chat": []}
    buf = C.create_string_buffer(1 << 16)
    ids = (C.c_int32 * 4096)()

    def text_of(fn, *args):  # the call first, the buffer after it
        n = fn(*args, buf, 1 << 16)
        assert n <= 1 << 16
        return buf.raw[:n]

    for kind in ("gpt2", "llama", "greedy"):
        md = synth.make_tokenizer(kind)
        md["general.architecture"] = "qwen3"
        with tempfile.TemporaryDirectory() as d:
            path = os.path.join(d, "tok.gguf")
            gguf_writer.write_gguf(path, md, [("dummy", 0, [4], np.zeros(4, np.float32))])
            assert R.ref_gguf_n_tensors(path.encode()) == 1
            h = R.ref_tokenizer_load(path.encode())
        cases = []
        for text in synth.tokenizer_texts(kind):
            for use_bos in (True, False):
                n = R.ref_tokenizer_encode(h, text, len(text), int(use_bos), ids, 4096)
                assert n <= 4096
                got = [int(ids[i]) for i in range(n)]
                a = (C.c_int32 * max(1, n))(*got)
                dec = [text_of(R.ref_tokenizer_decode, h, a, n, int(sk)) for sk in (True, False)]
                cases.append({"text": b64(text), "use_bos": use_bos, "ids": got, "decoded_skip": b64(dec[0]), "decoded_all": b64(dec[1])})
        n_vocab = len(md["tokenizer.ggml.tokens"])
        toks = [b64(text_of(R.ref_tokenizer_token, h, i)) for i in range(-1, n_vocab + 1)]
        out["tokenizers"][kind] = {"cases": cases, "token_bytes_from_minus1": toks}
        R.ref_tokenizer_free(h)
    for arch, name, sys_prompt, no_think, prompt in CHAT_CASES:
        for k, v in (("PT_SYSTEM_PROMPT", sys_prompt), ("PT_NO_THINK", "1" if no_think else None)):
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
        out["chat"].append({"arch": arch, "name": name, "system": sys_prompt, "no_think": no_think, "prompt": prompt,
                            "text": text_of(R.ref_chat_template, arch.encode(), name.encode(), prompt.encode()).decode()})
    os.environ.pop("PT_SYSTEM_PROMPT", None)
    os.environ.pop("PT_NO_THINK", None)
    with open(os.path.join(OUT, "golden_tokenizer.json"), "w") as f:
        json.dump(out, f, indent=0, sort_keys=True)


FORMAT_CASES = [(13, 24, 512), (13, 3, 2560), (8, 24, 512), (8, 5, 96), (6, 24, 512), (6, 7, 32)]  # (ggml type, N, K)


def make_formats_golden():
    """The reference's dispatcher on its other block formats (Q5_K, Q8_0, Q5_0: cpu_quant_gemv.h:1635-1688) and its
    dequantisers of the first two, on seeded blocks (synth.make_weight / make_x from SEEDS['blocks'], type, N, K)."""
    g = {}
    for qt, N, K in FORMAT_CASES:
        r = synth.rng_for(SEEDS["blocks"], qt, N, K)
        W = synth.make_weight(r, qt, N, K)
        x = synth.make_x(r, K)
        g["y_%d_%d_%d" % (qt, N, K)] = po.ref_gemv(qt, W, x)
        if qt != 6:
            g["dq_%d_%d_%d" % (qt, N, K)] = po.ref_dequant(qt, W)
    np.savez_compressed(os.path.join(OUT, "golden_formats.npz"), **g)


def make_mixed_golden():
    """The reference's forward_decode_cpu on synth.tiny_mixed: layers whose q/k/v share a type (fused QKV, 8-lane
    norm, gguf_model.h:3342-3350) beside layers where they do not, Q4_K and Q6_K in every projection role; and on
    synth.tiny_formats: Q8_0, Q5_K and Q5_0 matrices through the same step (golden_formats_model.npz)."""
    for maker, fname in ((synth.tiny_mixed, "golden_mixed.npz"), (synth.tiny_formats, "golden_formats_model.npz")):
        _model_golden(maker, fname)


def _model_golden(maker, fname):
    cfg, layers, head = maker(SEEDS["tiny"])
    emb = po.dequant(14, head["lm_head"]).reshape(cfg["vocab"], cfg["hidden"])
    rm = po.RefModel(cfg, layers, head, 64, emb)
    for i in range(cfg["n_layers"]):
        k, v = synth.make_kv_prefill(SEEDS["tiny"], i, cfg, 19)
        rm.set_kv(i, k, v)
    toks, lg = [], []
    for st in range(12):   # fed tokens are fixed (synth.MIXED_FEED): the greedy loop of this model settles on one token
        toks.append(rm.step(synth.MIXED_FEED[st]))
        lg.append(rm.logits.copy())
    rm.close()
    np.savez_compressed(os.path.join(OUT, fname), tokens=np.array(toks, np.int64), logits=np.stack(lg))


def make_llama_golden():
    """The reference's forward_decode_cpu on a llama-style tiny model (synth.tiny_llama): no QK-norm, interleaved
    rotation pairs; 12 greedy steps after a 19-position cache, plus the rotation alone."""
    R = po.ref()
    cfg, layers, head = synth.tiny_llama(SEEDS["tiny"])
    emb = po.dequant(14, head["lm_head"]).reshape(cfg["vocab"], cfg["hidden"])
    rm = po.RefModel(cfg, layers, head, 64, emb)
    for i in range(cfg["n_layers"]):
        k, v = synth.make_kv_prefill(SEEDS["tiny"], i, cfg, 19)
        rm.set_kv(i, k, v)
    tok, toks, lg = 3, [], []
    for _ in range(12):
        tok = rm.step(tok)
        toks.append(tok)
        lg.append(rm.logits.copy())
    rm.close()
    g = {"tokens": np.array(toks, np.int64), "logits": np.stack(lg)}
    r = synth.rng_for(SEEDS["blocks"], 77)
    q = (3 * r.standard_normal(32 * 128, dtype=np.float32)).astype(np.float32)
    k = (3 * r.standard_normal(8 * 128, dtype=np.float32)).astype(np.float32)
    c, s = po.rope_tables(2049, 128, 5.0e5)
    R.ref_rope_apply_norm(q.ctypes.data, k.ctypes.data, c.ctypes.data, s.ctypes.data, 32, 8, 128)
    g["rope_norm_q"], g["rope_norm_k"] = q, k
    # linear position scaling (rope.scaling.type = linear): the same model at scale 4, and the table alone
    cfg4 = dict(cfg, rope_scale=4.0)
    rm = po.RefModel(cfg4, layers, head, 64, emb)
    for i in range(cfg["n_layers"]):
        k, v = synth.make_kv_prefill(SEEDS["tiny"], i, cfg, 19)
        rm.set_kv(i, k, v)
    tok, toks, lg = 3, [], []
    for _ in range(12):
        tok = rm.step(tok)
        toks.append(tok)
        lg.append(rm.logits.copy())
    rm.close()
    g["scaled_tokens"], g["scaled_logits"] = np.array(toks, np.int64), np.stack(lg)
    c4, s4 = np.empty(64, np.float32), np.empty(64, np.float32)
    R.ref_rope_precompute_scaled(c4.ctypes.data, s4.ctypes.data, 2049, 128, 5.0e5, 4.0)
    g["scaled_cos"], g["scaled_sin"] = c4, s4
    np.savez_compressed(os.path.join(OUT, "golden_llama.npz"), **g)


def make_qwen2_golden():
    """The reference's forward_decode_cpu on a qwen2-style tiny model (synth.tiny_qwen2): q / k / v biases, no QK-norm,
    NeoX rotation; 12 greedy steps after a 19-position cache."""
    cfg, layers, head = synth.tiny_qwen2(SEEDS["tiny"])
    emb = po.dequant(14, head["lm_head"]).reshape(cfg["vocab"], cfg["hidden"])
    rm = po.RefModel(cfg, layers, head, 64, emb)
    for i in range(cfg["n_layers"]):
        k, v = synth.make_kv_prefill(SEEDS["tiny"], i, cfg, 19)
        rm.set_kv(i, k, v)
    tok, toks, lg = 3, [], []
    for _ in range(12):
        tok = rm.step(tok)
        toks.append(tok)
        lg.append(rm.logits.copy())
    rm.close()
    np.savez_compressed(os.path.join(OUT, "golden_qwen2.npz"), tokens=np.array(toks, np.int64), logits=np.stack(lg))


def make_gemma_golden():
    """The reference's forward_decode_cpu on a gemma3-style tiny model (synth.tiny_gemma): scaled embeddings, GELU gate,
    post-norms, sliding-window layers with their own rotation base; 16 greedy steps after a 19-position cache (the
    window of 8 is exceeded from the first step)."""
    cfg, layers, head = synth.tiny_gemma(SEEDS["tiny"])
    emb = po.dequant(14, head["lm_head"]).reshape(cfg["vocab"], cfg["hidden"])
    rm = po.RefModel(cfg, layers, head, 64, emb)
    for i in range(cfg["n_layers"]):
        k, v = synth.make_kv_prefill(SEEDS["tiny"], i, cfg, 19)
        rm.set_kv(i, k, v)
    tok, toks, lg = 3, [], []
    for _ in range(16):
        tok = rm.step(tok)
        toks.append(tok)
        lg.append(rm.logits.copy())
    rm.close()
    np.savez_compressed(os.path.join(OUT, "golden_gemma.npz"), tokens=np.array(toks, np.int64), logits=np.stack(lg))


def make_f32act_golden():
    """The reference's fp32-activation Q4_K kernel (q4k_gemv_scalar, cpu_quant_gemv.h:689-767) on seeded matrices:
    96 x 2560 and, for the ragged end, 5 x 256."""
    R = po.ref()
    out = {}
    for name, N, K in (("a", 96, 2560), ("b", 5, 256)):
        r = synth.rng_for(SEEDS["blocks"], 31, N)
        W = synth.make_q4k(r, N, K)
        x = synth.make_x(r, K)
        y = np.empty(N, np.float32)
        R.ref_q4k_gemv_scalar(W.ctypes.data, x.ctypes.data, y.ctypes.data, K, N, W.shape[1])
        out["y_" + name] = y
    np.savez_compressed(os.path.join(OUT, "golden_q4k_f32act.npz"), **out)


def longrope_cfg(seed):
    """synth.TINY with phi3-style LongRoPE terms: per-frequency factors (a short and a long set), the short set valid up to a
    22-token context - so a run that starts behind 19 cached positions crosses over after three steps - and an attention
    factor on cos / sin."""
    cfg = dict(synth.TINY)
    r = synth.rng_for(seed, 55)
    half = cfg["head_dim"] // 2
    cfg["rope_factors_short"] = (1.0 + 0.25 * r.random(half)).astype(np.float32)
    cfg["rope_factors_long"] = (1.0 + 8.0 * r.random(half)).astype(np.float32)
    cfg["rope_orig_ctx"] = 22
    cfg["rope_attn_factor"] = 1.19
    return cfg


def make_longrope_golden():
    """The reference's rope_precompute with per-frequency factors and attn_factor (hot_loops.cpp:1853-1876), alone and inside
    forward_decode_cpu (rope_factors_for(past + 1), gguf_model.h:285-296, :3456-3463): 12 steps behind 19 cached positions."""
    R = po.ref()
    cfg = longrope_cfg(SEEDS["tiny"])
    layers = [synth.make_layer(SEEDS["tiny"], i, cfg) for i in range(cfg["n_layers"])]
    head = synth.make_head(SEEDS["tiny"], cfg)
    g = {}
    hd = cfg["head_dim"]
    for pos in (0, 1, 21, 22, 2049):
        for which in ("short", "long"):
            c, s = np.empty(hd // 2, np.float32), np.empty(hd // 2, np.float32)
            f = cfg["rope_factors_" + which]
            R.ref_rope_precompute_factors(c.ctypes.data, s.ctypes.data, pos, hd, cfg["rope_base"], 1.0, f.ctypes.data,
                                          cfg["rope_attn_factor"])
            g["cos_%s_%d" % (which, pos)], g["sin_%s_%d" % (which, pos)] = c, s
    emb = po.dequant(14, head["lm_head"]).reshape(cfg["vocab"], cfg["hidden"])
    rm = po.RefModel(cfg, layers, head, 64, emb)
    for i in range(cfg["n_layers"]):
        k, v = synth.make_kv_prefill(SEEDS["tiny"], i, cfg, 19)
        rm.set_kv(i, k, v)
    tok, toks, lg = 3, [], []
    for _ in range(12):
        tok = rm.step(tok)
        toks.append(tok)
        lg.append(rm.logits.copy())
    rm.close()
    g["tokens"], g["logits"] = np.array(toks, np.int64), np.stack(lg)
    np.savez_compressed(os.path.join(OUT, "golden_longrope.npz"), **g)
    print("longrope tokens", toks)


LOADER_FEED = (3, 17, 900, 41, 5, 5, 260, 77)   # tokens fed to the loaded models step by step


def loader_cases(seed):
    """(name, cfg, layers, head, writer keyword arguments) of the files the loader fixture covers: one per architecture the
    loader accepts, tied and untied output matrices, and linear position scaling."""
    t = dict(synth.TINY)
    tl = [synth.make_layer(seed, i, t) for i in range(t["n_layers"])]
    th = synth.make_head(seed, t)
    lc, ll, lh = synth.tiny_llama(seed)
    qc, ql, qh = synth.tiny_qwen2(seed)
    gc, gl, gh = synth.tiny_gemma(seed)
    return [("qwen3_tied", t, tl, th, dict(arch="qwen3", tied=True)),
            ("qwen3_untied", t, tl, th, dict(arch="qwen3", tied=False, alignment=64)),
            ("llama", lc, ll, lh, dict(arch="llama")),
            ("llama_scaled", dict(lc, rope_scale=4.0), ll, lh, dict(arch="llama")),
            ("qwen2", qc, ql, qh, dict(arch="qwen2")),
            ("gemma3", gc, gl, gh, dict(arch="gemma3"))]


def make_loader_golden():
    """Files written by this repository's GGUF writer, read by the REFERENCE's own loader (GGUFModel::load,
    gguf_model.h:2038-2089): what its parser made of the metadata (config fields), which matrices it registered as
    quantised weights and with which type, and 8 steps of forward_decode_cpu logits behind a 19-position cache."""
    import tempfile
    from prometorch_amd.testing import gguf_writer
    out = {}
    with tempfile.TemporaryDirectory() as td:
        for name, cfg, layers, head, kw in loader_cases(SEEDS["tiny"]):
            path = os.path.join(td, name + ".gguf")
            gguf_writer.model_to_gguf(path, cfg, layers, head, **kw)
            rm = po.RefLoadedModel(path, 64)
            for i in range(cfg["n_layers"]):
                k, v = synth.make_kv_prefill(SEEDS["tiny"], i, cfg, 19)
                rm.set_kv(i, k, v)
            toks, lg = [], []
            for tok in LOADER_FEED:
                toks.append(rm.step(tok))
                lg.append(rm.logits.copy())
            out[name + "_ints"], out[name + "_floats"], out[name + "_types"] = rm.ints.copy(), rm.floats.copy(), rm.types.copy()
            out[name + "_tokens"], out[name + "_logits"] = np.array(toks, np.int64), np.stack(lg)
            out[name + "_sha"] = np.frombuffer(hashlib.sha256(open(path, "rb").read()).hexdigest().encode(), np.uint8)
            rm.close()
            print(name, dict(zip(po.LOADED_INT_FIELDS, rm.ints.tolist())), rm.floats.tolist(), toks, flush=True)
    np.savez_compressed(os.path.join(OUT, "golden_loader.npz"), **out)


def make_random_arch_golden():
    """The reference's forward_decode_cpu on synth.random_model(0..9): ten decoders whose architectural switches (head width,
    heads per kv head, QK-norm, rotation pairing and scaling, biases, the gemma features, per-matrix types) are drawn at
    random; 4 steps each behind 11 cached positions."""
    out = {}
    for seed in range(10):
        cfg, layers, head = synth.random_model(seed)
        emb = po.dequant(14, head["lm_head"]).reshape(cfg["vocab"], cfg["hidden"])
        rm = po.RefModel(cfg, layers, head, 32, emb)
        for i in range(cfg["n_layers"]):
            k, v = synth.make_kv_prefill(1000 + seed, i, cfg, 11)
            rm.set_kv(i, k, v)
        tok, lg = 5, []
        for _ in range(4):
            tok = rm.step(tok)
            lg.append(rm.logits.copy())
        rm.close()
        out["logits_%d" % seed] = np.stack(lg)
    np.savez_compressed(os.path.join(OUT, "golden_random_arch.npz"), **out)


def make_full(meta):
    """cfg4: Qwen3-4B shape, 36 layers, KV prefilled to 2048, 128 greedy steps on the reference CPU path
    (fp32 KV rows for new tokens, as forward_decode_cpu keeps them)."""
    cfg = dict(synth.QWEN3_4B)
    seed = SEEDS["cfg4"]
    t0 = time.time()
    layers = [synth.make_layer(seed, i, cfg) for i in range(cfg["n_layers"])]
    head = synth.make_head(seed, cfg)
    print("generated model in %.1fs" % (time.time() - t0), flush=True)
    emb = po.dequant(14, head["lm_head"]).reshape(cfg["vocab"], cfg["hidden"])
    max_seq, npos, steps = 2304, 2048, 128
    rm = po.RefModel(cfg, layers, head, max_seq, emb)
    for i in range(cfg["n_layers"]):
        k, v = synth.make_kv_prefill(seed, i, cfg, npos)
        rm.set_kv(i, k, v)
    g = {}
    tok, toks, margins, tops = 1, [], [], []
    t0 = time.time()
    for st in range(steps):
        tok = rm.step(tok)
        toks.append(tok)
        srt = np.sort(rm.logits)
        margins.append(float(srt[-1] - srt[-2]))
        tops.append(float(srt[-1]))
        if st in (0, 1, 63, 127):
            g[f"logits256_step{st}"] = rm.logits[:256].copy()
            g[f"logits_sha_step{st}"] = np.frombuffer(sha(rm.logits).encode(), np.uint8)
            g[f"logits_std_step{st}"] = np.array([rm.logits.std()], np.float32)
        if st % 16 == 0:
            print("step", st, "tok", tok, "margin", margins[-1], "%.1fs" % (time.time() - t0), flush=True)
    meta["cfg4_ref_tok_per_s_8core_container"] = steps / (time.time() - t0)
    g["tokens"] = np.array(toks, np.int64)
    g["margins"] = np.array(margins, np.float32)
    g["top1"] = np.array(tops, np.float32)
    rm.close()
    np.savez_compressed(os.path.join(OUT, "golden_cfg4.npz"), **g)


def forced_feed(seed, vocab, n):
    """n distinct token ids, seeded: what a teacher-forced run feeds instead of its own argmax."""
    return [int(t) for t in synth.rng_for(seed, 7700).choice(vocab, size=n, replace=False)]


FORCED_SAMPLE = 64   # logits kept per step of the full-size forced run: indices (k * vocab) // FORCED_SAMPLE


def _add_to_npz(fname, extra):
    path = os.path.join(OUT, fname)
    with np.load(path, allow_pickle=False) as z:
        g = {k: z[k] for k in z.files if not k.startswith("forced_")}
    g.update(extra)
    np.savez_compressed(path, **g)


def make_forced_tiny():
    """The greedy runs of the tiny llama / qwen2 / gemma models settle on one token; these runs feed 16 distinct seeded ids
    instead (teacher forcing), so that every step sees another embedding row and other cache rows.  Stored: the reference's
    argmax and full logits per step."""
    for maker, fname in ((synth.tiny_llama, "golden_llama.npz"), (synth.tiny_qwen2, "golden_qwen2.npz"),
                         (synth.tiny_gemma, "golden_gemma.npz")):
        cfg, layers, head = maker(SEEDS["tiny"])
        emb = po.dequant(14, head["lm_head"]).reshape(cfg["vocab"], cfg["hidden"])
        rm = po.RefModel(cfg, layers, head, 64, emb)
        for i in range(cfg["n_layers"]):
            k, v = synth.make_kv_prefill(SEEDS["tiny"], i, cfg, 19)
            rm.set_kv(i, k, v)
        feed = forced_feed(SEEDS["tiny"], cfg["vocab"], 16)
        toks, lg = [], []
        for t in feed:
            toks.append(rm.step(t))
            lg.append(rm.logits.copy())
        rm.close()
        _add_to_npz(fname, {"forced_feed": np.array(feed, np.int64), "forced_tokens": np.array(toks, np.int64),
                            "forced_logits": np.stack(lg)})


def make_forced_full():
    """cfg4 teacher-forced: the Qwen3-4B-shaped model of make_full, cache prefilled to 2048, fed 128 distinct seeded ids.  The
    greedy run of that model alternates between two ids; this run puts 128 different embedding rows and 128 different new
    cache rows through the full-size step.  Stored per step: the reference's argmax, top-2 margin and standard deviation of
    the logits, and FORCED_SAMPLE logits at fixed strided indices; for four steps also the first 256 logits and a hash."""
    cfg = dict(synth.QWEN3_4B)
    seed = SEEDS["cfg4"]
    t0 = time.time()
    layers = [synth.make_layer(seed, i, cfg) for i in range(cfg["n_layers"])]
    head = synth.make_head(seed, cfg)
    print("generated model in %.1fs" % (time.time() - t0), flush=True)
    emb = po.dequant(14, head["lm_head"]).reshape(cfg["vocab"], cfg["hidden"])
    max_seq, npos, steps = 2304, 2048, 128
    rm = po.RefModel(cfg, layers, head, max_seq, emb)
    for i in range(cfg["n_layers"]):
        k, v = synth.make_kv_prefill(seed, i, cfg, npos)
        rm.set_kv(i, k, v)
    feed = forced_feed(seed, cfg["vocab"], steps)
    idx = (np.arange(FORCED_SAMPLE, dtype=np.int64) * cfg["vocab"]) // FORCED_SAMPLE
    g = {"forced_feed": np.array(feed, np.int64), "forced_sample_index": idx}
    toks, margins, stds, samples = [], [], [], []
    t0 = time.time()
    for st, t in enumerate(feed):
        toks.append(rm.step(t))
        srt = np.sort(rm.logits)
        margins.append(float(srt[-1] - srt[-2]))
        stds.append(float(rm.logits.std()))
        samples.append(rm.logits[idx].copy())
        if st in (0, 1, 63, 127):
            g[f"forced_logits256_step{st}"] = rm.logits[:256].copy()
            g[f"forced_logits_sha_step{st}"] = np.frombuffer(sha(rm.logits).encode(), np.uint8)
        if st % 16 == 0:
            print("step", st, "fed", t, "argmax", toks[-1], "margin/std %.3f" % (margins[-1] / stds[-1]), "%.1fs" % (time.time() - t0), flush=True)
    rm.close()
    g["forced_tokens"] = np.array(toks, np.int64)
    g["forced_margins"] = np.array(margins, np.float32)
    g["forced_std"] = np.array(stds, np.float32)
    g["forced_samples"] = np.stack(samples)
    _add_to_npz("golden_cfg4.npz", g)


CENTERED_STEPS = 48


def make_forced_centered():
    """A token-sensitive full-size model: the cfg4 shapes and seeds with every Q4_K matrix centred (synth.make_layer_centered:
    block values d * scale * (q - 7.5)).  With the benchmark's own block distribution every Q4_K weight has a large positive
    mean and the network is close to rank one (two argmax ids whatever is fed); centred, the logits move by 5-8 of their
    standard deviations from one fed token to the next and the argmax follows the input.  48 distinct seeded ids are fed after
    the 2048 prefilled positions; stored per step: the reference's argmax, top-2 margin, logit spread and 64 strided logits."""
    cfg = dict(synth.QWEN3_4B)
    seed = SEEDS["cfg4"]
    layers = [synth.make_layer_centered(seed, i, cfg) for i in range(cfg["n_layers"])]
    head = synth.make_head(seed, cfg)
    emb = po.dequant(14, head["lm_head"]).reshape(cfg["vocab"], cfg["hidden"])
    rm = po.RefModel(cfg, layers, head, 2304, emb)
    for i in range(cfg["n_layers"]):
        k, v = synth.make_kv_prefill(seed, i, cfg, 2048)
        rm.set_kv(i, k, v)
    feed = forced_feed(seed, cfg["vocab"], 128)[:CENTERED_STEPS]
    idx = (np.arange(FORCED_SAMPLE, dtype=np.int64) * cfg["vocab"]) // FORCED_SAMPLE
    toks, margins, stds, samples = [], [], [], []
    t0 = time.time()
    for st, t in enumerate(feed):
        toks.append(rm.step(t))
        srt = np.sort(rm.logits)
        margins.append(float(srt[-1] - srt[-2]))
        stds.append(float(rm.logits.std()))
        samples.append(rm.logits[idx].copy())
        if st % 8 == 0:
            print("step", st, "fed", t, "argmax", toks[-1], "margin/std %.3f" % (margins[-1] / stds[-1]), "%.1fs" % (time.time() - t0), flush=True)
    rm.close()
    np.savez_compressed(os.path.join(OUT, "golden_cfg4_centered.npz"), feed=np.array(feed, np.int64), sample_index=idx,
                        tokens=np.array(toks, np.int64), margins=np.array(margins, np.float32), std=np.array(stds, np.float32),
                        samples=np.stack(samples))


if __name__ == "__main__":
    main()
