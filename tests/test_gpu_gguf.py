"""GPU: a model loaded from a .gguf file (ptm_model_load_gguf) decodes exactly like the same weights handed to
the decoder directly, and like the compiled reference's golden run."""
import numpy as np
import pytest

from conftest import bits
from prometorch_amd import gguf
from prometorch_amd.testing import gguf_writer, synth
from prometorch_amd._lib import PtmError

pytestmark = pytest.mark.gpu


def build_tiny(seeds):
    cfg = dict(synth.TINY)
    layers = [synth.make_layer(seeds["tiny"], i, cfg) for i in range(cfg["n_layers"])]
    head = synth.make_head(seeds["tiny"], cfg)
    kv = [synth.make_kv_prefill(seeds["tiny"], i, cfg, 19) for i in range(cfg["n_layers"])]
    return cfg, layers, head, kv


@pytest.mark.parametrize("tied", [True, False])
def test_gguf_model_decodes_like_direct_decoder(dev, seeds, golden, tmp_path, tied):
    from prometorch_amd.decode import Decoder
    cfg, layers, head, kv = build_tiny(seeds)
    path = str(tmp_path / "tiny.gguf")
    gguf_writer.model_to_gguf(path, cfg, layers, head, tied=tied, alignment=64)
    m = gguf.GGUFModel(path, max_seq=64, kv_fp16=False)
    for k in ("vocab", "hidden", "n_layers", "n_heads", "n_kv_heads", "head_dim", "inter"):
        assert m.cfg[k] == cfg[k], k
    assert m.cfg["tied"] == tied and abs(m.cfg["rope_base"] - cfg["rope_base"]) < 1 and abs(m.cfg["eps"] - cfg["eps"]) < 1e-12
    emb = None
    if not tied:  # an untied file gets an fp32 embedding table dequantised from token_embd
        from oracle import pyoracle as po
        emb = po.dequant(14, head["lm_head"]).reshape(cfg["vocab"], cfg["hidden"])
    d = Decoder(cfg, layers, head, max_seq=64, kv_fp16=False, embedding_f32=emb)
    for i, (k, v) in enumerate(kv):
        m.set_kv(i, k, v)
        d.set_kv(i, k, v)
    m.set_past_len(19)
    d.set_past_len(19)
    tm = td = 3
    for st in range(12):
        tm = m.step(tm)
        td = d.step(td)
        assert tm == td == int(golden["tiny_tokens"][st]), st
        assert np.array_equal(bits(m.logits()), bits(d.logits())), st
    assert m.greedy(tm, 8) == d.greedy(td, 8)
    m.close()
    d.close()


def test_gguf_model_refuses_what_it_cannot_run(dev, seeds, tmp_path):
    cfg, layers, head, _ = build_tiny(seeds)
    p = str(tmp_path / "phi3.gguf")
    gguf_writer.model_to_gguf(p, cfg, layers, head, arch="phi3")  # fused qkv / gate-up tensors, per-frequency factors: not a step built here
    with pytest.raises(PtmError) as e:
        gguf.GGUFModel(p, max_seq=64)
    assert e.value.code == -4
    # a tensor of the wrong shape
    bad = [dict(L) for L in layers]
    qt, W = bad[1]["down"]
    bad[1]["down"] = (qt, W[:-1])
    p2 = str(tmp_path / "short.gguf")
    gguf_writer.model_to_gguf(p2, cfg, bad, head)
    with pytest.raises(PtmError) as e:
        gguf.GGUFModel(p2, max_seq=64)
    assert e.value.code == -2
    # a missing tensor
    p3 = str(tmp_path / "missing.gguf")
    cfg3 = dict(cfg)
    cfg3["n_layers"] = 3
    gguf_writer.model_to_gguf(p3, cfg3, layers, head)
    with pytest.raises(PtmError) as e:
        gguf.GGUFModel(p3, max_seq=64)
    assert e.value.code == -10


def test_text_to_text_through_one_file(dev, po, seeds, tmp_path):
    """The whole path behind the C ABI from one .gguf file: chat template -> tokenizer -> prompt prefill -> sampled
    decode on the device -> text; the token stream is checked against the oracle's loop (step the prompt token by
    token, then penalise / sample / feed back with the same uniform draws)."""
    from prometorch_amd import ops
    from prometorch_amd.tokenizer import Tokenizer, chat_template
    cfg, layers, head, _ = build_tiny(seeds)
    tok_md = synth.make_tokenizer("gpt2", vocab_size=cfg["vocab"])
    assert len(tok_md["tokenizer.ggml.tokens"]) == cfg["vocab"]
    path = str(tmp_path / "chat.gguf")
    gguf_writer.model_to_gguf(path, cfg, layers, head, tokenizer=tok_md)
    f = gguf.GGUFFile(path)
    tk = Tokenizer.from_gguf(f)
    m = gguf.GGUFModel(path, max_seq=160, kv_fp16=True)
    text = chat_template(f.get_string("general.architecture"), "Hello there, what's 2+2?", system="Be brief.")
    ids = tk.encode(text)
    assert 20 < len(ids) < 100 and ids[0] == tok_md["tokenizer.ggml.tokens"].index("<|im_start|>")
    assert tk.decode(ids, skip_special=False) == text
    n_new, params = 24, (0.8, 40, 0.9, 1.1)
    us = ops.mt19937_uniforms(42, 0, n_new)
    first = m.prefill(ids[:-1])                 # everything but the last prompt token; its successor is resampled below
    m.sampling_begin(*params)
    got = m.sample(ids[-1], us)
    # oracle loop
    om = po.OracleModel(cfg, layers, head, 160, kv_fp16=True)
    for t in ids[:-1]:
        om.step(t)
    tok, generated = ids[-1], []
    for st in range(n_new):
        om.step(tok)
        lg = po.repetition_penalty(om.logits, generated, params[3]) if generated else om.logits
        tok, gap = po.sample_token(lg, params[0], params[1], params[2], us[st])
        if gap <= 1e-3:
            break   # the prefilled cache differs from the stepped one at the Q8-rounding-noise level: compare clear draws only
        assert got[st] == tok, (st, gap)
        generated.append(tok)
    assert len(generated) >= 8 and first >= 0
    reply = tk.decode(got)
    assert isinstance(reply, bytes) and len(reply) > 0
    m.close(); tk.close(); f.close()


def test_chat_is_the_manual_path_in_one_call(dev, seeds, tmp_path):
    """GGUFModel.chat = chat template + tokenizer + ptm_decode_generate with the file's stop tokens + decode."""
    from prometorch_amd import ops
    from prometorch_amd.tokenizer import Tokenizer, chat_template
    cfg, layers, head, _ = build_tiny(seeds)
    tok_md = synth.make_tokenizer("gpt2", vocab_size=cfg["vocab"])
    path = str(tmp_path / "chat.gguf")
    gguf_writer.model_to_gguf(path, cfg, layers, head, tokenizer=tok_md)
    m = gguf.GGUFModel(path, max_seq=160, kv_fp16=True)
    reply = m.chat("Hello there, what's 2+2?", system="Be brief.", max_new=24, temperature=0.8, top_k=40, top_p=0.9,
                   repeat_penalty=1.1, seed=42)
    assert isinstance(reply, str)
    with gguf.GGUFFile(path) as f:
        tk = Tokenizer.from_gguf(f)
        ids = tk.encode(chat_template(f.get_string("general.architecture"), "Hello there, what's 2+2?",
                                      model_name=f.get_string("general.name") or "", system="Be brief."))
        stops = sorted({tk.special_ids()["eos"]} | {tk.encode(t, use_bos=False)[0] for t in m.STOP_TOKENS
                                                    if len(tk.encode(t, use_bos=False)) == 1})
        m.set_past_len(0)
        want = m.generate(ids, ops.mt19937_uniforms(42, 0, 24), 0.8, 40, 0.9, 1.1, stop_ids=[s for s in stops if s >= 0])
        assert reply == tk.decode(want).decode("utf-8", errors="replace")
        assert all(t not in stops for t in want)
        # a second turn starts from an empty context again and, with the same seed, repeats the first
        assert m.chat("Hello there, what's 2+2?", system="Be brief.", max_new=24, temperature=0.8, top_k=40, top_p=0.9,
                      repeat_penalty=1.1, seed=42) == reply
        tk.close()
    with pytest.raises(ValueError):
        m.chat("x " * 400, max_new=8)
    m.close()


LOADER_CASES = ("qwen3_tied", "qwen3_untied", "llama", "llama_scaled", "qwen2", "gemma3")


@pytest.mark.parametrize("case", LOADER_CASES)
def test_loader_agrees_with_the_references_own_loader(dev, seeds, tmp_path, case):
    """golden_loader.npz: the same files (byte-identical: sha256 checked) as the REFERENCE's GGUFModel::load read them -
    its config fields, the type it registered for every matrix, and 8 steps of its forward_decode_cpu logits.
    ptm_model_load_gguf must arrive at the same configuration, the same types, and logits within the decode bars."""
    import hashlib
    import os
    import sys
    from conftest import GOLDEN_DIR
    sys.path.insert(0, GOLDEN_DIR)
    import make_golden as mg   # the case list and the fed tokens live beside the script that wrote the fixture
    g = np.load(os.path.join(GOLDEN_DIR, "golden_loader.npz"), allow_pickle=False)
    name, cfg, layers, head, kw = [c for c in mg.loader_cases(seeds["tiny"]) if c[0] == case][0]
    path = str(tmp_path / (case + ".gguf"))
    gguf_writer.model_to_gguf(path, cfg, layers, head, **kw)
    assert hashlib.sha256(open(path, "rb").read()).hexdigest() == bytes(g[case + "_sha"]).decode(), "not the file the reference read"
    m = gguf.GGUFModel(path, max_seq=64, kv_fp16=False)
    from oracle import pyoracle as po
    ref_cfg = dict(zip(po.LOADED_INT_FIELDS, (int(v) for v in g[case + "_ints"])))
    ref_cfg.update(zip(po.LOADED_FLOAT_FIELDS, (float(v) for v in g[case + "_floats"])))
    for k in ("vocab", "hidden", "n_layers", "n_heads", "n_kv_heads", "head_dim", "inter", "swa_window"):
        assert m.cfg[k] == ref_cfg[k], (k, m.cfg[k], ref_cfg[k])
    assert m.cfg["tied"] == bool(ref_cfg["tied"])
    assert m.cfg["rope_interleaved"] == (not ref_cfg["rope_neox"])
    assert m.cfg["scale_embeddings"] == bool(ref_cfg["scale_embeddings"]) and m.cfg["ffn_gelu"] == bool(ref_cfg["ffn_gelu"])
    assert np.float32(m.cfg["rope_base"]) == np.float32(ref_cfg["rope_base"]) and np.float32(m.cfg["eps"]) == np.float32(ref_cfg["eps"])
    assert np.float32(m.cfg["rope_scale"] or 1.0) == np.float32(ref_cfg["rope_scale"])
    if ref_cfg["swa_window"]:
        assert m.cfg["swa_pattern"] == ref_cfg["swa_pattern"]
        assert np.float32(m.cfg["rope_swa_base"]) == np.float32(ref_cfg["rope_swa_base"])
    types = g[case + "_types"]
    for i in range(cfg["n_layers"]):
        Ld = m.layer(i)
        got = [getattr(Ld, n).ggml_type for n in ("q", "k", "v", "o", "gate", "up", "down")]
        assert got == [int(t) for t in types[7 * i:7 * i + 7]], (i, got)
        assert bool(Ld.q_norm) == bool(ref_cfg["has_qk_norm"]) and bool(Ld.post_attn_norm) == bool(ref_cfg["has_post_norm"])
    for i in range(cfg["n_layers"]):
        m.set_kv(i, *synth.make_kv_prefill(seeds["tiny"], i, cfg, 19))
    m.set_past_len(19)
    errs = []
    for st, tok in enumerate(mg.LOADER_FEED):
        t = m.step(tok)
        ref = g[case + "_logits"][st]
        errs.append(float(np.abs(m.logits() - ref).max() / ref.std()))
        assert t == int(g[case + "_tokens"][st]), (st, errs[-1])
    errs = np.asarray(errs)
    # llama-style models (no QK-norm) amplify the Q8 rounding noise of single steps more: their bars are the llama tests' own
    loose = case.startswith("llama") or case == "qwen2"
    assert errs.max() <= (5e-2 if loose else 2e-2), errs
    assert int((errs > 1e-3).sum()) <= (8 if loose else 2), errs
    m.close()
