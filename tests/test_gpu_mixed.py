"""GPU: layers of different quant-type mixes in one model (synth.tiny_mixed) -- the Q4_K_M mix, an all-Q4_K layer
(about half the layers of a real Q4_K_M file keep attn_v and ffn_down in Q4_K) and an odd mix that reaches the
remaining branches of the step (Q6_K q beside Q4_K k/v, Q6_K o and gate) -- against the compiled reference's golden
run, the oracle, the prompt path and a .gguf round trip.  Bars as in test_gpu_decode / test_gpu_prefill."""
import os

import numpy as np
import pytest

from conftest import GOLDEN_DIR, bits
from prometorch_amd import gguf
from prometorch_amd.testing import gguf_writer, synth
from test_gpu_decode import LOGIT_TOL, LOGIT_TOL_FLIP, check_step_errors
from test_gpu_prefill import check_kv_rows, check_logits, follow

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def golden_mixed():
    return np.load(os.path.join(GOLDEN_DIR, "golden_mixed.npz"))


def mixed_with_cache(seeds, n=19):
    cfg, layers, head = synth.tiny_mixed(seeds["tiny"])
    return cfg, layers, head, [synth.make_kv_prefill(seeds["tiny"], i, cfg, n) for i in range(cfg["n_layers"])]


@pytest.mark.parametrize("use_graph", [False, True])
def test_mixed_decode_fp32_kv_vs_reference_golden(dev, golden_mixed, seeds, use_graph):
    from prometorch_amd.decode import Decoder
    cfg, layers, head, kv = mixed_with_cache(seeds)
    dec = Decoder(cfg, layers, head, max_seq=64, kv_fp16=False, use_graph=use_graph)
    for i, (k, v) in enumerate(kv):
        dec.set_kv(i, k, v)
    dec.set_past_len(19)
    errs = []
    for st in range(12):
        tok = dec.step(synth.MIXED_FEED[st])
        ref = golden_mixed["logits"][st]
        errs.append(np.abs(dec.logits() - ref).max() / ref.std())
        assert tok == int(golden_mixed["tokens"][st]), st
    check_step_errors(errs)
    dec.close()


def test_mixed_decode_fp16_kv_vs_oracle(dev, po, seeds):
    from prometorch_amd.decode import Decoder
    cfg, layers, head, kv = mixed_with_cache(seeds)
    om = po.OracleModel(cfg, layers, head, 64, kv_fp16=True)
    dec = Decoder(cfg, layers, head, max_seq=64, kv_fp16=True, use_graph=True)
    for i, (k, v) in enumerate(kv):
        om.set_kv(i, k, v)
        dec.set_kv(i, k, v)
    dec.set_past_len(19)
    errs = []
    for st in range(24):
        tok_o = om.step(synth.MIXED_FEED[st])
        tok_g = dec.step(synth.MIXED_FEED[st])
        errs.append(np.abs(dec.logits() - om.logits).max() / om.logits.std())
        assert tok_g == tok_o, st
    # The all-Q4_K layer rounds the inputs of all seven projections to int8 where the Q4_K_M mix rounds five, and
    # the model is a layer deeper: steps in which one activation lands on the other side of a rounding boundary
    # (see test_gpu_decode) are more frequent here (3 of 24 measured, up to 1.4e-2), so the count of such steps is
    # not bounded, only their size, and the typical step must hold the tight bar
    errs = np.asarray(errs)
    assert errs.max() <= LOGIT_TOL_FLIP and np.median(errs) <= LOGIT_TOL, errs
    dec.close()


@pytest.mark.parametrize("kv_fp16", [True, False])
@pytest.mark.parametrize("pos0,n,chunk", [(0, 23, 0), (19, 12, 5)])
def test_mixed_prefill_vs_oracle_token_by_token(dev, po, seeds, kv_fp16, pos0, n, chunk):
    from prometorch_amd.decode import Decoder
    cfg, layers, head = synth.tiny_mixed(seeds["tiny"])
    om = po.OracleModel(cfg, layers, head, 64, kv_fp16=kv_fp16)
    dec = Decoder(cfg, layers, head, max_seq=64, kv_fp16=kv_fp16, use_graph=True)
    if pos0:
        for i in range(cfg["n_layers"]):
            k, v = synth.make_kv_prefill(seeds["tiny"], i, cfg, pos0)
            om.set_kv(i, k, v)
            dec.set_kv(i, k, v)
        dec.set_past_len(pos0)
    prompt = [int(t) for t in synth.rng_for(68, pos0, n).integers(0, cfg["vocab"], n)]
    for t in prompt:
        tok_o = om.step(t)
    tok_g = dec.prefill(prompt, chunk_rows=chunk)
    for li in range(cfg["n_layers"]):
        for nm, gpu_c, cpu_c in (("k", dec.k_cache[li], om.k_cache[li]), ("v", dec.v_cache[li], om.v_cache[li])):
            check_kv_rows(gpu_c[pos0:pos0 + n].float().cpu().numpy(), cpu_c[pos0:pos0 + n], li, nm)
    check_logits(dec.logits(), om.logits, tok_g, tok_o, "prefill")
    follow(dec, om, tok_o, 6)
    dec.close()


def test_mixed_gguf_file_decodes_like_direct_decoder(dev, seeds, golden_mixed, tmp_path):
    from prometorch_amd.decode import Decoder
    cfg, layers, head, kv = mixed_with_cache(seeds)
    path = str(tmp_path / "tiny_mixed.gguf")
    gguf_writer.model_to_gguf(path, cfg, layers, head)
    m = gguf.GGUFModel(path, max_seq=64, kv_fp16=False)
    d = Decoder(cfg, layers, head, max_seq=64, kv_fp16=False)
    for i, (k, v) in enumerate(kv):
        m.set_kv(i, k, v)
        d.set_kv(i, k, v)
    m.set_past_len(19)
    d.set_past_len(19)
    for st in range(12):
        tm, td = m.step(synth.MIXED_FEED[st]), d.step(synth.MIXED_FEED[st])
        assert tm == td == int(golden_mixed["tokens"][st]), st
        assert np.array_equal(bits(m.logits()), bits(d.logits())), st
    m.close()
    d.close()


# ---- the dispatcher's other formats (Q8_0, Q5_K, Q5_0) through the decoder: plain kernels, prompts stepped token by token ----
@pytest.fixture(scope="module")
def golden_formats_model():
    return np.load(os.path.join(GOLDEN_DIR, "golden_formats_model.npz"))


@pytest.mark.parametrize("use_graph", [False, True])
def test_other_formats_decode_fp32_kv_vs_reference_golden(dev, golden_formats_model, seeds, use_graph):
    from prometorch_amd.decode import Decoder
    cfg, layers, head = synth.tiny_formats(seeds["tiny"])
    dec = Decoder(cfg, layers, head, max_seq=64, kv_fp16=False, use_graph=use_graph)
    for i in range(cfg["n_layers"]):
        dec.set_kv(i, *synth.make_kv_prefill(seeds["tiny"], i, cfg, 19))
    dec.set_past_len(19)
    errs = []
    for st in range(12):
        tok = dec.step(synth.MIXED_FEED[st])
        ref = golden_formats_model["logits"][st]
        errs.append(np.abs(dec.logits() - ref).max() / ref.std())
        assert tok == int(golden_formats_model["tokens"][st]), st
    check_step_errors(errs)
    dec.close()


@pytest.mark.parametrize("kv_fp16", [True, False])
def test_other_formats_prompt_and_generation_vs_oracle(dev, po, seeds, kv_fp16):
    """A decoder holding Q8_0 / Q5_K / Q5_0 matrices has no row-batched GEMM: its prefill steps the prompt, so the
    logits and cache rows agree with the oracle as closely as single steps do."""
    from prometorch_amd.decode import Decoder
    cfg, layers, head = synth.tiny_formats(seeds["tiny"])
    om = po.OracleModel(cfg, layers, head, 64, kv_fp16=kv_fp16)
    dec = Decoder(cfg, layers, head, max_seq=64, kv_fp16=kv_fp16, use_graph=True)
    prompt = [int(t) for t in synth.rng_for(70).integers(0, cfg["vocab"], 17)]
    for t in prompt:
        tok_o = om.step(t)
    tok_g = dec.prefill(prompt)
    assert tok_g == tok_o
    assert np.abs(dec.logits() - om.logits).max() <= LOGIT_TOL_FLIP * om.logits.std()
    for li in range(cfg["n_layers"]):
        k_gpu = dec.k_cache[li][:17].float().cpu().numpy()
        assert np.abs(k_gpu - om.k_cache[li][:17]).max() <= 2e-3 * np.abs(om.k_cache[li][:17]).max()
    errs = []
    for st in range(10):
        tok_o = om.step(tok_o)
        tok_g = dec.step(tok_g)
        errs.append(np.abs(dec.logits() - om.logits).max() / om.logits.std())
        assert tok_g == tok_o, st
    check_step_errors(errs)
    dec.close()


def test_other_formats_gguf_file_decodes_like_direct_decoder(dev, seeds, golden_formats_model, tmp_path):
    from prometorch_amd.decode import Decoder
    cfg, layers, head = synth.tiny_formats(seeds["tiny"])
    path = str(tmp_path / "tiny_formats.gguf")
    gguf_writer.model_to_gguf(path, cfg, layers, head)
    m = gguf.GGUFModel(path, max_seq=64, kv_fp16=False)
    d = Decoder(cfg, layers, head, max_seq=64, kv_fp16=False)
    for i in range(cfg["n_layers"]):
        k, v = synth.make_kv_prefill(seeds["tiny"], i, cfg, 19)
        m.set_kv(i, k, v)
        d.set_kv(i, k, v)
    m.set_past_len(19)
    d.set_past_len(19)
    for st in range(12):
        tm, td = m.step(synth.MIXED_FEED[st]), d.step(synth.MIXED_FEED[st])
        assert tm == td == int(golden_formats_model["tokens"][st]), st
        assert np.array_equal(bits(m.logits()), bits(d.logits())), st
    m.close()
    d.close()


@pytest.mark.parametrize("lm_type,tied", [(8, True), (13, True), (8, False), (12, True)])
def test_other_lm_head_types_from_gguf_vs_oracle(dev, po, seeds, tmp_path, lm_type, tied):
    """token_embd / output in Q8_0, Q5_K or Q4_K (a Q8_0 file keeps both in Q8_0): the loader dequantises the embedding
    table to fp32 on the device and the vocabulary projection goes through the dispatcher."""
    cfg, layers, head = synth.tiny_formats(seeds["tiny"])
    head = dict(head)
    head["lm_head_type"] = lm_type
    head["lm_head"] = synth.make_weight(synth.rng_for(seeds["tiny"], 3, lm_type), lm_type, cfg["vocab"], cfg["hidden"])
    emb = po.dequant(lm_type, head["lm_head"]).reshape(cfg["vocab"], cfg["hidden"])
    om = po.OracleModel(cfg, layers, head, 64, kv_fp16=False, embedding=emb)
    path = str(tmp_path / "lm.gguf")
    gguf_writer.model_to_gguf(path, cfg, layers, head, tied=tied)
    m = gguf.GGUFModel(path, max_seq=64, kv_fp16=False)
    errs, tok_o = [], 5
    tok_g = 5
    for st in range(10):
        tok_o = om.step(tok_o)
        tok_g = m.step(tok_g)
        errs.append(np.abs(m.logits() - om.logits).max() / om.logits.std())
        assert tok_g == tok_o, st
    check_step_errors(errs)
    m.close()


@pytest.mark.parametrize("seed", range(10))
def test_random_architectures_decode_and_prefill_vs_oracle(dev, po, seed):
    """Ten random combinations of the architectural switches: 6 decode steps behind a random number of cached positions
    and a 9-token prompt behind those, against the oracle (fp16 cache on even seeds, fp32 on odd ones).  Bars: every
    step within LOGIT_TOL_FLIP, the median within LOGIT_TOL, tokens equal where the oracle's margin exceeds twice the error."""
    from prometorch_amd.decode import Decoder
    from test_gpu_decode import LOGIT_TOL, LOGIT_TOL_FLIP
    from test_gpu_prefill import logit_errors
    cfg, layers, head = synth.random_model(seed)
    print("seed", seed, {k: v for k, v in cfg.items() if k not in ("vocab", "eps")},
          "qk_norm", layers[0]["q_norm"] is not None, "bias", "q_bias" in layers[0],
          "post", [n for n in ("post_attn_norm", "post_ffn_norm") if n in layers[0]], flush=True)
    kv_fp16 = seed % 2 == 0
    past = int(synth.rng_for(99, seed).integers(0, 60))
    om = po.OracleModel(cfg, layers, head, 96, kv_fp16=kv_fp16)
    dec = Decoder(cfg, layers, head, max_seq=96, kv_fp16=kv_fp16, use_graph=True)
    if past:
        for i in range(cfg["n_layers"]):
            k, v = synth.make_kv_prefill(1000 + seed, i, cfg, past)
            om.set_kv(i, k, v)
            dec.set_kv(i, k, v)
        dec.set_past_len(past)
    tok, errs = 5, []
    for st in range(6):
        tok_o = om.step(tok)
        tok_g = dec.step(tok)
        err, rms, margin = logit_errors(dec.logits(), om.logits)
        errs.append(err)
        if margin > 2 * err:
            assert tok_g == tok_o, (st, margin, err)
        tok = tok_o
    prompt = [int(t) for t in synth.rng_for(100, seed).integers(0, cfg["vocab"], 9)]
    for t in prompt:
        tok_o = om.step(t)
    tok_g = dec.prefill(prompt)
    err, rms, margin = logit_errors(dec.logits(), om.logits)
    errs.append(err)
    if margin > 2 * err:
        assert tok_g == tok_o, ("prefill", margin, err)
    errs = np.asarray(errs)
    print("logit err/std", np.array2string(errs, precision=2), flush=True)
    assert errs.max() <= LOGIT_TOL_FLIP and np.median(errs) <= LOGIT_TOL, errs
    dec.close()
