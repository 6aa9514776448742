"""GPU parity of the whole decode step (ptm_decode_*): logits against the CPU oracle / the
compiled reference's golden logits, greedy token ids identical."""
import time

import numpy as np
import torch
import pytest

from conftest import bits
from prometorch_amd.testing import synth

pytestmark = pytest.mark.gpu

LOGIT_TOL = 1e-3  # max |logit_gpu - logit_cpu| / std(logits_cpu)
# The Q4_K path quantises every activation vector to int8 (reference semantics).  GPU and CPU sum attention and
# norms in different orders, so an activation can differ by one ulp; when it sits exactly on a rounding boundary
# of the Q8 rule it then lands on the neighbouring int8 level (1/127 of its block's maximum) and the logits of
# THAT step move by up to ~1e-2 of their spread.  Such steps are rare (measured: 1 in 24 on the tiny model with
# one summation order, 0 with another) and do not carry over; they are bounded by LOGIT_TOL_FLIP, at most
# MAX_FLIP_STEPS of them are accepted per run, and the greedy tokens must be identical regardless.
LOGIT_TOL_FLIP = 2e-2
MAX_FLIP_STEPS = 2


def check_step_errors(errs):
    errs = np.asarray(errs)
    assert errs.max() <= LOGIT_TOL_FLIP, (int(errs.argmax()), float(errs.max()))
    assert int((errs > LOGIT_TOL).sum()) <= MAX_FLIP_STEPS, errs


def build_tiny(seeds):
    cfg = dict(synth.TINY)
    layers = [synth.make_layer(seeds["tiny"], i, cfg) for i in range(cfg["n_layers"])]
    head = synth.make_head(seeds["tiny"], cfg)
    kv = [synth.make_kv_prefill(seeds["tiny"], i, cfg, 19) for i in range(cfg["n_layers"])]
    return cfg, layers, head, kv


@pytest.mark.parametrize("use_graph", [False, True])
def test_tiny_decode_fp32_kv_vs_reference_golden(dev, golden, seeds, use_graph):
    """fp32 KV cache: the configuration the reference's forward_decode_cpu runs; golden logits are the
    compiled reference's."""
    from prometorch_amd.decode import Decoder
    cfg, layers, head, kv = build_tiny(seeds)
    dec = Decoder(cfg, layers, head, max_seq=64, kv_fp16=False, use_graph=use_graph)
    for i, (k, v) in enumerate(kv):
        dec.set_kv(i, k, v)
    dec.set_past_len(19)
    tok = 3
    errs = []
    for st in range(12):
        tok = dec.step(tok)
        ref = golden["tiny_logits"][st]
        errs.append(np.abs(dec.logits() - ref).max() / ref.std())
        assert tok == int(golden["tiny_tokens"][st]), st
    check_step_errors(errs)
    dec.close()


@pytest.mark.parametrize("embedding_f32", [False, True])
def test_tiny_decode_fp16_kv_vs_oracle_and_chained_greedy(dev, po, seeds, embedding_f32):
    from prometorch_amd.decode import Decoder
    cfg, layers, head, kv = build_tiny(seeds)
    om = po.OracleModel(cfg, layers, head, 64, kv_fp16=True)
    emb = po.dequant(14, head["lm_head"]).reshape(cfg["vocab"], cfg["hidden"]) if embedding_f32 else None
    dec = Decoder(cfg, layers, head, max_seq=64, kv_fp16=True, use_graph=True, embedding_f32=emb)
    dec2 = Decoder(cfg, layers, head, max_seq=64, kv_fp16=True, use_graph=True, embedding_f32=emb)
    for i, (k, v) in enumerate(kv):
        om.set_kv(i, k, v)
        dec.set_kv(i, k, v)
        dec2.set_kv(i, k, v)
    dec.set_past_len(19)
    dec2.set_past_len(19)
    tok_o = tok_g = 3
    want, errs = [], []
    for st in range(24):
        tok_o = om.step(tok_o)
        tok_g = dec.step(tok_g)
        want.append(tok_o)
        errs.append(np.abs(dec.logits() - om.logits).max() / om.logits.std())
        assert tok_g == tok_o, st
    check_step_errors(errs)
    # the same 24 tokens produced without host round trips (device-side feedback, graph replays)
    assert dec2.greedy(3, 24) == want
    # KV rows appended by the GPU are the fp16 rounding of the oracle's rows
    k_gpu = dec.k_cache[0][19:43].float().cpu().numpy()
    k_cpu = om.k_cache[0][19:43]
    assert np.abs(k_gpu - k_cpu).max() <= 2e-3 * np.abs(k_cpu).max()
    dec.close()
    dec2.close()


@pytest.mark.parametrize("use_graph", [False, True])
def test_steps_that_resume_on_the_device_equal_steps_that_reset(dev, seeds, use_graph):
    """A greedy step whose input is the token the previous greedy run produced starts from the device's own token, position
    and step index (no scalar-setting launch); any other input, a chained run, a sampled run, a prompt or a position reset
    in between must put the state back.  One decoder runs a mixed sequence of those; a second one has its position set
    before every single step, which forces the reset path each time.  Tokens and logits must be identical."""
    from prometorch_amd.decode import Decoder
    cfg, layers, head, kv = build_tiny(seeds)
    a = Decoder(cfg, layers, head, max_seq=96, kv_fp16=True, use_graph=use_graph)
    b = Decoder(cfg, layers, head, max_seq=96, kv_fp16=True, use_graph=use_graph)
    for i, (k, v) in enumerate(kv):
        a.set_kv(i, k, v)
        b.set_kv(i, k, v)
    pos = 19
    a.set_past_len(pos)

    def b_step(tok):
        nonlocal pos
        b.set_past_len(pos)
        out = b.step(tok)
        pos += 1
        return out

    def same_logits():
        assert np.array_equal(a.logits(), b.logits())

    tok = 3
    for _ in range(5):                       # resumed after the first
        ta, tb = a.step(tok), b_step(tok)
        assert ta == tb
        same_logits()
        tok = ta
    forced = (tok + 7) % cfg["vocab"]        # not the token the device holds: reset
    ta, tb = a.step(forced), b_step(forced)
    assert ta == tb
    same_logits()
    tok = ta
    chain = a.greedy(tok, 6)                 # a chained run resumes as well, and leaves the device in step with the host
    for t in chain:
        tok = b_step(tok)
        assert tok == t
    for _ in range(3):
        ta, tb = a.step(tok), b_step(tok)
        assert ta == tb
        same_logits()
        tok = ta
    prompt = [5, 9, 2, 11, 7, 1, 30, 4, 8, 6, 12, 3, 17, 21, 2, 9, 40]   # a prompt in between: 17 rows
    ta = a.prefill(prompt)
    b.set_past_len(pos)
    tb = b.prefill(prompt)
    pos += len(prompt)
    assert ta == tb
    tok = ta
    for _ in range(4):
        ta, tb = a.step(tok), b_step(tok)
        assert ta == tb
        same_logits()
        tok = ta
    a.set_past_len(25)                       # rewind: the same token id as the device holds, but another position
    pos = 25
    for _ in range(3):
        ta, tb = a.step(tok), b_step(tok)
        assert ta == tb
        same_logits()
        tok = ta
    a.close()
    b.close()


def test_decode_kv_overflow_and_bad_token_are_errors(dev, seeds):
    from prometorch_amd.decode import Decoder
    from prometorch_amd._lib import PtmError
    cfg, layers, head, kv = build_tiny(seeds)
    dec = Decoder(cfg, layers, head, max_seq=32, kv_fp16=True, use_graph=False)
    dec.set_past_len(30)
    dec.step(1)
    dec.step(1)
    with pytest.raises(PtmError) as e:   # position 32 does not exist
        dec.step(1)
    assert e.value.code == -6
    with pytest.raises(PtmError):
        dec.set_past_len(32)
    dec.set_past_len(0)
    with pytest.raises(PtmError):
        dec.step(cfg["vocab"])           # token id outside the table
    dec.close()


def test_cfg4_qwen3_4b_shape_128_greedy_tokens(dev, po, golden_cfg4, seeds):
    """Full size: 36 layers, fp16 KV prefilled to 2048, 128 greedy steps.  Every step is compared
    with the CPU oracle run beside it (same fp16 rounding of appended K/V rows): logits within
    LOGIT_TOL_FULL of std and identical token; the 128 ids must also equal the ids the compiled
    reference produced with its fp32 KV rows (golden)."""
    from prometorch_amd.decode import Decoder
    # measured on MI355X: worst logit error 3.3e-3 of the logits' spread over the 128 steps (a step whose activations sit on a
    # Q8 rounding boundary; typical steps ~1e-5), worst branch error 3.4e-3; the bars are three times that and more
    LOGIT_TOL_FULL = 1e-2
    RESID_TOL = 2e-2    # max |residual_gpu - residual_cpu| / rms(residual), any layer, either branch
    BRANCH_TOL = 2e-2   # rms error of one branch's own output over its rms
    cfg = dict(synth.QWEN3_4B)
    seed = seeds["cfg4"]
    t0 = time.time()
    layers = [synth.make_layer(seed, i, cfg) for i in range(cfg["n_layers"])]
    head = synth.make_head(seed, cfg)
    print("model generated in %.1fs" % (time.time() - t0), flush=True)
    om = po.OracleModel(cfg, layers, head, 2304, kv_fp16=True)
    dec = Decoder(cfg, layers, head, max_seq=2304, kv_fp16=True, use_graph=True)
    for i in range(cfg["n_layers"]):
        k, v = synth.make_kv_prefill(seed, i, cfg, 2048)
        dec.set_kv(i, k, v)
        om.set_kv(i, k, v)
    dec.set_past_len(2048)
    want_ref = [int(t) for t in golden_cfg4["tokens"]]
    to = tg = 1
    got, worst_err, min_margin = [], 0.0, 1e9
    branch_errs, worst_resid = [], 0.0
    for st in range(128):
        if st in (0, 127):
            # the first and the last step layer by layer: the residual stream after every attention branch and after every
            # feed-forward branch, and each branch's own contribution (so that an error in gate / up / down - 70 % of the
            # bytes, but a small part of the residual's magnitude in this model - cannot hide behind the residual)
            to, tr_o = om.step_trace(to)
            tg, tr_g = dec.step_trace(tg)
            prev_o = prev_g = None
            for li in range(cfg["n_layers"]):
                for br in (0, 1):
                    ro, rg = tr_o[li, br].astype(np.float64), tr_g[li, br].astype(np.float64)
                    resid_err = np.abs(rg - ro).max() / np.sqrt((ro ** 2).mean())
                    worst_resid = max(worst_resid, resid_err)
                    assert resid_err <= RESID_TOL, (st, li, br, resid_err)
                    if prev_o is not None:
                        do, dg = ro - prev_o, rg - prev_g   # what this branch added
                        berr = np.sqrt(((dg - do) ** 2).mean()) / np.sqrt((do ** 2).mean())
                        branch_errs.append((berr, st, li, br))
                        assert berr <= BRANCH_TOL, (st, li, br, berr)
                    prev_o, prev_g = ro, rg
        else:
            to = om.step(to)
            tg = dec.step(tg)
        got.append(tg)
        sd = float(om.logits.std())
        err = float(np.abs(dec.logits() - om.logits).max()) / sd
        srt = np.sort(om.logits)
        margin = float(srt[-1] - srt[-2]) / sd
        worst_err, min_margin = max(worst_err, err), min(min_margin, margin)
        if st % 16 == 0:
            print("step %3d token %6d  logit err/std %.2e  top-2 margin/std %.3f  (%.0fs)" % (st, tg, err, margin, time.time() - t0), flush=True)
        assert tg == to, f"token mismatch at step {st}: gpu {tg} vs oracle {to} (margin/std {margin:.4f}, err/std {err:.2e})"
        assert err <= LOGIT_TOL_FULL, (st, err)
    print("worst logit err/std %.2e, min top-2 margin/std %.3f" % (worst_err, min_margin), flush=True)
    print("worst residual error %.2e" % worst_resid, flush=True)
    print("worst branch error (rms of the branch's own output): %.2e at step %d layer %d %s" %
          (max(branch_errs)[0], max(branch_errs)[1], max(branch_errs)[2], "ffn" if max(branch_errs)[3] else "attention"), flush=True)
    assert got == want_ref, "GPU (fp16 KV) ids differ from the compiled reference's (fp32 KV) ids"
    # device-chained generation (no host round trip between tokens) reproduces the same ids
    dec.set_past_len(2048)
    assert dec.greedy(1, 128) == want_ref
    dec.close()


def test_padded_row_strides_are_honoured(dev, seeds):
    """Every matrix with 16 bytes of padding behind each row: the decode step and the prompt path read each matrix
    with its descriptor's stride, so logits are bit-identical to the dense layout; q / k strides that differ are refused."""
    from prometorch_amd import _lib
    from prometorch_amd.decode import Decoder
    cfg, layers, head, kv = build_tiny(seeds)
    padded = []
    for Ld in layers:
        P = dict(Ld)
        for name in ("q", "k", "v", "o", "gate", "up", "down"):
            qt, W = Ld[name]
            P[name] = (qt, np.ascontiguousarray(np.pad(W, ((0, 0), (0, 16)), constant_values=0xA5)))
        padded.append(P)
    outs = []
    for ls in (layers, padded):
        dec = Decoder(cfg, ls, head, max_seq=64, kv_fp16=True, use_graph=True)
        for i, (k, v) in enumerate(kv):
            dec.set_kv(i, k, v)
        dec.set_past_len(19)
        toks, lg = [], []
        t = 3
        for _ in range(4):
            t = dec.step(t)
            toks.append(t)
            lg.append(dec.logits())
        t = dec.prefill([5, 9, 200, 31, 7, 7, 64, 2])
        toks.append(t)
        lg.append(dec.logits())
        outs.append((toks, lg))
        dec.close()
    assert outs[0][0] == outs[1][0]
    for a, b in zip(outs[0][1], outs[1][1]):
        assert np.array_equal(bits(a), bits(b))
    bad = [dict(L) for L in padded]
    bad[0]["k"] = layers[0]["k"]   # q padded, k dense: one launch cannot serve two strides
    with pytest.raises(_lib.PtmError) as e:
        Decoder(cfg, bad, head, max_seq=64, kv_fp16=True, use_graph=True)
    assert e.value.code == -2


@pytest.mark.parametrize("use_graph", [False, True])
def test_longrope_factors_decode_vs_reference_golden(dev, seeds, use_graph):
    """phi3-style LongRoPE terms in the decoder's rotation table (per-frequency factors switching from the short to the long
    set inside the run, attn_factor): 12 steps against the compiled reference's golden_longrope.npz; and the graph-state
    query reports a captured step."""
    import os
    import sys
    from conftest import GOLDEN_DIR
    sys.path.insert(0, GOLDEN_DIR)
    import make_golden as mg
    from prometorch_amd.decode import Decoder
    g = np.load(os.path.join(GOLDEN_DIR, "golden_longrope.npz"), allow_pickle=False)
    cfg = mg.longrope_cfg(seeds["tiny"])
    layers = [synth.make_layer(seeds["tiny"], i, cfg) for i in range(cfg["n_layers"])]
    head = synth.make_head(seeds["tiny"], cfg)
    dec = Decoder(cfg, layers, head, max_seq=64, kv_fp16=False, use_graph=use_graph)
    for i in range(cfg["n_layers"]):
        dec.set_kv(i, *synth.make_kv_prefill(seeds["tiny"], i, cfg, 19))
    dec.set_past_len(19)
    assert dec.L.ptm_decode_graph_state(dec.h, 0) == 0
    tok, errs = 3, []
    for st in range(12):
        tok = dec.step(tok)
        ref = g["logits"][st]
        errs.append(np.abs(dec.logits() - ref).max() / ref.std())
        assert tok == int(g["tokens"][st]), (st, errs[-1])
    check_step_errors(errs)
    assert dec.L.ptm_decode_graph_state(dec.h, 0) == (1 if use_graph else 0)
    assert dec.L.ptm_decode_graph_state(dec.h, 1) == 0   # no sampled step has run
    dec.close()


@pytest.mark.parametrize("kv_fp16", [True, False])
def test_cfg4_qwen3_4b_shape_teacher_forced_128_distinct_ids(dev, po, golden_cfg4, seeds, kv_fp16):
    """The greedy run of the cfg4 model alternates between two ids (133268, 125944), so its 128 identical tokens see two
    embedding rows and near-identical new cache rows.  Here the same full-size model (36 layers, cache prefilled to 2048) is
    fed 128 DISTINCT seeded ids, and after every step the rows the oracle appended are copied into the GPU cache, so that
    each step is a comparison of ONE step on identical inputs (without that, the rows appended at an unstable step - below -
    differ and every later step inherits the difference: median 6.8e-3 instead of 1e-3).  Every step is compared with the
    oracle beside it and three steps layer by layer; with an fp32 cache (the reference's own arithmetic: its CPU cache rows
    are fp32) also with what the compiled reference produced for the same feed (forced_* of golden_cfg4.npz: argmax, 64
    strided logits per step, the first 256 logits of four steps).
    Unstable steps: this model is close to rank one (every Q4_K weight of the benchmark's block distribution has a large
    positive mean), its logits point along +u or -u, and on a few of the 128 inputs the coefficient is so small that the
    int8 rounding of one activation decides the sign: the logits then differ by up to 11 spreads between any two evaluations
    (measured: fp32 cache step 48, GPU against oracle AND against the reference; fp16 cache steps 22, 29, 48).  Bars: all but
    MAX_UNSTABLE steps within LOGIT_TOL of the spread (measured: all but 3 / 1), median below MEDIAN_TOL (measured 1.1e-3 /
    7.4e-4), the same argmax on every other step whose top-2 margin exceeds twice LOGIT_TOL."""
    from prometorch_amd.decode import Decoder
    if "forced_feed" not in golden_cfg4.files:
        pytest.skip("golden_cfg4.npz holds no teacher-forced run")
    LOGIT_TOL, MEDIAN_TOL, MAX_UNSTABLE, RESID_TOL = 1e-2, 3e-3, 5, 2e-2
    cfg = dict(synth.QWEN3_4B)
    seed = seeds["cfg4"]
    t0 = time.time()
    layers = [synth.make_layer(seed, i, cfg) for i in range(cfg["n_layers"])]
    head = synth.make_head(seed, cfg)
    om = po.OracleModel(cfg, layers, head, 2304, kv_fp16=kv_fp16)
    dec = Decoder(cfg, layers, head, max_seq=2304, kv_fp16=kv_fp16, use_graph=True)
    for i in range(cfg["n_layers"]):
        k, v = synth.make_kv_prefill(seed, i, cfg, 2048)
        dec.set_kv(i, k, v)
        om.set_kv(i, k, v)
    dec.set_past_len(2048)
    feed = [int(t) for t in golden_cfg4["forced_feed"]]
    assert len(set(feed)) == 128
    idx = golden_cfg4["forced_sample_index"]
    errs, gerrs, worst_resid, argmax_checked = [], [], 0.0, 0
    for st, t in enumerate(feed):
        if st in (0, 64, 127):
            to, tr_o = om.step_trace(t)
            tg, tr_g = dec.step_trace(t)
            for li in range(cfg["n_layers"]):
                for br in (0, 1):
                    ro = tr_o[li, br].astype(np.float64)
                    e = np.abs(tr_g[li, br] - ro).max() / np.sqrt((ro ** 2).mean())
                    worst_resid = max(worst_resid, e)
                    assert e <= RESID_TOL, (st, li, br, e)
        else:
            to = om.step(t)
            tg = dec.step(t)
        lg = dec.logits()
        sd = float(om.logits.std())
        errs.append(float(np.abs(lg - om.logits).max()) / sd)
        srt = np.sort(om.logits)
        stable = errs[-1] <= LOGIT_TOL
        if stable and (srt[-1] - srt[-2]) / sd > 2 * LOGIT_TOL:
            assert tg == to, (st, tg, to, errs[-1])
            argmax_checked += 1
        if not kv_fp16:   # the compiled reference's run of the same feed
            gsd = float(golden_cfg4["forced_std"][st])
            gerrs.append(float(np.abs(lg[idx] - golden_cfg4["forced_samples"][st]).max()) / gsd)
            if stable and gerrs[-1] <= LOGIT_TOL:
                if float(golden_cfg4["forced_margins"][st]) / gsd > 2 * LOGIT_TOL:
                    assert tg == int(golden_cfg4["forced_tokens"][st]), (st, tg)
                if st in (0, 1, 63, 127):
                    assert np.abs(lg[:256] - golden_cfg4["forced_logits256_step%d" % st]).max() / gsd <= LOGIT_TOL, st
        pos = 2048 + st   # both caches go on from the oracle's appended rows
        for li in range(cfg["n_layers"]):
            dec.k_cache[li][pos].copy_(torch.from_numpy(om.k_cache[li][pos]))
            dec.v_cache[li][pos].copy_(torch.from_numpy(om.v_cache[li][pos]))
        if st % 32 == 0:
            print("forced step %3d fed %6d argmax %6d  err/std vs oracle %.2e  (%.0fs)" % (st, t, tg, errs[-1], time.time() - t0), flush=True)
    unstable = [(i, round(e, 4)) for i, e in enumerate(errs) if e > LOGIT_TOL]
    print("kv_fp16=%s: per-step logit err/std vs oracle: median %.2e, unstable steps %s; worst residual %.2e; argmax compared on %d steps"
          % (kv_fp16, float(np.median(errs)), unstable, worst_resid, argmax_checked), flush=True)
    assert len(unstable) <= MAX_UNSTABLE and float(np.median(errs)) <= MEDIAN_TOL
    assert argmax_checked >= 110
    if gerrs:
        g_unstable = [(i, round(e, 4)) for i, e in enumerate(gerrs) if e > LOGIT_TOL]
        print("   vs the compiled reference's golden: median %.2e, unstable steps %s" % (float(np.median(gerrs)), g_unstable), flush=True)
        assert len(g_unstable) <= MAX_UNSTABLE and float(np.median(gerrs)) <= MEDIAN_TOL
    dec.close()


@pytest.mark.parametrize("kv_fp16", [True, False])
def test_cfg4_shape_centered_weights_teacher_forced(dev, po, seeds, kv_fp16):
    """A token-sensitive full-size model.  The benchmark's Q4_K blocks (independent scales and mins) give every weight a large
    positive mean, which makes the cfg4 network nearly rank one: two argmax ids whatever is fed, logits that move by ~0.06 of
    their spread from step to step.  With the same seeds but centred blocks (synth.make_layer_centered) the logits move by 2-8
    spreads per fed token and the argmax follows the input - and, with no rank-one term to inflate the spread, the noise of the
    int8 activation rounding shows at its true size: ~0.11 of the spread between ANY two fp32 evaluations of the step (measured:
    GPU against oracle, oracle with fp16 cache rows against oracle with fp32 ones).  Bars are therefore 0.25 of the spread for
    the logits and equal argmax where the top-2 margin exceeds 0.5 - 4 % of the token-to-token signal, where the bar of the
    rank-one model (1e-2 of a spread that moves by 0.06) is 16 %.  kv_fp16: against the oracle beside it; fp32 cache: also
    against the compiled reference's run of the same feed (golden_cfg4_centered.npz)."""
    import os
    from conftest import GOLDEN_DIR
    from prometorch_amd.decode import Decoder
    TOL, MARGIN = 0.25, 0.5
    path = os.path.join(GOLDEN_DIR, "golden_cfg4_centered.npz")
    if not os.path.exists(path):
        pytest.skip("golden_cfg4_centered.npz not generated")
    g = np.load(path, allow_pickle=False)
    cfg = dict(synth.QWEN3_4B)
    seed = seeds["cfg4"]
    layers = [synth.make_layer_centered(seed, i, cfg) for i in range(cfg["n_layers"])]
    head = synth.make_head(seed, cfg)
    om = po.OracleModel(cfg, layers, head, 2304, kv_fp16=kv_fp16)
    dec = Decoder(cfg, layers, head, max_seq=2304, kv_fp16=kv_fp16, use_graph=True)
    for i in range(cfg["n_layers"]):
        k, v = synth.make_kv_prefill(seed, i, cfg, 2048)
        dec.set_kv(i, k, v)
        om.set_kv(i, k, v)
    dec.set_past_len(2048)
    feed = [int(t) for t in g["feed"]][:32]
    idx = g["sample_index"]
    errs, gerrs, moved, checked, ids, prev = [], [], [], 0, set(), None
    for st, t in enumerate(feed):
        to, tg = om.step(t), dec.step(t)
        lg = dec.logits()
        sd = float(om.logits.std())
        errs.append(float(np.abs(lg - om.logits).max()) / sd)
        srt = np.sort(om.logits)
        if (srt[-1] - srt[-2]) / sd > MARGIN:
            assert tg == to, (st, tg, to, errs[-1])
            checked += 1
        ids.add(to)
        if prev is not None:
            moved.append(float(np.abs(om.logits - prev).max()) / sd)
        prev = om.logits.copy()
        if not kv_fp16:
            gsd = float(g["std"][st])
            gerrs.append(float(np.abs(lg[idx] - g["samples"][st]).max()) / gsd)
            if float(g["margins"][st]) / gsd > MARGIN:
                assert tg == int(g["tokens"][st]), (st, tg)
    print("centred model, kv_fp16=%s: logit err/std max %.3f median %.3f; vs reference golden max %.3f; logits move by %.1f..%.1f "
          "spreads per token; %d distinct argmax ids, %d steps with a clear margin compared" %
          (kv_fp16, max(errs), float(np.median(errs)), max(gerrs) if gerrs else float("nan"), min(moved), max(moved), len(ids), checked), flush=True)
    assert max(errs) <= TOL, errs
    assert not gerrs or max(gerrs) <= TOL, gerrs
    assert min(moved) > 1.0 and len(ids) >= 16      # the model is token-sensitive: that is its point
    dec.close()


def test_capture_failure_falls_back_to_plain_launches(dev, po, seeds):
    """The eager continuation after a failed graph capture (the reference's fallback, gguf_model.h:2660-2665, :3100-3104).  The
    failure is forced on the host through ptm_decode_debug_fail_next_capture, before anything is recorded: no GPU error is
    provoked.  State 2, tokens and logits as the oracle's, no second capture attempt after set_past_len; the sampled step
    keeps its own state."""
    from prometorch_amd.decode import Decoder
    cfg = dict(synth.TINY)
    layers = [synth.make_layer(seeds["tiny"], i, cfg) for i in range(cfg["n_layers"])]
    head = synth.make_head(seeds["tiny"], cfg)
    kv = [synth.make_kv_prefill(seeds["tiny"], i, cfg, 19) for i in range(cfg["n_layers"])]
    om = po.OracleModel(cfg, layers, head, 64, kv_fp16=True)
    dec = Decoder(cfg, layers, head, max_seq=64, kv_fp16=True, use_graph=True)
    ref = Decoder(cfg, layers, head, max_seq=64, kv_fp16=True, use_graph=True)   # the same run on a captured graph
    for i, (k, v) in enumerate(kv):
        om.set_kv(i, k, v)
        dec.set_kv(i, k, v)
        ref.set_kv(i, k, v)
    dec.set_past_len(19)
    ref.set_past_len(19)
    state = dec.L.ptm_decode_graph_state
    assert state(dec.h, 0) == 0
    assert dec.L.ptm_decode_debug_fail_next_capture(dec.h) == 0
    to = tg = tr = 3
    errs = []
    for st in range(10):
        to, tg, tr = om.step(to), dec.step(tg), ref.step(tr)
        assert state(dec.h, 0) == 2, st                      # the very first step already attempted (and failed) the capture
        errs.append(np.abs(dec.logits() - om.logits).max() / om.logits.std())
        assert tg == to == tr, (st, errs[-1])
        assert np.array_equal(dec.logits(), ref.logits()), st    # plain launches and the replayed graph run the same kernels
    check_step_errors(errs)
    assert state(ref.h, 0) == 1
    # a rewind does not retry the capture (the seam is spent; a retry would succeed and report 1)
    dec.set_past_len(19)
    ref.set_past_len(19)
    assert dec.greedy(3, 6) == ref.greedy(3, 6)
    assert state(dec.h, 0) == 2
    # the sampled step has a graph of its own: it still captures
    assert state(dec.h, 1) == 0
    dec.sampling_begin(0.8, 40, 0.9)
    ref.sampling_begin(0.8, 40, 0.9)
    dec.set_past_len(19)
    ref.set_past_len(19)
    us = [0.11, 0.52, 0.93, 0.34]
    assert dec.sample(3, us) == ref.sample(3, us)
    assert state(dec.h, 1) == 1 and state(dec.h, 0) == 2
    # and falls back the same way when its capture fails
    d2 = Decoder(cfg, layers, head, max_seq=64, kv_fp16=True, use_graph=True)
    for i, (k, v) in enumerate(kv):
        d2.set_kv(i, k, v)
    d2.set_past_len(19)
    d2.sampling_begin(0.8, 40, 0.9)
    d2.L.ptm_decode_debug_fail_next_capture(d2.h)
    ref.set_past_len(19)
    ref.sampling_begin(0.8, 40, 0.9)
    assert d2.sample(3, us) == ref.sample(3, us)
    assert state(d2.h, 1) == 2 and state(d2.h, 0) == 0
    for d in (dec, ref, d2):
        d.close()


def test_tiny_decode_with_a_strong_ffn_branch_vs_oracle(dev, po, seeds):
    """The default synthetic gains keep the feed-forward branch small beside attention (synth.NORM_SCALE); here its norm gain is
    ten times larger, so that gate / up / down move the logits by several of their standard deviations (checked against the
    oracle below) and an error there could not pass the end-to-end comparison.  24 steps, layer by layer on the first."""
    from prometorch_amd.decode import Decoder
    cfg = dict(synth.TINY)
    ns = dict(synth.NORM_SCALE, ffn=1.0e-2)
    layers = [synth.make_layer(seeds["tiny"], i, cfg, norm_scale=ns) for i in range(cfg["n_layers"])]
    head = synth.make_head(seeds["tiny"], cfg)
    kv = [synth.make_kv_prefill(seeds["tiny"], i, cfg, 19) for i in range(cfg["n_layers"])]

    def oracle(ls):
        om = po.OracleModel(cfg, ls, head, 64, kv_fp16=True)
        for i, (k, v) in enumerate(kv):
            om.set_kv(i, k, v)
        return om

    om = oracle(layers)
    no_ffn = [dict(L, ffn_norm=np.zeros_like(L["ffn_norm"])) for L in layers]
    om0 = oracle(no_ffn)
    om0.step(3)
    dec = Decoder(cfg, layers, head, max_seq=64, kv_fp16=True, use_graph=True)
    for i, (k, v) in enumerate(kv):
        dec.set_kv(i, k, v)
    dec.set_past_len(19)
    to, tr_o = om.step_trace(3)
    tg, tr_g = dec.step_trace(3)
    assert np.abs(om.logits - om0.logits).max() / om.logits.std() > 3.0    # the branch matters: > 3 sigma of the logits
    assert tg == to
    for li in range(cfg["n_layers"]):
        for br in (0, 1):
            ro = tr_o[li, br].astype(np.float64)
            assert np.abs(tr_g[li, br] - ro).max() / np.sqrt((ro ** 2).mean()) < 1e-4, (li, br)
    errs = [np.abs(dec.logits() - om.logits).max() / om.logits.std()]
    for st in range(23):
        to = om.step(to)
        tg = dec.step(tg)
        errs.append(np.abs(dec.logits() - om.logits).max() / om.logits.std())
        assert tg == to, (st, errs[-1])
    check_step_errors(errs)
    dec.close()
